// Kernels of the pre-norm hybrid decoders (windowed attention with mixed heads + gated delta-rule layers + dense or
// routed feed-forwards, depth-averaged residual stream), gfx950, wave = 64 lanes.  Second translation unit of
// libmsgl_mix.so; C ABI in include/msgl_mix.h.
//
// Precision contract (as in seqmix.hip): the residual stream and its history, every norm, attention scores and weights,
// decays, step sizes, unit vectors, the recurrent state, router logits and expert weights are fp32 in registers and in
// memory; tensors that feed a matrix product are stored in the model dtype T (bf16 or fp32).  With T = float every kernel
// here is true 32-bit.
//
//   embed_norm_kernel        X_0[t] = rms(table[id[t]]) * w                                   (fp32)
//   prenorm_kernel           s = x + sum_p g[t,p] y[t,p];  optional depth average over the stored history;  h = rms(.) * w;
//                            ROUTE: logits of the normed row, top-`top` by logit, softmax over the chosen ones
//   poly_act_kernel          a N(z) + b N(z^2) + c N(z^3) + e,  N = divide a row by its root mean square
//   silu_mul_kernel          silu(gate) * up over rows [gate | up]
//   route_top_kernel         stand-alone router on given fp32 logits (long batches)
//   kv_store_kernel          k and the (blended) v of a token -> cache rows at out_loc
//   window_attn_kernel       sliding-window attention over the paged rows: raw scores of all heads, mixed by the H x H table,
//                            fp32 online softmax, per-head sigmoid output gate; one workgroup per query token
//   short_conv_kernel        causal per-channel convolution over time + SiLU, inputs before the portion from the request's
//                            conv state; q / k heads made unit vectors (q also * d^-1/2);  conv_state_kernel shifts the state
//   delta_rule_kernel        S <- decay S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q   per (request, head); a thread
//                            owns one value column of S in registers; scalar or per-key-channel decay; long portions as
//                            parallel chunks: per-chunk transition (L | P), delta_scan_kernel over a request's chunks, outputs
//   head_gated_norm_kernel   per-head rms over dv * w * (sigmoid | silu)(gate)
#include "mix_common.h"

namespace {

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// request of token t: the b with cu_q[b] <= t < cu_q[b + 1]
__device__ __forceinline__ int request_of(const int* __restrict__ cu_q, int batch, int t) {
  int lo = 0, hi = batch;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (cu_q[mid] <= t) lo = mid; else hi = mid;
  }
  return lo;
}

// ------------------------------------------------------------------------------------------------ embedding + norm
template <typename T>
__global__ __launch_bounds__(256) void embed_norm_kernel(float* __restrict__ x32, const T* __restrict__ table, const int* __restrict__ ids,
                                                         const T* __restrict__ w, float eps, int W) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float v = ld(row + i);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum256(ss, red) / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) x32[(size_t)t * W + i] = ld(row + i) * inv * ld(w + i);
}

// ------------------------------------------------------------------------------------------------ router on logits
// s[e * st]: one token's logits (bias already added).  The `top` largest win (ties: lowest index), weights = softmax over them.
__device__ __forceinline__ void select_top_logits(float* s, int st, int E, int top, int* __restrict__ ids, float* __restrict__ wts) {
  float first = 0.f, tot = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = 0;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      const float v = s[e * st];
      if (v > bv) {
        best = e;
        bv = v;
      }
    }
    if (k == 0) first = bv;
    ids[k] = best;
    const float p = expf(bv - first);
    wts[k] = p;
    tot += p;
    s[best * st] = -INFINITY;
  }
  for (int k = 0; k < top; ++k) wts[k] /= tot;
}

template <typename T>
__global__ __launch_bounds__(64) void route_top_kernel(int* __restrict__ ids, float* __restrict__ wts, const float* __restrict__ z,
                                                       const T* __restrict__ bias, int tokens, int E, int top, int TPB) {
  extern __shared__ float lds[];
  const int t = blockIdx.x * TPB + threadIdx.x;
  if (threadIdx.x >= TPB || t >= tokens) return;
  float* s = lds + threadIdx.x;
  for (int e = 0; e < E; ++e) s[e * TPB] = z[(size_t)t * E + e] + (bias ? ld(bias + e) : 0.f);
  select_top_logits(s, TPB, E, top, ids + (size_t)t * top, wts + (size_t)t * top);
}

// ------------------------------------------------------------------------------------------------ pre-norm, residual sum, depth average
// One workgroup per token row.  s = x + sum_p g[p] y[p] (fp32, p ascending) -> sum_out;  with n_mix > 0 the row that goes on is
// sum_{j < n_mix - 1} c[j] hist[j] + c[n_mix - 1] s  (hist: earlier rows of the stream, `hist_stride` floats apart) -> x_out;
// h = row * rsqrt(mean(row^2) + eps) * w in T.  ROUTE: the normed row (its copy in T) is routed in the same launch.
template <typename T, bool ROUTE>
__global__ __launch_bounds__(256) void prenorm_kernel(const float* __restrict__ x_in, const T* __restrict__ y, int parts,
                                                      const float* __restrict__ gate, float* __restrict__ sum_out,
                                                      const float* __restrict__ hist, int64_t hist_stride, const float* __restrict__ c,
                                                      int n_mix, float* __restrict__ x_out, const T* __restrict__ w, T* __restrict__ h_out,
                                                      float eps, int W, const T* __restrict__ router, const T* __restrict__ bias, int E,
                                                      int top, int* __restrict__ ids, float* __restrict__ wts) {
  extern __shared__ float srow[];  // W floats + 4 (+ E with ROUTE)
  float* red = srow + W;
  const int t = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float s = x_in[(size_t)t * W + i];
    for (int p = 0; p < parts; ++p) {
      const float yv = ld(y + ((size_t)t * parts + p) * W + i);
      s = gate ? fmaf(gate[(size_t)t * parts + p], yv, s) : s + yv;
    }
    if (sum_out) sum_out[(size_t)t * W + i] = s;
    if (n_mix > 0) {
      float m = 0.f;
      for (int j = 0; j < n_mix - 1; ++j) m = fmaf(c[j], hist[(size_t)j * hist_stride + (size_t)t * W + i], m);
      s = fmaf(c[n_mix - 1], s, m);
      if (x_out) x_out[(size_t)t * W + i] = s;
    }
    srow[i] = s;
    ss += s * s;
  }
  if (!w) return;
  const float inv = 1.0f / sqrtf(block_sum256(ss, red) / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float v = srow[i] * inv * ld(w + i);
    st(h_out + (size_t)t * W + i, v);
    if (ROUTE) {
      T rounded;
      st(&rounded, v);
      srow[i] = ld(&rounded);
    }
  }
  if (!ROUTE) return;
  float* sc = red + 4;
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // a wave takes experts wave, wave + 4, ...; up to kRouteAcc of them at once, so that one pass over the row keeps that many
  // independent weight loads in flight per lane (16-byte loads where the row allows; element order per expert fixed)
  constexpr int kRouteAcc = 8;
  const bool wide = (W & 7) == 0 && ((uintptr_t)router & 15u) == 0;
  for (int e0 = wave; e0 < E; e0 += 4 * kRouteAcc) {
    float acc[kRouteAcc];
#pragma unroll
    for (int a = 0; a < kRouteAcc; ++a) acc[a] = 0.f;
    if (wide) {
      for (int i = lane * 8; i < W; i += 512) {
        float hv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) hv[u] = srow[i + u];
#pragma unroll
        for (int a = 0; a < kRouteAcc; ++a) {
          const int e = e0 + 4 * a;
          if (e < E) {
            float wv[8];
            read8(router + (size_t)e * W + i, wv);
#pragma unroll
            for (int u = 0; u < 8; ++u) acc[a] = fmaf(hv[u], wv[u], acc[a]);
          }
        }
      }
    } else {
      for (int i = lane; i < W; i += 64) {
        const float hv = srow[i];
#pragma unroll
        for (int a = 0; a < kRouteAcc; ++a) {
          const int e = e0 + 4 * a;
          if (e < E) acc[a] = fmaf(hv, ld(router + (size_t)e * W + i), acc[a]);
        }
      }
    }
#pragma unroll
    for (int a = 0; a < kRouteAcc; ++a) {
      const int e = e0 + 4 * a;
      const float v = wave_sum(acc[a]);
      if (e < E && lane == 0) sc[e] = v + (bias ? ld(bias + e) : 0.f);
    }
  }
  __syncthreads();
  if (wave != 0) return;
  // the `top` largest logits by the 64 lanes of one wave (a lane owns experts lane, lane + 64, ...; ties: lowest index)
  float first = 0.f, tot = 0.f, mine = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int best = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = sc[e];
      if (v > bv) {
        bv = v;
        best = e;
      }
    }
#pragma unroll
    for (int o = 32; o >= 1; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(best, o, 64);
      if (ov > bv || (ov == bv && oi < best)) {
        bv = ov;
        best = oi;
      }
    }
    if (k == 0) first = bv;
    const float p = expf(bv - first);
    tot += p;
    if (lane == k % 64) mine = p;  // lane k keeps the k-th weight (top <= 64 per pass of this loop is all a model has)
    if (lane == 0) {
      ids[(size_t)t * top + k] = best;
      sc[best] = -INFINITY;
    }
    if (k % 64 == 63 || k == top - 1) {
      // flush the weights gathered so far (unnormalised; the division follows once the total is known)
      const int base = k - (k % 64);
      if (base + lane <= k) wts[(size_t)t * top + base + lane] = mine;
    }
  }
  for (int k = lane; k < top; k += 64) wts[(size_t)t * top + k] /= tot;
}

// ------------------------------------------------------------------------------------------------ activations
template <typename T>
__global__ __launch_bounds__(256) void poly_act_kernel(T* __restrict__ out, const T* __restrict__ z, int64_t ldz, const float* __restrict__ coef,
                                                       float eps, int N) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int i = threadIdx.x; i < N; i += 256) {
    const float v = ld(z + (size_t)t * ldz + i), v2 = v * v;
    s2 += v2;
    s4 += v2 * v2;
    s6 += v2 * v2 * v2;
  }
  const float n = (float)N;
  const float i1 = 1.0f / sqrtf(block_sum256(s2, red) / n + eps);
  const float i2 = 1.0f / sqrtf(block_sum256(s4, red) / n + eps);
  const float i3 = 1.0f / sqrtf(block_sum256(s6, red) / n + eps);
  const float a = coef[0] * i1, b = coef[1] * i2, c = coef[2] * i3, e = coef[3];
  for (int i = threadIdx.x; i < N; i += 256) {
    const float v = ld(z + (size_t)t * ldz + i);
    st(out + (size_t)t * N + i, a * v + b * (v * v) + c * (v * v * v) + e);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int64_t total, int N) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t r = i / N;
  const int col = (int)(i - r * N);
  const T* row = gu + r * 2 * N;
  st(out + i, siluf_(ld(row + col)) * ld(row + N + col));
}

// ------------------------------------------------------------------------------------------------ cache rows of the windowed attention
// k = src[t, k_off : k_off + nk] -> k_cache[out_loc[t]];  v = src[t, v_off : v_off + nv], blended with the first value-mixing
// layer's v of the same token when v_first is given: (1 - lam) v + lam v_first  (lam: one number in T on the device).
template <typename T>
__global__ __launch_bounds__(256) void kv_store_kernel(T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ out_loc,
                                                       const T* __restrict__ src, int64_t ld_src, int k_off, int v_off, int nk, int nv,
                                                       const T* __restrict__ v_first, int64_t ld_first, const T* __restrict__ lam) {
  const int t = blockIdx.x;
  const size_t slot = (size_t)out_loc[t];
  const T* row = src + (size_t)t * ld_src;
  for (int i = threadIdx.x; i < nk; i += 256) k_cache[slot * nk + i] = row[k_off + i];
  if (v_first) {
    const float l = ld(lam);
    for (int i = threadIdx.x; i < nv; i += 256)
      st(v_cache + slot * nv + i, (1.0f - l) * ld(row + v_off + i) + l * ld(v_first + (size_t)t * ld_first + i));
  } else {
    for (int i = threadIdx.x; i < nv; i += 256) v_cache[slot * nv + i] = row[v_off + i];
  }
}

// ------------------------------------------------------------------------------------------------ windowed attention with mixed heads
// One workgroup (256 threads) = QT consecutive query tokens of one request x all H heads (x one of `splits` ranges of the keys).
// Keys from the first query's window start to the last query's position, in tiles of 64:
//   raw[g][q][key] = q_g . k_{group(g)}[key]        thread = (key, every fourth head): a key row is loaded once for the QT queries
//   s[h][q][key]   = scale * sum_g talk[h][g] raw[g][q][key], masked per query (causal, window)
//   online softmax per (head, query) (a wave takes every fourth head, lane = key), p -> LDS
//   acc[q][h][e]  = acc * corr + sum_key p[h][q][key] v_{group(h)}[key][e]    thread = (head, 8 consecutive e): 16-byte value loads
// splits == 1: out[t, h, e] = acc / l * sigmoid(gate[t, h]) in T.  splits > 1: every range leaves (acc, m, l) in the workspace and
// window_merge_kernel joins them -- for steps with few query tokens (decode), where one workgroup per token leaves the chip empty.
constexpr int kAttnAcc = 16;  // H * dv <= 256 * kAttnAcc

template <typename T, int QT>
__global__ __launch_bounds__(256) void window_attn_kernel(T* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
                                                          const T* __restrict__ src, int64_t ld_src, int g_off,
                                                          const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                          const int* __restrict__ table, int64_t table_stride,
                                                          const int* __restrict__ req_rows, const int* __restrict__ seq_lens,
                                                          const int* __restrict__ cu_q, int batch, int total_q, int H, int G, int d, int dv,
                                                          int window, float scale, const float* __restrict__ talk, int splits) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* tk = lds;                       // H * H
  float* raw = tk + H * H;               // H * QT * 64
  float* pr = raw + H * QT * 64;         // H * QT * 64
  float* mrow = pr + H * QT * 64;        // H * QT
  float* lrow = mrow + H * QT;           // H * QT
  float* corr = lrow + H * QT;           // H * QT
  int* slots = reinterpret_cast<int*>(corr + H * QT);  // 64
  T* qs = reinterpret_cast<T*>(lds + ((H * H + 2 * H * QT * 64 + 3 * H * QT + 64 + 3) & ~3));  // QT * H * d, 16-byte aligned
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // which request and which of its query tiles
  int wg = blockIdx.x, b = 0, n_new = 0;
  for (; b < batch; ++b) {
    n_new = cu_q[b + 1] - cu_q[b];
    const int nt = (n_new + QT - 1) / QT;
    if (wg < nt) break;
    wg -= nt;
  }
  if (b == batch) return;
  const int q0 = wg * QT, nq = n_new - q0 < QT ? n_new - q0 : QT;
  const int t0 = cu_q[b] + q0, p0 = seq_lens[b] - n_new + q0;
  const int j_lo = window > 0 && p0 - window + 1 > 0 ? p0 - window + 1 : 0, j_hi = p0 + nq - 1;
  const int ntiles = (j_hi - j_lo) / 64 + 1, per = (ntiles + splits - 1) / splits;
  const int tile_lo = blockIdx.y * per, tile_hi = tile_lo + per < ntiles ? tile_lo + per : ntiles;
  const int* trow = table + (size_t)req_rows[b] * table_stride;
  const int Hd = H * d;
  for (int i = tid; i < nq * Hd; i += 256) qs[i] = src[(size_t)(t0 + i / Hd) * ld_src + i % Hd];
  for (int i = tid; i < H * H; i += 256) tk[i] = talk[i] * scale;
  for (int i = tid; i < H * QT; i += 256) {
    mrow[i] = -INFINITY;
    lrow[i] = 0.f;
  }
  const int rep = H / G, nk = G * d, nv = G * dv, no = H * dv;
  float acc[QT][kAttnAcc];
#pragma unroll
  for (int qi = 0; qi < QT; ++qi)
#pragma unroll
    for (int a = 0; a < kAttnAcc; ++a) acc[qi][a] = 0.f;
  const bool wide_k = (d & 7) == 0, wide_v = (dv & 7) == 0;
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int base = j_lo + tile * 64;
    __syncthreads();
    if (tid < 64) slots[tid] = base + tid <= j_hi ? trow[base + tid] : -1;
    __syncthreads();
    const int slot = slots[lane], pos = base + lane;
    for (int g = wave; g < H; g += 4) {
      float s[QT];
#pragma unroll
      for (int qi = 0; qi < QT; ++qi) s[qi] = 0.f;
      if (slot >= 0) {
        const T* kr = k_cache + (size_t)slot * nk + (size_t)(g / rep) * d;
        if (wide_k) {
          for (int i = 0; i < d; i += 8) {
            float kv[8];
            read8(kr + i, kv);
#pragma unroll
            for (int qi = 0; qi < QT; ++qi) {
              if (qi < nq) {
                float qv[8];
                read8(qs + qi * Hd + g * d + i, qv);
#pragma unroll
                for (int u = 0; u < 8; ++u) s[qi] = fmaf(qv[u], kv[u], s[qi]);
              }
            }
          }
        } else {
          for (int i = 0; i < d; ++i) {
            const float kv = ld(kr + i);
#pragma unroll
            for (int qi = 0; qi < QT; ++qi)
              if (qi < nq) s[qi] = fmaf(ld(qs + qi * Hd + g * d + i), kv, s[qi]);
          }
        }
      }
#pragma unroll
      for (int qi = 0; qi < QT; ++qi) raw[(g * QT + qi) * 64 + lane] = s[qi];
    }
    __syncthreads();
    for (int h = wave; h < H; h += 4) {
#pragma unroll
      for (int qi = 0; qi < QT; ++qi) {
        if (qi >= nq) break;
        float s = 0.f;
        for (int g = 0; g < H; ++g) s = fmaf(tk[h * H + g], raw[(g * QT + qi) * 64 + lane], s);
        const int pq = p0 + qi;
        const bool seen = slot >= 0 && pos <= pq && (window <= 0 || pq - pos < window);
        if (!seen) s = -INFINITY;
        const float m_old = mrow[h * QT + qi];
        const float m_new = fmaxf(m_old, wave_max(s));
        const float pv = seen ? expf(s - m_new) : 0.f;
        const float sum = wave_sum(pv);
        pr[(h * QT + qi) * 64 + lane] = pv;
        if (lane == 0) {
          const float cf = m_new == -INFINITY ? 1.f : expf(m_old - m_new);  // no key of this query so far: nothing to rescale
          corr[h * QT + qi] = cf;
          lrow[h * QT + qi] = lrow[h * QT + qi] * cf + sum;
          mrow[h * QT + qi] = m_new;
        }
      }
    }
    __syncthreads();
    const int keys = j_hi - base + 1 < 64 ? j_hi - base + 1 : 64;
    if (wide_v) {
      const int per_head = dv >> 3;
#pragma unroll
      for (int a = 0; a < kAttnAcc / 8; ++a) {
        const int c = tid + 256 * a;
        if (c < H * per_head) {
          const int h = c / per_head, e0 = (c - h * per_head) << 3;
          const T* vcol = v_cache + (size_t)(h / rep) * dv + e0;
#pragma unroll
          for (int qi = 0; qi < QT; ++qi) {
            const float cf = corr[h * QT + qi];
#pragma unroll
            for (int u = 0; u < 8; ++u) acc[qi][a * 8 + u] *= cf;
          }
          for (int key = 0; key < keys; ++key) {
            float vv[8];
            read8(vcol + (size_t)slots[key] * nv, vv);
#pragma unroll
            for (int qi = 0; qi < QT; ++qi) {
              const float p = pr[(h * QT + qi) * 64 + key];
#pragma unroll
              for (int u = 0; u < 8; ++u) acc[qi][a * 8 + u] = fmaf(p, vv[u], acc[qi][a * 8 + u]);
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int a = 0; a < kAttnAcc; ++a) {
        const int o = tid + 256 * a;
        if (o < no) {
          const int h = o / dv, e = o - h * dv;
          const T* vcol = v_cache + (size_t)(h / rep) * dv + e;
#pragma unroll
          for (int qi = 0; qi < QT; ++qi) acc[qi][a] *= corr[h * QT + qi];
          for (int key = 0; key < keys; ++key) {
            const float vv = ld(vcol + (size_t)slots[key] * nv);
#pragma unroll
            for (int qi = 0; qi < QT; ++qi) acc[qi][a] = fmaf(pr[(h * QT + qi) * 64 + key], vv, acc[qi][a]);
          }
        }
      }
    }
  }
  __syncthreads();
  // element o of a token's output row <-> (a, u) of this thread
  const int per_head = dv >> 3;
#pragma unroll
  for (int a = 0; a < kAttnAcc; ++a) {
    int o;
    if (wide_v) {
      const int c = tid + 256 * (a >> 3);
      o = c < H * per_head ? c * 8 + (a & 7) : no;
    } else {
      o = tid + 256 * a;
    }
    if (o >= no) continue;
    const int h = o / dv;
#pragma unroll
    for (int qi = 0; qi < QT; ++qi) {
      if (qi >= nq) break;
      const size_t t = (size_t)(t0 + qi);
      if (splits == 1)
        st(out + t * no + o, acc[qi][a] / lrow[h * QT + qi] * sigmoidf_(ld(src + t * ld_src + g_off + h)));
      else
        part_o[((size_t)blockIdx.y * total_q + t) * no + o] = acc[qi][a];
    }
  }
  if (splits > 1)
    for (int i = tid; i < H * nq; i += 256) {
      const int h = i / nq, qi = i - h * nq;
      float* ml = part_ml + (((size_t)blockIdx.y * total_q + t0 + qi) * H + h) * 2;
      ml[0] = mrow[h * QT + qi];
      ml[1] = lrow[h * QT + qi];
    }
}

// Joins the key ranges of window_attn_kernel: one workgroup per token.  The (m, l) pairs of all ranges and heads are folded once into
// per-range factors exp(m_s - M) / L in LDS; every output element is then a short sum of independent loads.
template <typename T>
__global__ __launch_bounds__(256) void window_merge_kernel(T* __restrict__ out, const float* __restrict__ part_o,
                                                           const float* __restrict__ part_ml, const T* __restrict__ src, int64_t ld_src,
                                                           int g_off, int total_q, int H, int dv, int splits) {
  extern __shared__ float fac[];  // [splits][H]
  const size_t t = blockIdx.x;
  const int no = H * dv;
  for (int h = threadIdx.x; h < H; h += 256) {
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, part_ml[(((size_t)s * total_q + t) * H + h) * 2]);
    float l = 0.f;
    for (int s = 0; s < splits; ++s) {
      const float* ml = part_ml + (((size_t)s * total_q + t) * H + h) * 2;
      const float f = ml[0] == -INFINITY ? 0.f : expf(ml[0] - m);
      fac[s * H + h] = f;
      l = fmaf(ml[1], f, l);
    }
    const float g = sigmoidf_(ld(src + t * ld_src + g_off + h)) / l;
    for (int s = 0; s < splits; ++s) fac[s * H + h] *= g;
  }
  __syncthreads();
  for (int o = threadIdx.x; o < no; o += 256) {
    const int h = o / dv;
    float v = 0.f;
    for (int s = 0; s < splits; ++s) v = fmaf(part_o[((size_t)s * total_q + t) * no + o], fac[s * H + h], v);
    st(out + t * no + o, v);
  }
}

// ------------------------------------------------------------------------------------------------ short convolution
// One workgroup per token.  y[c] = silu(bias[c] + sum_j taps[c][j] in[pos - (n - 1) + j][c]) (bias may be null); inputs of this portion come from `src`, earlier
// ones from the request's conv state (state[slot][s][c] = the input at position start - (n - 1) + s), positions < 0 are zero.
// The first `unit_heads` groups of d channels are made unit vectors (x / sqrt(sum x^2 + 1e-6)); the first `scaled_heads` of them
// are also multiplied by d^-1/2.
template <typename T>
__global__ __launch_bounds__(256) void short_conv_kernel(float* __restrict__ out, T* __restrict__ out_t, const T* __restrict__ src,
                                                         int64_t ld_src,
                                                         const T* __restrict__ taps, const T* __restrict__ bias,
                                                         const T* __restrict__ state, const int* __restrict__ cu_q,
                                                         const int* __restrict__ seq_lens, const int* __restrict__ slots, int batch, int C,
                                                         int n, int unit_heads, int scaled_heads, int d) {
  extern __shared__ float row[];  // C
  const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int b = request_of(cu_q, batch, t);
  const int local = t - cu_q[b];
  const int pos = seq_lens[b] - (cu_q[b + 1] - cu_q[b]) + local;
  const T* st_row = state + (size_t)slots[b] * (n - 1) * C;
  for (int c = tid; c < C; c += 256) {
    float s = bias ? ld(bias + c) : 0.f;
    for (int j = 0; j < n; ++j) {
      const int back = n - 1 - j;  // how many tokens before this one
      if (pos - back < 0) continue;
      const float x = local - back >= 0 ? ld(src + (size_t)(t - back) * ld_src + c)
                                        : ld(st_row + (size_t)(n - 1 + local - back) * C + c);
      s = fmaf(ld(taps + (size_t)c * n + j), x, s);
    }
    row[c] = siluf_(s);
  }
  __syncthreads();
  for (int h = wave; h < unit_heads; h += 4) {
    float ss = 0.f;
    for (int i = lane; i < d; i += 64) ss = fmaf(row[h * d + i], row[h * d + i], ss);
    ss = wave_sum(ss);
    const float f = (h < scaled_heads ? 1.0f / sqrtf((float)d) : 1.0f) / sqrtf(ss + 1e-6f);
    for (int i = lane; i < d; i += 64) row[h * d + i] *= f;
  }
  __syncthreads();
  if (out)
    for (int c = tid; c < C; c += 256) out[(size_t)t * C + c] = row[c];
  if (out_t)
    for (int c = tid; c < C; c += 256) st(out_t + (size_t)t * C + c, row[c]);
}

// After short_conv_kernel: the state of every request in the batch moves on to its last n - 1 inputs.  Thread = (request, channel).
template <typename T>
__global__ __launch_bounds__(256) void conv_state_kernel(T* __restrict__ state, const T* __restrict__ src, int64_t ld_src,
                                                         const int* __restrict__ cu_q, const int* __restrict__ slots, int C, int n) {
  const int b = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  if (c >= C) return;
  const int first = cu_q[b], n_new = cu_q[b + 1] - first;
  if (n_new <= 0) return;
  T* sr = state + (size_t)slots[b] * (n - 1) * C + c;
  constexpr int kMax = 16;
  T keep[kMax];
  for (int s = 0; s < n - 1 && s < kMax; ++s) keep[s] = sr[(size_t)s * C];
  for (int s = 0; s < n - 1; ++s) {
    const int li = n_new - (n - 1) + s;  // index within the portion of the input that lands in state row s
    sr[(size_t)s * C] = li >= 0 ? src[(size_t)(first + li) * ld_src + c] : keep[s + n_new];
  }
}

// ------------------------------------------------------------------------------------------------ gated delta rule
// Workgroup = (column block of 64, head, request or chunk); a thread owns column e of the head's state S [d, dv] (DP >= d
// registers, the tail zero).  Per token, with g the decay (one number per head, or one per key channel = row of S):
//   S <- g S;  u = beta (v_e - S^T k);  S <- S + k u;  o_e = S^T q
// computed as  dk = S_old . (g k), u = beta (v_e - dk), S = g S_old + k u, o_e = S . q  (two passes over the column).  q, k (fp32,
// unit vectors) come from qkv rows [q: G x d | k: G x d | v: H x dv]; beta = sigmoid(b_raw[t, h]);
// g = exp(rate[h] * softplus(a_raw[t, .] + dt_bias[.])) with rate = -exp(A_log) (fp32, from the host).  16 tokens (8 for the
// widest heads) are staged in LDS at a time: k, g k, g, q per key channel, the block's 64 values, beta.
//
// MODE 0  a request's whole portion from its state row (zero when the portion starts at position 0), state row written back.
// Long portions are cut into chunks that run in parallel.  The rule is linear in S: over a chunk S_end = P S_start + L with
// P [d, d] the product of the tokens' transitions and L [d, dv] the state the chunk builds from zero.
// MODE 1  a chunk's (L | P): the same recurrence over dv + d columns, values = (v | 0), start = (0 | identity), no outputs;
//         -> scratch[item][h][d][dv + d].  The last chunk of a request is skipped (nothing follows it).
//         delta_scan_kernel then walks a request's chunks: start[c + 1] = P_c start[c] + L_c.
// MODE 2  a chunk's outputs from its start state; the last chunk of a request writes the state row.
template <typename T, int DP, bool CHANNEL, int MODE>
__global__ __launch_bounds__(64) void delta_rule_kernel(float* __restrict__ out, const float* __restrict__ qkv, float* __restrict__ state,
                                                        const T* __restrict__ b_raw, int64_t ld_b, const T* __restrict__ a_raw,
                                                        int64_t ld_a, const float* __restrict__ rate, const float* __restrict__ dt_bias,
                                                        const int* __restrict__ cu_q, const int* __restrict__ seq_lens,
                                                        const int* __restrict__ slots, int H, int G, int d, int dv,
                                                        const int* __restrict__ items, const int* __restrict__ item_first,
                                                        float* __restrict__ scratch, float* __restrict__ start) {
  constexpr int kStage = DP > 128 ? 8 : 16;
  __shared__ __attribute__((aligned(16))) float sk[kStage][DP], sgk[kStage][DP], sq[kStage][DP], sg[kStage][DP];
  __shared__ float sv[kStage][64], sbeta[kStage], sdec[kStage];
  const int h = blockIdx.y, e = blockIdx.x * 64 + threadIdx.x, lane = threadIdx.x;
  int b, first, n_new;
  bool last_chunk = true;
  if (MODE == 0) {
    b = blockIdx.z;
    first = cu_q[b];
    n_new = cu_q[b + 1] - first;
  } else {
    const int it = blockIdx.z;
    b = items[3 * it];
    first = cu_q[b] + items[3 * it + 1];
    n_new = items[3 * it + 2] - items[3 * it + 1];
    last_chunk = it == item_first[b + 1] - 1;
    if (MODE == 1 && last_chunk) return;
  }
  if (n_new <= 0) return;
  const int C = 2 * G * d + H * dv, kvh = h / (H / G);
  const int cols = MODE == 1 ? dv + d : dv;
  const bool live = e < cols, value_col = e < dv;
  float S[DP];
  if (MODE == 0) {
    const bool fresh = seq_lens[b] == n_new;
    const float* Srow = state + ((size_t)slots[b] * H + h) * d * dv;
#pragma unroll
    for (int i = 0; i < DP; ++i) S[i] = (!fresh && live && i < d) ? Srow[(size_t)i * dv + e] : 0.f;
  } else if (MODE == 1) {
#pragma unroll
    for (int i = 0; i < DP; ++i) S[i] = (live && !value_col && i == e - dv) ? 1.f : 0.f;
  } else {
    const float* Srow = start + ((size_t)blockIdx.z * H + h) * d * dv;
#pragma unroll
    for (int i = 0; i < DP; ++i) S[i] = (live && i < d) ? Srow[(size_t)i * dv + e] : 0.f;
  }
  const float r = rate[h];
  for (int t0 = 0; t0 < n_new; t0 += kStage) {
    const int nt = n_new - t0 < kStage ? n_new - t0 : kStage;
    __syncthreads();
    if (lane < nt) {
      const size_t t = (size_t)(first + t0 + lane);
      sbeta[lane] = sigmoidf_(ld(b_raw + t * ld_b + h));
      if (!CHANNEL) sdec[lane] = expf(r * softplusf_(ld(a_raw + t * ld_a + h) + dt_bias[h]));
    }
    for (int idx = lane; idx < nt * 64; idx += 64) {
      const int tt = idx >> 6;
      sv[tt][lane] = (live && value_col) ? qkv[(size_t)(first + t0 + tt) * C + 2 * G * d + h * dv + e] : 0.f;
    }
    if (!CHANNEL) __syncthreads();
    for (int idx = lane; idx < nt * DP; idx += 64) {
      const int tt = idx / DP, i = idx - tt * DP;
      const size_t t = (size_t)(first + t0 + tt);
      float kv = 0.f, qv = 0.f, g = 1.f;
      if (i < d) {
        qv = qkv[t * C + kvh * d + i];
        kv = qkv[t * C + (G + kvh) * d + i];
        g = CHANNEL ? expf(r * softplusf_(ld(a_raw + t * ld_a + h * d + i) + dt_bias[h * d + i])) : sdec[tt];
      }
      sk[tt][i] = kv;
      sgk[tt][i] = g * kv;
      sq[tt][i] = qv;
      sg[tt][i] = g;
    }
    __syncthreads();
    if (d == DP) {
      // q and k of a token are the same for every lane: read straight from the fp32 rows through uniform addresses (the scalar
      // unit's loads), so that the LDS carries only what had to be computed (the per-channel decays) -- LDS reads bound this loop
      for (int tt = 0; tt < nt; ++tt) {
        const float* __restrict__ qp = qkv + (size_t)(first + t0 + tt) * C + kvh * DP;
        const float* __restrict__ kp = qkv + (size_t)(first + t0 + tt) * C + (G + kvh) * DP;
        float dk = 0.f;
        if (CHANNEL) {
#pragma unroll
          for (int i = 0; i < DP; ++i) dk = fmaf(S[i], sgk[tt][i], dk);
        } else {
#pragma unroll
          for (int i = 0; i < DP; ++i) dk = fmaf(S[i], kp[i], dk);
          dk *= sdec[tt];
        }
        const float u = sbeta[tt] * (sv[tt][lane] - dk);
        const float gs = sdec[tt];
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < DP; ++i) {
          S[i] = fmaf(kp[i], u, (CHANNEL ? sg[tt][i] : gs) * S[i]);
          if (MODE != 1) o = fmaf(S[i], qp[i], o);
        }
        if (MODE != 1 && live) out[(size_t)(first + t0 + tt) * (size_t)(H * dv) + h * dv + e] = o;
      }
      continue;
    }
    for (int tt = 0; tt < nt; ++tt) {
      float dk = 0.f;
#pragma unroll
      for (int i = 0; i < DP; ++i) dk = fmaf(S[i], sgk[tt][i], dk);
      const float u = sbeta[tt] * (sv[tt][lane] - dk);
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DP; ++i) {
        S[i] = fmaf(sk[tt][i], u, sg[tt][i] * S[i]);
        if (MODE != 1) o = fmaf(S[i], sq[tt][i], o);
      }
      if (MODE != 1 && live) out[(size_t)(first + t0 + tt) * (size_t)(H * dv) + h * dv + e] = o;
    }
  }
  if (!live) return;
  if (MODE == 1) {
    float* dst = scratch + ((size_t)blockIdx.z * H + h) * d * (size_t)(dv + d);
#pragma unroll
    for (int i = 0; i < DP; ++i)
      if (i < d) dst[(size_t)i * (dv + d) + e] = S[i];
  } else if (last_chunk) {
    float* Srow = state + ((size_t)slots[b] * H + h) * d * dv;
#pragma unroll
    for (int i = 0; i < DP; ++i)
      if (i < d) Srow[(size_t)i * dv + e] = S[i];
  }
}

// Walks the chunks of a request: start[first chunk] = the request's state (zero for a fresh one), start[c + 1] = P_c start[c] + L_c.
// Workgroup = (column block of 64, head, request), NW waves; a lane owns column e, the waves share the rows: wave w computes rows
// 16 w .. 16 w + 15 of every block of 16 NW rows from its own LDS tile of P_c.  The current start state sits in LDS (one column per
// lane), the new one is built in a second LDS buffer and written to start[c + 1] on the way; the buffers swap per chunk.
template <int DP>
struct ScanShape {
  static constexpr int NW = DP > 128 ? 2 : 4;   // waves
  static constexpr int PR = DP > 128 ? 8 : 16;  // rows of P per wave and block
  static constexpr size_t lds_bytes = (size_t)(2 * DP * 64 + NW * PR * DP) * sizeof(float);
};

template <int DP>
__global__ __launch_bounds__(ScanShape<DP>::NW * 64) void delta_scan_kernel(const float* __restrict__ state,
                                                                            const float* __restrict__ scratch, float* __restrict__ start,
                                                                            const int* __restrict__ cu_q, const int* __restrict__ seq_lens,
                                                                            const int* __restrict__ slots,
                                                                            const int* __restrict__ item_first, int H, int d, int dv) {
  constexpr int NW = ScanShape<DP>::NW, PR = ScanShape<DP>::PR;
  extern __shared__ __attribute__((aligned(16))) float scan_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* cur = scan_lds;                              // [DP][64]
  float* nxt = scan_lds + DP * 64;                    // [DP][64]
  float* P = scan_lds + 2 * DP * 64 + wave * PR * DP; // [PR][DP], this wave's
  const int b = blockIdx.z, h = blockIdx.y, e = blockIdx.x * 64 + lane;
  const int c0 = item_first[b], c1 = item_first[b + 1];
  if (c1 <= c0) return;
  const bool live = e < dv;
  const bool fresh = seq_lens[b] == cu_q[b + 1] - cu_q[b];
  const float* Srow = state + ((size_t)slots[b] * H + h) * d * dv;
  float* dst = start + ((size_t)c0 * H + h) * d * dv;
  for (int i = wave; i < DP; i += NW) {
    const float v = (!fresh && live && i < d) ? Srow[(size_t)i * dv + e] : 0.f;
    cur[i * 64 + lane] = v;
    nxt[i * 64 + lane] = 0.f;
    if (live && i < d) dst[(size_t)i * dv + e] = v;
  }
  for (int c = c0; c + 1 < c1; ++c) {
    const float* LP = scratch + ((size_t)c * H + h) * d * (size_t)(dv + d);
    dst = start + ((size_t)(c + 1) * H + h) * d * dv;
    for (int blk = 0; blk < d; blk += NW * PR) {
      const int i0 = blk + wave * PR;
      __syncthreads();  // the state of this chunk is complete (first block) / the wave's tile is free again
      for (int idx = lane; idx < PR * DP; idx += 64) {
        const int r = idx / DP, j = idx - r * DP;
        P[idx] = (i0 + r < d && j < d) ? LP[(size_t)(i0 + r) * (dv + d) + dv + j] : 0.f;
      }
      __syncthreads();
      float acc[PR];
#pragma unroll
      for (int r = 0; r < PR; ++r) acc[r] = (live && i0 + r < d) ? LP[(size_t)(i0 + r) * (dv + d) + e] : 0.f;
      for (int j = 0; j < DP; j += 4) {
        const float s0 = cur[j * 64 + lane], s1 = cur[(j + 1) * 64 + lane], s2 = cur[(j + 2) * 64 + lane], s3 = cur[(j + 3) * 64 + lane];
#pragma unroll
        for (int r = 0; r < PR; ++r) {
          const float4 p = *reinterpret_cast<const float4*>(P + r * DP + j);
          acc[r] = fmaf(p.x, s0, fmaf(p.y, s1, fmaf(p.z, s2, fmaf(p.w, s3, acc[r]))));
        }
      }
#pragma unroll
      for (int r = 0; r < PR; ++r) {
        if (i0 + r < d) {
          nxt[(i0 + r) * 64 + lane] = acc[r];
          if (live) dst[(size_t)(i0 + r) * dv + e] = acc[r];
        }
      }
    }
    float* t = cur;
    cur = nxt;
    nxt = t;
  }
}

// ------------------------------------------------------------------------------------------------ per-head gated norm
// out[t, h, e] = o / sqrt(mean_e(o[t, h]^2) + eps) * w[e] * act(gate[t, h, e]);  act = sigmoid (0) or SiLU (1).  A wave per head.
template <typename T>
__global__ __launch_bounds__(256) void head_gated_norm_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ g,
                                                              int64_t ld_g, const T* __restrict__ w, float eps, int H, int dv, int act) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int h = wave; h < H; h += 4) {
    const float* oh = o + ((size_t)t * H + h) * dv;
    float ss = 0.f;
    for (int i = lane; i < dv; i += 64) ss = fmaf(oh[i], oh[i], ss);
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
    for (int i = lane; i < dv; i += 64) {
      const float z = ld(g + (size_t)t * ld_g + h * dv + i);
      st(out + ((size_t)t * H + h) * dv + i, oh[i] * inv * ld(w + i) * (act ? siluf_(z) : sigmoidf_(z)));
    }
  }
}

}  // namespace

extern "C" {

int msgl_mix_embed_norm(float* x32, const void* table, const int* ids, const void* w, float eps, int tokens, int W, int dtype,
                        void* stream) {
  MIX_REQUIRE(x32 && table && ids && w && tokens >= 0 && W >= 1 && dtype_ok(dtype), "embed_norm: bad arguments");
  if (tokens == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(embed_norm_kernel<T>, dim3(tokens), dim3(256), 0, s, x32, cp<T>(table), ids, cp<T>(w), eps, W);)
  MIX_LAUNCHED("embed_norm");
  return MSGL_MIX_OK;
}

int msgl_mix_prenorm(const float* x_in, const void* y, int parts, const float* gate, float* sum_out, const float* hist,
                     int64_t hist_stride, const float* mix_w, int n_mix, float* x_out, const void* w, void* h_out, float eps, int rows,
                     int W, int dtype, const void* router, const void* bias, int E, int top, int* ids, float* wts, void* stream) {
  MIX_REQUIRE(x_in && rows >= 0 && W >= 1 && dtype_ok(dtype), "prenorm: bad arguments");
  MIX_REQUIRE((parts == 0) == (y == nullptr) && parts >= 0, "prenorm: parts = %d does not match y", parts);
  MIX_REQUIRE((w == nullptr) == (h_out == nullptr), "prenorm: a norm weight needs h_out and the reverse");
  MIX_REQUIRE(n_mix >= 0 && (n_mix == 0 || (mix_w && x_out && (n_mix == 1 || hist))), "prenorm: depth average without its rows");
  const bool route = router != nullptr;
  if (route) MIX_REQUIRE(w && ids && wts && E >= 1 && top >= 1 && top <= E, "prenorm: bad router arguments (E %d top %d)", E, top);
  if (rows == 0) return MSGL_MIX_OK;
  const size_t lds = (size_t)(W + 4 + (route ? E : 0)) * sizeof(float);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define PRE_LAUNCH(ROUTE)                                                                                                               \
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)prenorm_kernel<T, ROUTE>, lds) == 0, "prenorm: row of %d does not fit LDS", W); \
             hipLaunchKernelGGL((prenorm_kernel<T, ROUTE>), dim3(rows), dim3(256), lds, s, x_in, cp<T>(y), parts, gate, sum_out, hist,  \
                                hist_stride, mix_w, n_mix, x_out, cp<T>(w), mp<T>(h_out), eps, W, cp<T>(router), cp<T>(bias), E, top,   \
                                ids, wts);)
  if (route) {
    PRE_LAUNCH(true)
  } else {
    PRE_LAUNCH(false)
  }
#undef PRE_LAUNCH
  MIX_LAUNCHED("prenorm");
  return MSGL_MIX_OK;
}

int msgl_mix_poly_act(void* out, const void* z, int64_t ldz, const float* coef, float eps, int rows, int N, int dtype, void* stream) {
  MIX_REQUIRE(out && z && coef && rows >= 0 && N >= 1 && ldz >= N && dtype_ok(dtype), "poly_act: bad arguments");
  if (rows == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(poly_act_kernel<T>, dim3(rows), dim3(256), 0, s, mp<T>(out), cp<T>(z), ldz, coef, eps, N);)
  MIX_LAUNCHED("poly_act");
  return MSGL_MIX_OK;
}

int msgl_mix_silu_mul(void* out, const void* gate_up, int rows, int N, int dtype, void* stream) {
  MIX_REQUIRE(out && gate_up && rows >= 0 && N >= 1 && dtype_ok(dtype), "silu_mul: bad arguments");
  if (rows == 0) return MSGL_MIX_OK;
  const int64_t total = (int64_t)rows * N;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(silu_mul_kernel<T>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, mp<T>(out),
                                       cp<T>(gate_up), total, N);)
  MIX_LAUNCHED("silu_mul");
  return MSGL_MIX_OK;
}

int msgl_mix_route_top(int* ids, float* wts, const float* z, const void* bias, int tokens, int E, int top, int dtype, void* stream) {
  MIX_REQUIRE(ids && wts && z && dtype_ok(dtype) && E >= 1 && top >= 1 && top <= E, "route_top: bad arguments (E %d top %d)", E, top);
  if (tokens == 0) return MSGL_MIX_OK;
  int tpb = 64;
  while (tpb > 1 && (size_t)E * tpb * sizeof(float) > 64 * 1024) tpb >>= 1;
  const size_t lds = (size_t)E * tpb * sizeof(float);
  MIX_REQUIRE(lds <= 64 * 1024, "route_top: too many experts");
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(route_top_kernel<T>, dim3((tokens + tpb - 1) / tpb), dim3(64), lds, s, ids, wts, z, cp<T>(bias),
                                       tokens, E, top, tpb);)
  MIX_LAUNCHED("route_top");
  return MSGL_MIX_OK;
}

int msgl_mix_kv_store(void* k_cache, void* v_cache, const int* out_loc, const void* src, int64_t ld_src, int k_off, int v_off, int nk,
                      int nv, const void* v_first, int64_t ld_first, const void* lam, int tokens, int dtype, void* stream) {
  MIX_REQUIRE(k_cache && v_cache && out_loc && src && tokens >= 0 && nk >= 1 && nv >= 1 && k_off >= 0 && v_off >= 0 && dtype_ok(dtype),
              "kv_store: bad arguments");
  MIX_REQUIRE(ld_src >= k_off + nk && ld_src >= v_off + nv, "kv_store: columns past the source row");
  MIX_REQUIRE(!v_first || (lam && ld_first >= nv), "kv_store: value blending needs its factor and rows of at least nv");
  if (tokens == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(kv_store_kernel<T>, dim3(tokens), dim3(256), 0, s, mp<T>(k_cache), mp<T>(v_cache), out_loc,
                                       cp<T>(src), ld_src, k_off, v_off, nk, nv, cp<T>(v_first), ld_first, cp<T>(lam));)
  MIX_LAUNCHED("kv_store");
  return MSGL_MIX_OK;
}

int msgl_mix_window_attn_workspace_floats(int total_q, int H, int dv, int splits) {
  return splits > 1 ? splits * total_q * (H * dv + 2 * H) : 0;
}

int msgl_mix_window_attn(void* out, const void* src, int64_t ld_src, int g_off, const void* k_cache, const void* v_cache, const int* table,
                         int64_t table_stride, const int* req_rows, const int* seq_lens, const int* cu_q, int batch, int total_q, int H,
                         int G, int d, int dv, int window, float scale, const float* talk, int dtype, int splits, float* workspace,
                         void* stream) {
  MIX_REQUIRE(out && src && k_cache && v_cache && table && req_rows && seq_lens && cu_q && talk && dtype_ok(dtype),
              "window_attn: null pointer / dtype");
  MIX_REQUIRE(batch >= 0 && total_q >= 0 && H >= 1 && G >= 1 && H % G == 0 && d >= 1 && dv >= 1 && window >= 0,
              "window_attn: bad sizes H %d G %d d %d dv %d window %d", H, G, d, dv, window);
  MIX_REQUIRE(H * dv <= 256 * kAttnAcc, "window_attn: %d output elements per token (at most %d)", H * dv, 256 * kAttnAcc);
  MIX_REQUIRE(ld_src >= (int64_t)H * d && ld_src >= g_off + H && g_off >= 0, "window_attn: columns past the source row");
  MIX_REQUIRE(splits >= 1 && splits <= 64 && (splits == 1 || workspace), "window_attn: %d key ranges need a workspace", splits);
  if (total_q == 0 || batch == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t es = dtype == MSGL_MIX_BF16 ? 2 : 4;
  float* part_o = workspace;
  float* part_ml = workspace ? workspace + (size_t)splits * total_q * H * dv : nullptr;
  // query tokens per workgroup: 8 where portions are long and the tile fits half the LDS (two workgroups per CU), else 4, else 1
#define WA_LAUNCH(QT)                                                                                                                  \
  {                                                                                                                                    \
    const size_t lds = (size_t)(H * H + 2 * H * QT * 64 + 3 * H * QT + 64 + 3) * sizeof(float) + (size_t)QT * H * d * es;                  \
    const int tiles = total_q / QT + batch;                                                                                            \
    DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)window_attn_kernel<T, QT>, lds) == 0, "window_attn: %zu bytes of LDS", lds); \
               hipLaunchKernelGGL((window_attn_kernel<T, QT>), dim3(tiles, splits), dim3(256), lds, s, mp<T>(out), part_o, part_ml,     \
                                  cp<T>(src), ld_src, g_off, cp<T>(k_cache), cp<T>(v_cache), table, table_stride, req_rows, seq_lens,  \
                                  cu_q, batch, total_q, H, G, d, dv, window, scale, talk, splits);)                                     \
  }
  const auto lds_of = [&](int qt) { return (size_t)(H * H + 2 * H * qt * 64 + 3 * H * qt + 64 + 3) * 4 + (size_t)qt * H * d * es; };
  if (total_q >= 8 * batch && lds_of(8) <= 80 * 1024) {
    WA_LAUNCH(8)
  } else if (total_q >= 4 * batch && lds_of(4) <= 80 * 1024) {
    WA_LAUNCH(4)
  } else {
    WA_LAUNCH(1)
  }
#undef WA_LAUNCH
  MIX_LAUNCHED("window_attn");
  if (splits > 1) {
    DISPATCH_T(dtype, hipLaunchKernelGGL(window_merge_kernel<T>, dim3(total_q), dim3(256), (size_t)splits * H * sizeof(float), s, mp<T>(out),
                                         part_o, part_ml, cp<T>(src), ld_src, g_off, total_q, H, dv, splits);)
    MIX_LAUNCHED("window_attn (merge)");
  }
  return MSGL_MIX_OK;
}

int msgl_mix_short_conv(float* out, void* out_t, const void* src, int64_t ld_src, const void* taps, const void* bias, void* state, const int* cu_q,
                        const int* seq_lens, const int* slots, int batch, int total, int C, int n, int unit_heads, int scaled_heads, int d,
                        int dtype, void* stream) {
  MIX_REQUIRE((out || out_t) && src && taps && cu_q && seq_lens && slots && dtype_ok(dtype), "short_conv: null pointer / dtype");
  MIX_REQUIRE(batch >= 0 && total >= 0 && C >= 1 && n >= 1 && n <= 17 && ld_src >= C && (n == 1 || state),
              "short_conv: bad sizes C %d taps %d", C, n);
  MIX_REQUIRE(unit_heads >= 0 && scaled_heads >= 0 && scaled_heads <= unit_heads && d >= 1 && (int64_t)unit_heads * d <= C,
              "short_conv: unit-vector heads past the row");
  if (total == 0 || batch == 0) return MSGL_MIX_OK;
  const size_t lds = (size_t)C * sizeof(float);
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)short_conv_kernel<T>, lds) == 0, "short_conv: row of %d does not fit LDS", C);
             hipLaunchKernelGGL(short_conv_kernel<T>, dim3(total), dim3(256), lds, s, out, mp<T>(out_t), cp<T>(src), ld_src, cp<T>(taps), cp<T>(bias),
                                cp<T>(state), cu_q, seq_lens, slots, batch, C, n, unit_heads, scaled_heads, d);
             if (n > 1) hipLaunchKernelGGL(conv_state_kernel<T>, dim3((C + 255) / 256, batch), dim3(256), 0, s, mp<T>(state), cp<T>(src),
                                           ld_src, cu_q, slots, C, n);)
  MIX_LAUNCHED("short_conv");
  return MSGL_MIX_OK;
}

int msgl_mix_delta_rule(float* out, const float* qkv, float* state, const void* b_raw, int64_t ld_b, const void* a_raw, int64_t ld_a,
                        int per_channel, const float* rate, const float* dt_bias, const int* cu_q, const int* seq_lens, const int* slots,
                        int batch, int H, int G, int d, int dv, int dtype, int n_items, const int* items, const int* item_first,
                        float* scratch, void* stream) {
  MIX_REQUIRE(out && qkv && state && b_raw && a_raw && rate && dt_bias && cu_q && seq_lens && slots && dtype_ok(dtype),
              "delta_rule: null pointer / dtype");
  MIX_REQUIRE(batch >= 0 && H >= 1 && G >= 1 && H % G == 0 && d >= 1 && d <= 256 && dv >= 1, "delta_rule: bad sizes H %d G %d d %d dv %d", H,
              G, d, dv);
  MIX_REQUIRE(ld_b >= H && ld_a >= (per_channel ? H * d : H), "delta_rule: rows shorter than their heads");
  MIX_REQUIRE(n_items >= 0 && (n_items == 0 || (items && item_first && scratch)), "delta_rule: chunks without their lists / scratch");
  if (batch == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* start = scratch ? scratch + (size_t)n_items * H * d * (size_t)(dv + d) : nullptr;  // [n_items, H, d, dv] after (L | P)
#define DR_LAUNCH(DP, CH, MODE, GRID)                                                                                                  \
  DISPATCH_T(dtype, hipLaunchKernelGGL((delta_rule_kernel<T, DP, CH, MODE>), GRID, dim3(64), 0, s, out, qkv, state, cp<T>(b_raw), ld_b, \
                                       cp<T>(a_raw), ld_a, rate, dt_bias, cu_q, seq_lens, slots, H, G, d, dv, items, item_first,       \
                                       scratch, start);)
#define DR_RUN(DP, CH)                                                                                                         \
  if (n_items == 0) {                                                                                                          \
    DR_LAUNCH(DP, CH, 0, dim3((dv + 63) / 64, H, batch))                                                                       \
  } else {                                                                                                                     \
    DR_LAUNCH(DP, CH, 1, dim3((dv + d + 63) / 64, H, n_items))                                                                 \
    MIX_LAUNCHED("delta_rule (chunk transitions)");                                                                            \
    MIX_REQUIRE(ensure_lds((const void*)delta_scan_kernel<DP>, ScanShape<DP>::lds_bytes) == 0, "delta_rule: scan LDS");         \
    hipLaunchKernelGGL((delta_scan_kernel<DP>), dim3((dv + 63) / 64, H, batch), dim3(ScanShape<DP>::NW * 64),                  \
                       ScanShape<DP>::lds_bytes, s, state, scratch, start, cu_q, seq_lens, slots, item_first, H, d, dv);       \
    MIX_LAUNCHED("delta_rule (scan)");                                                                                         \
    DR_LAUNCH(DP, CH, 2, dim3((dv + 63) / 64, H, n_items))                                                                     \
  }
#define DR_CASE(DP)     \
  if (per_channel) {    \
    DR_RUN(DP, true)    \
  } else {              \
    DR_RUN(DP, false)   \
  }
  if (d <= 16) {
    DR_CASE(16)
  } else if (d <= 32) {
    DR_CASE(32)
  } else if (d <= 64) {
    DR_CASE(64)
  } else if (d <= 96) {
    DR_CASE(96)
  } else if (d <= 128) {
    DR_CASE(128)
  } else if (d <= 192) {
    DR_CASE(192)
  } else {
    DR_CASE(256)
  }
#undef DR_CASE
#undef DR_RUN
#undef DR_LAUNCH
  MIX_LAUNCHED("delta_rule");
  return MSGL_MIX_OK;
}

int msgl_mix_head_gated_norm(void* out, const float* o, const void* gate, int64_t ld_gate, const void* w, float eps, int rows, int H,
                             int dv, int gate_act, int dtype, void* stream) {
  MIX_REQUIRE(out && o && gate && w && rows >= 0 && H >= 1 && dv >= 1 && ld_gate >= (int64_t)H * dv && dtype_ok(dtype) &&
                  (gate_act == 0 || gate_act == 1),
              "head_gated_norm: bad arguments");
  if (rows == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(head_gated_norm_kernel<T>, dim3(rows), dim3(256), 0, s, mp<T>(out), o, cp<T>(gate), ld_gate,
                                       cp<T>(w), eps, H, dv, gate_act);)
  MIX_LAUNCHED("head_gated_norm");
  return MSGL_MIX_OK;
}

}  // extern "C"
