// Kernels of the hybrid sequence-mixing models (latent attention + linear-recurrence layers + routed experts),
// gfx950, wave = 64 lanes.  Built into libmsgl_mix.so; C ABI at the end of the file (include/msgl_mix.h).
//
// Precision contract: the residual stream, every norm, rotary angles, attention scores and weights, the recurrent
// state, router scores and expert weights are fp32 in registers and in memory; tensors that feed a matrix product
// are stored in the model dtype T (bf16 or fp32).  With T = float every kernel here is true 32-bit.
//
//   embed_rows_kernel        x32[t] = table[id[t]]  (+ the T copy the first projection reads)
//   postnorm_kernel          x32 <- rms(alpha * x32 + sum_p g[t,p] * y[t,p]) * (1 + w)   (+ T copy); also the final norm;
//                            ROUTE: router logits, softmax, group-limited top-k and weights of the row it just normed
//   latent_prep_kernel       latent row: rms-norm(c) | rotate(k_r) -> cache[out_loc];  rotate(q_r) -> q_abs tail
//   latent_attn_mfma_kernel  bf16 caches: one shared (c | k_r) key row for all heads through LDS, both products on the matrix
//                            cores, fp32 online softmax, output in latent space; key ranges + latent_attn_merge_kernel for decode
//   latent_attn_kernel       the same in plain fp32 (fp32 caches, shapes past the matrix-core instances)
//   lightning_kernel         S <- decay * S + k v^T, o = S^T q per (request, head), state rows indexed by slot; long portions
//                            as parallel chunks joined by lightning_scan_kernel
//   gated_norm_kernel        rms over the concatenated heads * w * sigmoid(g)
//   route_kernel             fp32 router on fp32 logits: softmax, bias-corrected group-limited top-k, normalised weights
//   moe_count / moe_place    (token, choice) pairs bucketed by expert -> segment offsets + permutation
//   gemm_nt_mfma_kernel      grouped / segmented / gathered C = act(A B^T) for 16-bit weights on the matrix cores: per-head
//                            latent products, expert layers, router logits of long batches
//   gemm_nt_kernel           the same in fp32 FMA: fp32 engines, and every shape the library refuses
#include "mix_common.h"

namespace {

// ------------------------------------------------------------------------------------------------ embedding
template <typename T>
__global__ __launch_bounds__(256) void embed_rows_kernel(float* __restrict__ x32, T* __restrict__ h, const T* __restrict__ table,
                                                         const int* __restrict__ ids, int W) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * W;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float v = ld(row + i);
    x32[(size_t)t * W + i] = v;
    st(h + (size_t)t * W + i, v);
  }
}

// ------------------------------------------------------------------------------------------------ post-norm
// One workgroup per token row.  s = alpha * x + sum_p g[p] * y[p] (fp32, p ascending), out = s * rsqrt(mean(s^2) + eps) * (1 + w).
// ROUTE: the row that was just normed is also the router's input (its copy in T): every wave takes every fourth expert's logit
// (fp32 dot over the row, wave reduction in a fixed order), then one thread runs the selection -- the feed-forward's choices
// leave the same launch that closes the mixer's residual sum.  Defined after select_experts.
template <typename T, bool ROUTE>
__global__ __launch_bounds__(256) void postnorm_kernel(const float* __restrict__ x_in, float* __restrict__ x_out, T* __restrict__ h_out,
                                                       const T* __restrict__ y, int parts, const float* __restrict__ gate,
                                                       const T* __restrict__ w, float alpha, float eps, int W, const T* __restrict__ router,
                                                       const T* __restrict__ bias, int E, int top, int G, int keep, int* __restrict__ ids,
                                                       float* __restrict__ wts);

// ------------------------------------------------------------------------------------------------ latent prep
// One workgroup per token.  proj row = [ q: H x (d + r) | (has_kv) latent R | shared rotated key part r ].
// cos_sin row p = [cos(p f_i) * amp, i < rd/2 | sin(p f_i) * amp]; the first rd entries of a rotated part turn, the rest pass.
// Entry i is paired with i + rd / 2, or, with `interleaved`, entries 2i and 2i + 1 form pair i.
template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const T* __restrict__ proj, int64_t ld_proj, float* __restrict__ q_abs,
                                                          T* __restrict__ cache, const int* __restrict__ out_loc,
                                                          const int* __restrict__ positions, const float* __restrict__ cos_sin,
                                                          const T* __restrict__ c_norm_w, float eps, int H, int d, int r, int rd, int R,
                                                          int has_kv, int interleaved) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * ld_proj;
  const float* cs = cos_sin + (size_t)positions[t] * rd;
  const int half = rd >> 1;
  const int dk = R + r;
  // rotated query parts -> fp32 tail of the absorbed query rows
  for (int i = threadIdx.x; i < H * r; i += 256) {
    const int hh = i / r, j = i - hh * r;
    const T* qr = row + (size_t)hh * (d + r) + d;
    float v = ld(qr + j);
    if (j < rd && interleaved) {
      const float c = cs[j >> 1], s = cs[half + (j >> 1)], other = ld(qr + (j ^ 1));
      v = (j & 1) ? v * c + other * s : v * c - other * s;
    } else if (j < rd) {
      const int pidx = j < half ? j : j - half;
      const float c = cs[pidx], s = cs[half + pidx];
      const float u0 = ld(qr + pidx), v0 = ld(qr + pidx + half);
      v = j < half ? u0 * c - v0 * s : v0 * c + u0 * s;
    }
    q_abs[((size_t)t * H + hh) * dk + R + j] = v;
  }
  if (!has_kv) return;
  const T* kv = row + (size_t)H * (d + r);
  T* dst = cache + (size_t)out_loc[t] * dk;
  float ss = 0.f;
  for (int i = threadIdx.x; i < R; i += 256) {
    const float v = ld(kv + i);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum256(ss, red) / (float)R + eps);
  for (int i = threadIdx.x; i < R; i += 256) st(dst + i, ld(kv + i) * inv * ld(c_norm_w + i));
  for (int j = threadIdx.x; j < r; j += 256) {
    float v = ld(kv + R + j);
    if (j < rd && interleaved) {
      const float c = cs[j >> 1], s = cs[half + (j >> 1)], other = ld(kv + R + (j ^ 1));
      v = (j & 1) ? v * c + other * s : v * c - other * s;
    } else if (j < rd) {
      const int pidx = j < half ? j : j - half;
      const float c = cs[pidx], s = cs[half + pidx];
      const float u0 = ld(kv + R + pidx), v0 = ld(kv + R + pidx + half);
      v = j < half ? u0 * c - v0 * s : v0 * c + u0 * s;
    }
    st(dst + R + j, v);
  }
}

// ------------------------------------------------------------------------------------------------ latent attention
// A sink is one more term exp(sink[h]) in a head's softmax denominator, with no key and no value.  With running maximum m
// over the keys and M = max(m, sink): out = f o / (f l + w), f = exp(m - M), w = exp(sink - M)  (no sink: f = 1, w = 0).
__device__ __forceinline__ float sink_factor(const float* __restrict__ sink, int head, float m) {
  return (sink && sink[head] > m) ? expf(m - sink[head]) : 1.f;
}
__device__ __forceinline__ float sink_weight(const float* __restrict__ sink, int head, float m) {
  return sink ? (sink[head] > m ? 1.f : expf(sink[head] - m)) : 0.f;
}

// Query rows are (token, head) pairs; all heads read the same key row (latent R | rotated r) and the same value row
// (the latent).  A workgroup = 16 query rows (QT tokens of one request x HB heads) x 16 lanes; keys in tiles of KT through
// LDS as fp32; online softmax per row in fp32; output = softmax-weighted latent, fp32.
constexpr int kAttnRows = 16;
constexpr int kAttnMaxC = 32;  // value columns per lane: dv <= 512

template <typename T>
__global__ __launch_bounds__(256) void latent_attn_kernel(float* __restrict__ out, const float* __restrict__ q_abs,
                                                          const T* __restrict__ cache, const int* __restrict__ table,
                                                          int64_t table_stride, const int* __restrict__ req_rows,
                                                          const int* __restrict__ seq_lens, const int* __restrict__ cu_q, int B,
                                                          int H, int dk, int dv, float scale, int QT, int HB, int KT,
                                                          const float* __restrict__ sink) {
  extern __shared__ float lds[];
  const int qs = dk + 1;
  float* sq = lds;                       // [16][dk + 1]
  float* sk = sq + kAttnRows * qs;       // [KT][dk + 1]
  float* sp = sk + KT * qs;              // [16][KT]
  __shared__ int s_req, s_tok0, s_cnt[256];
  find_group(cu_q, B, QT, s_cnt, &s_req, &s_tok0);
  const int b = s_req;
  if (b < 0) return;
  const int q_len = cu_q[b + 1] - cu_q[b];
  const int start = seq_lens[b] - q_len;  // position of the request's first new token
  const int h0 = blockIdx.y * HB;
  const int r = threadIdx.x >> 4, l = threadIdx.x & 15;
  const int tl = s_tok0 + r / HB, hh = h0 + r % HB;
  const bool valid = r < QT * HB && tl < q_len && hh < H;
  const int tok = cu_q[b] + (valid ? tl : s_tok0);
  const int head = valid ? hh : h0;
  const int limit = start + (valid ? tl : s_tok0);  // last visible key
  const int last_tok = min(s_tok0 + QT, q_len) - 1;
  const int n_keys = start + last_tok + 1;
  for (int i = l; i < dk; i += 16) sq[r * qs + i] = q_abs[((size_t)tok * H + head) * dk + i];
  const int* trow = table + (size_t)req_rows[b] * table_stride;
  float m = -INFINITY, lsum = 0.f;
  float o[kAttnMaxC];
#pragma unroll
  for (int i = 0; i < kAttnMaxC; ++i) o[i] = 0.f;
  for (int j0 = 0; j0 < n_keys; j0 += KT) {
    __syncthreads();
    const int nk = min(KT, n_keys - j0);
    for (int e = threadIdx.x; e < nk * dk; e += 256) {
      const int j = e / dk, i = e - j * dk;
      sk[j * qs + i] = ld(cache + (size_t)trow[j0 + j] * dk + i);
    }
    __syncthreads();
    float tile_max = -INFINITY;
    for (int j = l; j < KT; j += 16) {
      float s = -INFINITY;
      if (j < nk && j0 + j <= limit) {
        float acc = 0.f;
        const float* qp = sq + r * qs;
        const float* kp = sk + j * qs;
        for (int i = 0; i < dk; ++i) acc = fmaf(qp[i], kp[i], acc);
        s = acc * scale;
      }
      sp[r * KT + j] = s;
      tile_max = fmaxf(tile_max, s);
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) tile_max = fmaxf(tile_max, __shfl_xor(tile_max, off, 64));
    const float m_new = fmaxf(m, tile_max);
    float corr = 1.f, psum = 0.f;
    if (m_new > -INFINITY) {
      corr = expf(m - m_new);
      for (int j = l; j < KT; j += 16) {
        const float p = expf(sp[r * KT + j] - m_new);
        sp[r * KT + j] = p;
        psum += p;
      }
    } else {
      for (int j = l; j < KT; j += 16) sp[r * KT + j] = 0.f;
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) psum += __shfl_xor(psum, off, 64);
    lsum = lsum * corr + psum;
    m = m_new;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kAttnMaxC; ++i) {
      const int c = l + 16 * i;
      if (c < dv) {
        float acc = o[i] * corr;
        for (int j = 0; j < nk; ++j) acc = fmaf(sp[r * KT + j], sk[j * qs + c], acc);
        o[i] = acc;
      }
    }
  }
  if (!valid) return;
  const float inv = sink_factor(sink, head, m) / (sink_factor(sink, head, m) * lsum + sink_weight(sink, head, m));
#pragma unroll
  for (int i = 0; i < kAttnMaxC; ++i) {
    const int c = l + 16 * i;
    if (c < dv) out[((size_t)tok * H + head) * dv + c] = o[i] * inv;
  }
}

// ------------------------------------------------------------------------------------------------ lightning recurrence
// Workgroup = one (head, request, block of CB state columns): columns of the d x dv state never mix (o[v] = sum_r S[r][v] q[r]),
// so they spread over workgroups freely.  Thread (column v, slice s) keeps rows s, s + NS, ... of column v in registers.
// Tokens go through in batches of kLtTok: q, k, v rows staged in LDS (SiLU applied in fp32), every thread walks the batch
// sequentially (S <- decay S + k v^T, partial o = sum over its rows of S q), the NS partials of a column are added in slice
// order.  A request that starts at position 0 starts from a zero state; the state row is the request's slot.  The arithmetic
// of a token does not depend on where a portion starts or ends: cutting a prompt anywhere gives the same bits.
constexpr int kLtTok = 16;
constexpr int kLtMaxRows = 64;
constexpr int kLtMaxCols = 64;

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }

// R = state rows per thread (compile time): thread (column v, slice s) owns rows s R .. s R + R - 1; q and k rows are padded
// with zeros to NS * R in LDS, so rows past d stay zero without a branch and a thread's q / k come as 16-byte LDS reads.
template <typename T, int R>
__global__ __launch_bounds__(256) void lightning_kernel(float* __restrict__ out, const T* __restrict__ qkv, int64_t ld_qkv,
                                                        float* __restrict__ state, const float* __restrict__ decay,
                                                        const int* __restrict__ cu_q, const int* __restrict__ seq_lens,
                                                        const int* __restrict__ slots, int H, int d, int dv, int CB, int NS,
                                                        const int* __restrict__ items, float* __restrict__ scratch, int mode) {
  // mode 0: one workgroup row per request, state row in and out.  With `items` (request, first token, end token of a chunk of a
  // long portion; offsets from the request's first new token): mode 1 = the chunk's own contribution to the state from zero
  // -> scratch[item], no outputs; mode 2 = outputs of the chunk from the state before it (scratch[item], written by the scan).
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int dp = NS * R;              // padded key size
  float* sq = lds;                    // [kLtTok][dp]
  float* skk = sq + kLtTok * dp;      // [kLtTok][dp]
  float* sv = skk + kLtTok * dp;      // [kLtTok][CB]
  float* part = sv + kLtTok * CB;     // [kLtTok][NS][CB]
  const int hh = blockIdx.x, v0 = blockIdx.z * CB;
  const int b = mode ? items[3 * blockIdx.y] : blockIdx.y;
  int t0 = cu_q[b], n = cu_q[b + 1] - t0;
  if (n <= 0) return;
  bool fresh = seq_lens[b] - n == 0;
  float* S = state + ((size_t)slots[b] * H + hh) * d * dv;
  if (mode) {
    t0 += items[3 * blockIdx.y + 1];
    n = items[3 * blockIdx.y + 2] - items[3 * blockIdx.y + 1];
    fresh = mode == 1;
    S = scratch + ((size_t)blockIdx.y * H + hh) * d * dv;
  }
  const int vl = threadIdx.x % CB, s = threadIdx.x / CB;
  const int v = v0 + vl;
  const int nc = min(CB, dv - v0);  // columns of this block
  const bool active = s < NS && v < dv;
  const float dec = decay[hh];
  float reg[R];
#pragma unroll
  for (int i = 0; i < R; ++i) {
    const int row = s * R + i;
    reg[i] = (active && row < d && !fresh) ? S[(size_t)row * dv + v] : 0.f;
  }
  const int64_t qo = (int64_t)hh * d, ko = (int64_t)H * d + (int64_t)hh * d, vo = 2 * (int64_t)H * d + (int64_t)hh * dv + v0;
  for (int c0 = 0; c0 < n; c0 += kLtTok) {
    const int nt = min(kLtTok, n - c0);
    __syncthreads();
    for (int e = threadIdx.x; e < nt * dp; e += 256) {
      const int tt = e / dp, i = e - tt * dp;
      const T* row = qkv + (size_t)(t0 + c0 + tt) * ld_qkv;
      if (mode != 1) sq[e] = i < d ? silu_f(ld(row + qo + i)) : 0.f;
      skk[e] = i < d ? silu_f(ld(row + ko + i)) : 0.f;
    }
    for (int e = threadIdx.x; e < nt * nc; e += 256) {
      const int tt = e / nc, i = e - tt * nc;
      sv[tt * CB + i] = silu_f(ld(qkv + (size_t)(t0 + c0 + tt) * ld_qkv + vo + i));
    }
    __syncthreads();
    if (active && mode == 1) {
      for (int tt = 0; tt < nt; ++tt) {
        const float vv = sv[tt * CB + vl];
        const float* kp = skk + tt * dp + s * R;
#pragma unroll
        for (int i = 0; i < R; ++i) reg[i] = fmaf(dec, reg[i], kp[i] * vv);
      }
    } else if (active) {
      for (int tt = 0; tt < nt; ++tt) {
        const float vv = sv[tt * CB + vl];
        const float* kp = skk + tt * dp + s * R;
        const float* qp = sq + tt * dp + s * R;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
          reg[i] = fmaf(dec, reg[i], kp[i] * vv);
          acc = fmaf(reg[i], qp[i], acc);
        }
        part[(tt * NS + s) * CB + vl] = acc;
      }
    }
    if (mode == 1) continue;
    __syncthreads();
    for (int e = threadIdx.x; e < nt * nc; e += 256) {
      const int tt = e / nc, i = e - tt * nc;
      float acc = 0.f;
      for (int k = 0; k < NS; ++k) acc += part[(tt * NS + k) * CB + i];
      out[(size_t)(t0 + c0 + tt) * ((size_t)H * dv) + (size_t)hh * dv + v0 + i] = acc;
    }
  }
  if (active && mode != 2) {
#pragma unroll
    for (int i = 0; i < R; ++i) {
      const int row = s * R + i;
      if (row < d) S[(size_t)row * dv + v] = reg[i];
    }
  }
}

// Between the two chunk passes: per state element, walk a request's chunks in order.  scratch[item] holds the chunk's own
// contribution U on entry and the state BEFORE the chunk on exit; S <- decay^len S + U; the state row gets the last S.
__global__ __launch_bounds__(256) void lightning_scan_kernel(float* __restrict__ state, float* __restrict__ scratch,
                                                             const float* __restrict__ decay, const int* __restrict__ cu_q,
                                                             const int* __restrict__ seq_lens, const int* __restrict__ slots,
                                                             const int* __restrict__ items, const int* __restrict__ item_first, int H,
                                                             int dd) {
  const int hh = blockIdx.x, b = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  const int i0 = item_first[b], i1 = item_first[b + 1];
  if (e >= dd || i0 >= i1) return;
  const int n = cu_q[b + 1] - cu_q[b];
  float* S = state + ((size_t)slots[b] * H + hh) * dd + e;
  float cur = (seq_lens[b] - n == 0) ? 0.f : *S;
  const float lg = logf(decay[hh]);
  for (int i = i0; i < i1; ++i) {
    float* u = scratch + ((size_t)i * H + hh) * dd + e;
    const float add = *u;
    *u = cur;
    cur = fmaf(expf((float)(items[3 * i + 2] - items[3 * i + 1]) * lg), cur, add);
  }
  *S = cur;
}

// ------------------------------------------------------------------------------------------------ gated norm
template <typename T>
__global__ __launch_bounds__(256) void gated_norm_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ g,
                                                         int64_t ld_g, const T* __restrict__ w, float eps, int N) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += 256) {
    const float v = o[(size_t)t * N + i];
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum256(ss, red) / (float)N + eps);
  for (int i = threadIdx.x; i < N; i += 256) {
    const float gate = 1.0f / (1.0f + expf(-ld(g + (size_t)t * ld_g + i)));
    st(out + (size_t)t * N + i, o[(size_t)t * N + i] * inv * ld(w + i) * gate);
  }
}

// ------------------------------------------------------------------------------------------------ router
// One thread per token over router logits z [T, E] that a product kernel wrote in fp32 (bf16 x bf16 products are exact in fp32,
// so the matrix cores' fp32 accumulation IS the 32-bit router on the token's 16-bit copy).  s = softmax(z); choice = s + bias;
// experts outside the `keep` best groups (a group's score = its largest choice) are out; the `top` largest choices win (ties:
// lowest index); weight = s / (sum of chosen s + 1e-20).  Scores live in LDS columns, one per thread.
// s[e * st] holds the router logits of one token on entry (st = column stride: one column per thread); c is scratch of the
// same shape, gs of G entries.  Writes the token's `top` expert ids and weights.
template <typename T>
__device__ __forceinline__ void select_experts(float* s, float* c, float* gs, int st, const T* __restrict__ bias, int E, int top, int G,
                                               int keep, int* __restrict__ ids, float* __restrict__ wts) {
  float mx = -INFINITY;
  for (int e = 0; e < E; ++e) mx = fmaxf(mx, s[e * st]);
  float sum = 0.f;
  for (int e = 0; e < E; ++e) {
    const float v = expf(s[e * st] - mx);
    s[e * st] = v;
    sum += v;
  }
  for (int e = 0; e < E; ++e) {
    const float v = s[e * st] / sum;
    s[e * st] = v;
    c[e * st] = v + (bias ? ld(bias + e) : 0.f);
  }
  const int per = E / G;
  if (keep < G) {
    // a group's score = its largest choice; it stays if fewer than `keep` groups beat it (ties: the lower index wins)
    for (int g = 0; g < G; ++g) {
      float best = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, c[e * st]);
      gs[g * st] = best;
    }
    for (int g = 0; g < G; ++g) {
      const float mine = gs[g * st];
      int better = 0;
      for (int o2 = 0; o2 < G; ++o2) better += (gs[o2 * st] > mine) || (gs[o2 * st] == mine && o2 < g);
      if (better >= keep)
        for (int e = g * per; e < (g + 1) * per; ++e) c[e * st] = -INFINITY;
    }
  }
  float tot = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      const float v = c[e * st];
      if (v > bv) {
        best = e;
        bv = v;
      }
    }
    if (best < 0) best = 0;  // unreachable: the host checks top <= keep * (E / G) and choice scores are finite
    ids[k] = best;
    const float sv = s[best * st];
    wts[k] = sv;
    tot += sv;
    c[best * st] = -INFINITY;
  }
  for (int k = 0; k < top; ++k) wts[k] /= (tot + 1e-20f);
}

// The same selection by the 64 lanes of one wave over one token (lane owns experts lane, lane + 64, ...): reductions by
// lane exchange in a fixed order, so the result does not depend on anything but the logits.  s, c: E entries of LDS each, gs: G + top.
__device__ __forceinline__ float wave_max_f(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
template <typename T>
__device__ __forceinline__ void select_experts_wave(float* s, float* c, float* gs, const T* __restrict__ bias, int E, int top, int G,
                                                    int keep, int* __restrict__ ids, float* __restrict__ wts) {
  const int lane = threadIdx.x & 63;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) mx = fmaxf(mx, s[e]);
  mx = wave_max_f(mx);
  float sum = 0.f;
  for (int e = lane; e < E; e += 64) {
    const float v = expf(s[e] - mx);
    s[e] = v;
    sum += v;
  }
  sum = wave_sum(sum);
  for (int e = lane; e < E; e += 64) {
    const float v = s[e] / sum;
    s[e] = v;
    c[e] = v + (bias ? ld(bias + e) : 0.f);
  }
  const int per = E / G;
  if (keep < G) {
    for (int g = lane; g < G; g += 64) {
      float best = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) best = fmaxf(best, c[e]);
      gs[g] = best;
    }
    for (int g = lane; g < G; g += 64) {
      const float mine = gs[g];
      int better = 0;
      for (int o2 = 0; o2 < G; ++o2) better += (gs[o2] > mine) || (gs[o2] == mine && o2 < g);
      if (better >= keep)
        for (int e = g * per; e < (g + 1) * per; ++e) c[e] = -INFINITY;
    }
  }
  float tot = 0.f;
  for (int k = 0; k < top; ++k) {
    float bv = -INFINITY;
    int best = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = c[e];
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
    if (best == 0x7fffffff) best = 0;  // unreachable: the host checks top <= keep * (E / G) and choice scores are finite
    const float sv = s[best];
    tot += sv;
    if (lane == 0) {
      ids[k] = best;
      gs[G + k] = sv;  // the chosen scores wait in LDS (in order within the wave) for the sum
      c[best] = -INFINITY;
    }
  }
  const float inv = 1.0f / (tot + 1e-20f);
  for (int k = lane; k < top; k += 64) wts[k] = gs[G + k] * inv;
}

template <typename T>
__global__ __launch_bounds__(64) void route_kernel(int* __restrict__ ids, float* __restrict__ wts, const float* __restrict__ z,
                                                   const T* __restrict__ bias, int tokens, int E, int top, int G, int keep, int TPB) {
  extern __shared__ float lds[];
  const int t = blockIdx.x * TPB + threadIdx.x;
  if (threadIdx.x >= TPB || t >= tokens) return;
  float* s = lds + threadIdx.x;             // s[e * TPB]
  float* c = lds + (size_t)E * TPB + threadIdx.x;
  const float* zr = z + (size_t)t * E;
#pragma unroll 8
  for (int e = 0; e < E; ++e) s[e * TPB] = zr[e];
  select_experts<T>(s, c, c + (size_t)E * TPB, TPB, bias, E, top, G, keep, ids + (size_t)t * top, wts + (size_t)t * top);
}

template <typename T, bool ROUTE>
__global__ __launch_bounds__(256) void postnorm_kernel(const float* __restrict__ x_in, float* __restrict__ x_out, T* __restrict__ h_out,
                                                       const T* __restrict__ y, int parts, const float* __restrict__ gate,
                                                       const T* __restrict__ w, float alpha, float eps, int W, const T* __restrict__ router,
                                                       const T* __restrict__ bias, int E, int top, int G, int keep, int* __restrict__ ids,
                                                       float* __restrict__ wts) {
  extern __shared__ float srow[];  // W floats + 4 (+ 2 E + G + top with ROUTE)
  float* red = srow + W;
  const int t = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float s = alpha * x_in[(size_t)t * W + i];
    for (int p = 0; p < parts; ++p) {
      const float yv = ld(y + ((size_t)t * parts + p) * W + i);
      s = gate ? fmaf(gate[(size_t)t * parts + p], yv, s) : s + yv;
    }
    srow[i] = s;
    ss += s * s;
  }
  const float tot = block_sum256(ss, red);
  const float inv = 1.0f / sqrtf(tot / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float v = srow[i] * inv * (1.0f + ld(w + i));
    if (x_out) x_out[(size_t)t * W + i] = v;
    if (h_out) st(h_out + (size_t)t * W + i, v);
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
  // a wave takes experts wave, wave + 4, ...; up to kRouteAcc of them at once, so that one pass over the row has that many
  // independent weight loads in flight per lane (element order per expert: lane-strided, then the wave reduction: fixed)
  constexpr int kRouteAcc = 8;
  const bool wide = (W & 7) == 0 && ((uintptr_t)router & 15u) == 0;
  for (int e0 = wave; e0 < E; e0 += 4 * kRouteAcc) {
    float acc[kRouteAcc];
#pragma unroll
    for (int a = 0; a < kRouteAcc; ++a) acc[a] = 0.f;
    if (wide) {  // eight consecutive weights per lane and load: 16 bytes (bf16) or 32 (fp32)
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
      if (e < E && lane == 0) sc[e] = v;
    }
  }
  __syncthreads();
  if (wave == 0) select_experts_wave<T>(sc, sc + E, sc + 2 * E, bias, E, top, G, keep, ids + (size_t)t * top, wts + (size_t)t * top);
}

// ------------------------------------------------------------------------------------------------ expert bucketing
// seg[e] .. seg[e + 1] = the sorted positions of expert e; perm[position] = flat (token * top + choice), in flat order inside a
// segment (stable: the layout does not depend on scheduling).  Two launches of one workgroup per expert, no atomics and nothing
// to clear: first every expert counts its entries, then it adds up the counts before it and places its entries by a running
// workgroup-wide rank.
__device__ __forceinline__ int block_rank256(bool flag, int* wsum, int& total) {
  const unsigned long long bal = __ballot(flag);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int before = __popcll(bal & ((1ull << lane) - 1ull));
  __syncthreads();
  if (lane == 0) wsum[wave] = __popcll(bal);
  __syncthreads();
  int off = 0;
  for (int w = 0; w < wave; ++w) off += wsum[w];
  total = wsum[0] + wsum[1] + wsum[2] + wsum[3];
  return off + before;
}

__global__ __launch_bounds__(256) void moe_count_kernel(int* __restrict__ counts, const int* __restrict__ ids, int n) {
  __shared__ int wsum[4];
  const int e = blockIdx.x;
  int cnt = 0;
  for (int i0 = 0; i0 < n; i0 += 256) {
    const int i = i0 + threadIdx.x;
    int tot;
    block_rank256(i < n && ids[i] == e, wsum, tot);
    cnt += tot;
  }
  if (threadIdx.x == 0) counts[e] = cnt;
}

__global__ __launch_bounds__(256) void moe_place_kernel(int* __restrict__ seg, int* __restrict__ perm, const int* __restrict__ counts,
                                                        const int* __restrict__ ids, int n, int E) {
  __shared__ int wsum[4];
  const int e = blockIdx.x;
  int base = 0;
  for (int k = 0; k < e; ++k) base += counts[k];
  if (threadIdx.x == 0) {
    seg[e] = base;
    if (e == E - 1) seg[E] = base + counts[e];
  }
  for (int i0 = 0; i0 < n; i0 += 256) {
    const int i = i0 + threadIdx.x;
    const bool mine = i < n && ids[i] == e;
    int tot;
    const int rank = block_rank256(mine, wsum, tot);
    if (mine) perm[base + rank] = i;
    base += tot;
  }
}

// ------------------------------------------------------------------------------------------------ grouped GEMM
// C[g][m][n] = act(sum_k A[g][m][k] * B[g][n][k]), fp32 accumulation in a fixed k order.
//   groups: A, B, C advance by a_gs, b_gs, c_gs elements per group (heads of one projection, experts);
//   seg != null: group g owns rows seg[g] .. seg[g + 1] of the row space (expert segments), M is an upper bound;
//   a_rows / c_rows != null: the row space is indirect (row m of A is a_rows[m] / a_div, row m of C is c_rows[m]).
// 64 x 64 tile, 256 threads, 4 x 4 outputs per thread, k in steps of 16 through LDS.
constexpr int kTile = 64, kStepK = 16;

template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_kernel(TC* __restrict__ C, const TA* __restrict__ A, const TB* __restrict__ Bm, int M, int N,
                                                      int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t a_gs, int64_t b_gs,
                                                      int64_t c_gs, const int* __restrict__ seg, const int* __restrict__ a_rows, int a_div,
                                                      const int* __restrict__ c_rows, int act) {
  __shared__ float sa[kStepK][kTile + 1];
  __shared__ float sb[kStepK][kTile + 1];
  const int g = blockIdx.z;
  int row0 = 0, rows = M;
  if (seg) {
    row0 = seg[g];
    rows = seg[g + 1] - row0;
  }
  const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;
  if (m0 >= rows) return;
  const TA* Ag = A + (seg ? 0 : g * a_gs);
  const TB* Bg = Bm + g * b_gs;
  TC* Cg = C + (seg ? 0 : g * c_gs);
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  // loader mapping: thread -> (row of the tile = tid / 4, four consecutive k = (tid % 4) * 4)
  const int lr = threadIdx.x >> 2, lk = (threadIdx.x & 3) * 4;
  int64_t a_off = -1;
  if (m0 + lr < rows) {
    const int m = row0 + m0 + lr;
    a_off = (int64_t)(a_rows ? a_rows[m] / a_div : m) * lda;
  }
  const int64_t b_off = n0 + lr < N ? (int64_t)(n0 + lr) * ldb : -1;
  for (int k0 = 0; k0 < K; k0 += kStepK) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int k = k0 + lk + u;
      sa[lk + u][lr] = (a_off >= 0 && k < K) ? ld(Ag + a_off + k) : 0.f;
      sb[lk + u][lr] = (b_off >= 0 && k < K) ? ld(Bg + b_off + k) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < kStepK; ++kk) {
      float av[4], bv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = sa[kk][ty + 16 * i];
#pragma unroll
      for (int j = 0; j < 4; ++j) bv[j] = sb[kk][tx + 16 * j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ml = m0 + ty + 16 * i;
    if (ml >= rows) continue;
    const int m = row0 + ml;
    const int64_t c_off = (int64_t)(c_rows ? c_rows[m] : m) * ldc;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (act == MSGL_MIX_ACT_RELU2) {
        v = fmaxf(v, 0.f);
        v = v * v;
      }
      st(Cg + c_off + n, v);
    }
  }
}

// ------------------------------------------------------------------------------------------------ grouped GEMM on the matrix cores
// The same contract as gemm_nt_kernel for 16-bit B (weights): A is rounded to bf16 on its way into LDS (it IS bf16 except for
// the fp32 latent that meets W_uv), products on v_mfma_f32_16x16x32_bf16 with fp32 accumulation.  128 x 128 tile, 4 waves of
// 64 x 64 (4 x 4 MFMA tiles each), k in steps of 64 (two MFMA k-blocks); the next step's global loads are issued before the
// current step's MFMAs.  LDS rows are 72 elements apart (144 B): the 16 lanes of a fragment read land on 16 different bank quads.  A wave
// whose rows lie past the end of a (short) expert segment skips its MFMAs, so a decode step pays for the weight stream only.
// An output element's k order is fixed, wherever its row sits in a segment: results do not depend on the batch around it.
constexpr int kMT = 128, kMK = 64, kMLd = 72;

template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_mfma_kernel(TC* __restrict__ C, const TA* __restrict__ A, const bf16_t* __restrict__ Bm, int M,
                                                           int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int64_t a_gs, int64_t b_gs,
                                                           int64_t c_gs, const int* __restrict__ seg, const int* __restrict__ a_rows,
                                                           int a_div, const int* __restrict__ c_rows, int act, int a_vec, int b_vec) {
  __shared__ __attribute__((aligned(16))) uint16_t sa[kMT * kMLd];
  __shared__ __attribute__((aligned(16))) uint16_t sb[kMT * kMLd];
  const int g = blockIdx.z;
  int row0 = 0, rows = M;
  if (seg) {
    row0 = seg[g];
    rows = seg[g + 1] - row0;
  }
  const int m0 = blockIdx.y * kMT, n0 = blockIdx.x * kMT;
  if (m0 >= rows) return;
  const TA* Ag = A + (seg ? 0 : g * a_gs);
  const bf16_t* Bg = Bm + g * b_gs;
  TC* Cg = C + (seg ? 0 : g * c_gs);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int lr = threadIdx.x >> 3, ks = (threadIdx.x & 7) * 8;  // loader: rows lr + 32 u, eight k from ks
  int64_t a_off[4], b_off[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int ml = m0 + lr + 32 * u, n = n0 + lr + 32 * u;
    a_off[u] = -1;
    if (ml < rows) {
      const int m = row0 + ml;
      a_off[u] = (int64_t)(a_rows ? a_rows[m] / a_div : m) * lda;
    }
    b_off[u] = n < N ? (int64_t)n * ldb : -1;
  }
  Q4 ra[4], rb[4];
  auto gload = [&](int k0) {
    const int k = k0 + ks, n = K - k;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      ra[u] = (a_off[u] >= 0 && n > 0) ? load8(Ag + a_off[u] + k, n, a_vec != 0) : Q4{0u, 0u, 0u, 0u};
      rb[u] = (b_off[u] >= 0 && n > 0) ? load8(Bg + b_off[u] + k, n, b_vec != 0) : Q4{0u, 0u, 0u, 0u};
    }
  };
  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int live_i = min(4, (rows - m0 - wm + 15) / 16);  // 16-row tiles of this wave that hold rows (<= 0: none)
  gload(0);
  for (int k0 = 0; k0 < K; k0 += kMK) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      *reinterpret_cast<Q4*>(&sa[(lr + 32 * u) * kMLd + ks]) = ra[u];
      *reinterpret_cast<Q4*>(&sb[(lr + 32 * u) * kMLd + ks]) = rb[u];
    }
    __syncthreads();
    if (k0 + kMK < K) gload(k0 + kMK);
    if (live_i > 0) {
#pragma unroll
      for (int kb = 0; kb < kMK / 32; ++kb) {
        bf16x8_t fb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
          fb[j] = *reinterpret_cast<const bf16x8_t*>(&sb[(wn + j * 16 + (lane & 15)) * kMLd + kb * 32 + (lane >> 4) * 8]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (i < live_i) {
            const bf16x8_t fa = *reinterpret_cast<const bf16x8_t*>(&sa[(wm + i * 16 + (lane & 15)) * kMLd + kb * 32 + (lane >> 4) * 8]);
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fb[j], fa, acc[i][j], 0, 0, 0);
          }
        }
      }
    }
  }
  // lane holds C[m = tile row (lane & 15)][n = 4 (lane >> 4) .. + 3] of every 16 x 16 tile
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ml = m0 + wm + i * 16 + (lane & 15);
    if (ml >= rows) continue;
    const int m = row0 + ml;
    const int64_t c_off = (int64_t)(c_rows ? c_rows[m] : m) * ldc;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int n = n0 + wn + j * 16 + 4 * (lane >> 4) + c;
        if (n >= N) continue;
        float v = acc[i][j][c];
        if (act == MSGL_MIX_ACT_RELU2) {
          v = fmaxf(v, 0.f);
          v = v * v;
        }
        st(Cg + c_off + n, v);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ latent attention on the matrix cores
// bf16 caches.  A workgroup = 64 query rows ((token, head) pairs of one request: QT tokens x HB heads) in 4 waves of 16 rows,
// one key range (split z of the keys its last token sees).  Keys come through LDS in tiles of 64 rows, row-major, 16-byte
// padded (fragment reads of 16 rows hit 16 different bank quads).  Per 16-key subtile and wave:
//   S^T[16 keys x 16 rows] = K . Q^T     KC x v_mfma_f32_16x16x32_bf16   (Q fragments live in registers, rounded to bf16 once)
//   a lane then holds ONE query row and FOUR keys: the B-operand layout of the second product, so P stays in its lane;
//   O^T[16 v x 16 rows] += V^T . P^T     VC x v_mfma_f32_16x16x16_bf16, V^T fragments read TRANSPOSED out of the same row-major
//   key tile (the latent is both key and value): in a 16-lane group, source lane s points at row 4 g + s / 4, columns
//   4 (s % 4) .. + 3 and ds_read_b64_tr_b16 hands lane j the four keys of column j.
// Softmax in fp32 per row, one step per 64-key tile: tile max across the four lane groups, running (m, l), O rescaled when
// a row's max moved.
// splits > 1 (decode: few rows, many keys): (m, l, O) partials per split, merged by latent_attn_merge_kernel.
constexpr int kAKT = 64;

template <int KC, int VC>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(float* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
                                                               const float* __restrict__ q_abs, const bf16_t* __restrict__ cache,
                                                               const int* __restrict__ table, int64_t table_stride,
                                                               const int* __restrict__ req_rows, const int* __restrict__ seq_lens,
                                                               const int* __restrict__ cu_q, int B, int H, int dk, int dv, float scale,
                                                               int QT, int HB, int splits, int vec, const float* __restrict__ sink) {
  constexpr int KS = KC * 32 + 8;
  extern __shared__ __attribute__((aligned(16))) uint16_t sk[];  // [kAKT][KS]
  __shared__ int s_req, s_tok0, s_cnt[256];
  find_group(cu_q, B, QT, s_cnt, &s_req, &s_tok0);
  const int b = s_req;
  if (b < 0) return;
  const int q_len = cu_q[b + 1] - cu_q[b];
  const int start = seq_lens[b] - q_len;
  const int h0 = blockIdx.y * HB, z = blockIdx.z;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int r = wave * 16 + lr;
  const int tl = s_tok0 + r / HB, hh = h0 + r % HB;
  const bool valid = r < QT * HB && tl < q_len && hh < H;
  const int tok = cu_q[b] + (valid ? tl : s_tok0);
  const int head = valid ? hh : h0;
  const int limit = valid ? start + tl : -1;
  const int last_tok = min(s_tok0 + QT, q_len) - 1;
  const int n_keys = start + last_tok + 1;
  const int per = ((n_keys + splits - 1) / splits + kAKT - 1) / kAKT * kAKT;
  const int k_begin = z * per, k_end = min(n_keys, k_begin + per);
  const bool wave_live = __builtin_amdgcn_ballot_w64(valid) != 0;
  // query fragments: row lr of this wave, k = 32 kc + 8 lg .. + 7
  bf16x8_t qf[KC];
  {
    const float* qrow = q_abs + ((size_t)tok * H + head) * dk;
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) {
      const int k = kc * 32 + lg * 8;
      Q4 v = (valid && k < dk) ? load8(qrow + k, dk - k, (dk & 3) == 0) : Q4{0u, 0u, 0u, 0u};
      qf[kc] = __builtin_bit_cast(bf16x8_t, v);
    }
  }
  f32x4_t o[VC];
#pragma unroll
  for (int vt = 0; vt < VC; ++vt) o[vt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;
  const int* trow = table + (size_t)req_rows[b] * table_stride;
  // the next tile's rows are requested before the current tile's products: their latency hides under the MFMAs
  constexpr int NCH = (kAKT * KC * 4 + 255) / 256;
  Q4 pre[NCH];
  // a tile's pool slots are read from the page table one tile ahead into LDS: the row loads never wait for a table load
  __shared__ int s_slot[2][kAKT];
  auto request = [&](int j0, int buf) {
#pragma unroll
    for (int u = 0; u < NCH; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (KC * 4), ch = e - key * (KC * 4);
      const int j = j0 + key, k = ch * 8;
      pre[u] = Q4{0u, 0u, 0u, 0u};
      if (e < kAKT * KC * 4 && j < k_end && k < dk) pre[u] = load8(cache + (size_t)s_slot[buf][key] * dk + k, dk - k, vec != 0);
    }
  };
  constexpr bool kAhead = KC <= 6;  // the wider instances have no registers to spare for a tile in flight
  if (threadIdx.x < kAKT && k_begin + (int)threadIdx.x < k_end) s_slot[0][threadIdx.x] = trow[k_begin + threadIdx.x];
  __syncthreads();
  if (kAhead && k_begin < k_end) request(k_begin, 0);
  int buf = 0;
  for (int j0 = k_begin; j0 < k_end; j0 += kAKT, buf ^= 1) {
    __syncthreads();
    if (threadIdx.x < kAKT && j0 + kAKT + (int)threadIdx.x < k_end) s_slot[buf ^ 1][threadIdx.x] = trow[j0 + kAKT + threadIdx.x];
    if (kAhead) {
#pragma unroll
      for (int u = 0; u < NCH; ++u) {
        const int e = u * 256 + threadIdx.x;
        const int key = e / (KC * 4), ch = e - key * (KC * 4);
        if (e < kAKT * KC * 4) *reinterpret_cast<Q4*>(&sk[key * KS + ch * 8]) = pre[u];
      }
    } else {
      // batches of up to 8 row pieces per thread: all loads of a batch are issued before its first LDS store (a store that
      // waits for its load would hold back the next piece's slot read behind it: LDS operations of a wave stay in order)
      constexpr int kBatch = 8;
      if constexpr (KC > 10) {  // the widest instances have no registers for a batch: piece by piece
#pragma unroll 8
        for (int e = threadIdx.x; e < kAKT * KC * 4; e += 256) {
          const int key = e / (KC * 4), ch = e - key * (KC * 4);
          const int j = j0 + key, k = ch * 8;
          Q4 v{0u, 0u, 0u, 0u};
          if (j < k_end && k < dk) v = load8(cache + (size_t)s_slot[buf][key] * dk + k, dk - k, vec != 0);
          *reinterpret_cast<Q4*>(&sk[key * KS + k]) = v;
        }
      } else
#pragma unroll
      for (int u0 = 0; u0 < NCH; u0 += kBatch) {
        Q4 tmp[kBatch];
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int e = (u0 + u) * 256 + threadIdx.x;
          const int key = e / (KC * 4), ch = e - key * (KC * 4);
          const int j = j0 + key, k = ch * 8;
          tmp[u] = Q4{0u, 0u, 0u, 0u};
          if (u0 + u < NCH && e < kAKT * KC * 4 && j < k_end && k < dk)
            tmp[u] = load8(cache + (size_t)s_slot[buf][key] * dk + k, dk - k, vec != 0);
        }
#pragma unroll
        for (int u = 0; u < kBatch; ++u) {
          const int e = (u0 + u) * 256 + threadIdx.x;
          const int key = e / (KC * 4), ch = e - key * (KC * 4);
          if (u0 + u < NCH && e < kAKT * KC * 4) *reinterpret_cast<Q4*>(&sk[key * KS + ch * 8]) = tmp[u];
        }
      }
    }
    __syncthreads();
    if (kAhead && j0 + kAKT < k_end) request(j0 + kAKT, buf ^ 1);
    if (!wave_live) continue;
    // scores of the whole 64-key tile first (four independent MFMA chains), ONE softmax step for the tile (one exchange
    // across the lane groups, one rescale of O), then the four value products; rows past k_end are zero rows with weight 0
    constexpr int NKS = kAKT / 16;
    float sc[NKS][4], mx = -INFINITY;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      f32x4_t sacc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) {
        const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(&sk[(ks * 16 + lr) * KS + kc * 32 + lg * 8]);
        sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[kc], sacc, 0, 0, 0);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int j = j0 + ks * 16 + 4 * lg + c;
        sc[ks][c] = (j <= limit && j < k_end) ? sacc[c] * scale : -INFINITY;
        mx = fmaxf(mx, sc[ks][c]);
      }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const bool none = m_new == -INFINITY;  // this row has seen no key yet
    const float corr = none ? 1.f : __expf(m - m_new);
    float ps = 0.f;
    s16x4_t pf[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      float pe[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        pe[c] = none ? 0.f : __expf(sc[ks][c] - m_new);
        ps += pe[c];
      }
      const uint32_t p01 = bf16_bits(pe[0]) | (bf16_bits(pe[1]) << 16), p23 = bf16_bits(pe[2]) | (bf16_bits(pe[3]) << 16);
      pf[ks] = __builtin_bit_cast(s16x4_t, uint2{p01, p23});
    }
    lsum = lsum * corr + ps;
    m = m_new;
    if (__builtin_amdgcn_ballot_w64(corr != 1.f) != 0) {
#pragma unroll
      for (int vt = 0; vt < VC; ++vt) {
        o[vt][0] *= corr; o[vt][1] *= corr; o[vt][2] *= corr; o[vt][3] *= corr;
      }
    }
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (j0 + ks * 16 >= k_end) break;
      const uint16_t* vbase = &sk[(ks * 16 + 4 * lg + (lr >> 2)) * KS + 4 * (lr & 3)];
#pragma unroll
      for (int vt = 0; vt < VC; ++vt) {
        const s16x4_t vf = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(vbase + vt * 16));
        o[vt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pf[ks], o[vt], 0, 0, 0);
      }
    }
  }
  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);
  if (!valid) return;
  const size_t row = (size_t)tok * H + head;
  if (splits == 1) {
    const float inv = sink_factor(sink, head, m) / (sink_factor(sink, head, m) * lsum + sink_weight(sink, head, m));
#pragma unroll
    for (int vt = 0; vt < VC; ++vt)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int v = vt * 16 + 4 * lg + c;
        if (v < dv) out[row * dv + v] = o[vt][c] * inv;
      }
  } else {
    float* po = part_o + (row * splits + z) * dv;
#pragma unroll
    for (int vt = 0; vt < VC; ++vt)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int v = vt * 16 + 4 * lg + c;
        if (v < dv) po[v] = o[vt][c];
      }
    if (lg == 0) {
      part_ml[(row * splits + z) * 2] = m;
      part_ml[(row * splits + z) * 2 + 1] = lsum;
    }
  }
}

// out[row] = sum_z e^(m_z - m*) o_z / (sum_z e^(m_z - m*) l_z + e^(sink - m*)), splits in order; a split without keys has l = 0
// and m = -inf; without a sink its term is absent
__global__ __launch_bounds__(64) void latent_attn_merge_kernel(float* __restrict__ out, const float* __restrict__ part_o,
                                                               const float* __restrict__ part_ml, int splits, int dv,
                                                               const float* __restrict__ sink, int H) {
  __shared__ float sw[1024];  // per split: its max, then its weight e^(m_z - m*)
  __shared__ float sl[1024];
  const size_t row = blockIdx.x;
  for (int z = threadIdx.x; z < splits; z += 64) {  // every (m, l) pair is read from memory once
    sw[z] = part_ml[(row * splits + z) * 2];
    sl[z] = part_ml[(row * splits + z) * 2 + 1];
  }
  __syncthreads();
  float ms = sink ? sink[row % H] : -INFINITY;  // the sink joins the maximum and the denominator like one more range
  for (int z = 0; z < splits; ++z) ms = fmaxf(ms, sw[z]);
  float l = sink ? __expf(sink[row % H] - ms) : 0.f;
  for (int z = 0; z < splits; ++z) l += sw[z] > -INFINITY ? sl[z] * __expf(sw[z] - ms) : 0.f;
  __syncthreads();
  for (int z = threadIdx.x; z < splits; z += 64) sw[z] = sw[z] > -INFINITY ? __expf(sw[z] - ms) : 0.f;
  __syncthreads();
  const float inv = 1.0f / l;
  for (int v = threadIdx.x; v < dv; v += 64) {
    float acc = 0.f;
#pragma unroll 8
    for (int z = 0; z < splits; ++z) acc = fmaf(part_o[(row * splits + z) * dv + v], sw[z], acc);
    out[row * dv + v] = acc * inv;
  }
}

}  // namespace

extern "C" {

static thread_local char g_err[512] = "";
const char* msgl_mix_last_error(void) { return g_err; }
void msgl_mix_set_error(const char* text) { snprintf(g_err, sizeof(g_err), "%s", text); }
int msgl_mix_abi_version(void) { return MSGL_MIX_ABI_VERSION; }

int msgl_mix_embed(float* x32, void* h, const void* table, const int* ids, int tokens, int W, int dtype, void* stream) {
  MIX_REQUIRE(x32 && h && table && ids && tokens >= 0 && W >= 1 && dtype_ok(dtype), "embed: bad arguments");
  if (tokens == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(embed_rows_kernel<T>, dim3(tokens), dim3(256), 0, s, x32, mp<T>(h), cp<T>(table), ids, W);)
  MIX_LAUNCHED("embed");
  return MSGL_MIX_OK;
}

int msgl_mix_postnorm(const float* x_in, float* x_out, void* h_out, const void* y, int parts, const float* gate, const void* w,
                      float alpha, float eps, int rows, int W, int dtype, const void* router, const void* bias, int E, int top, int G,
                      int keep, int* ids, float* wts, void* stream) {
  MIX_REQUIRE(x_in && w && (x_out || h_out) && rows >= 0 && W >= 1 && dtype_ok(dtype), "postnorm: bad arguments");
  MIX_REQUIRE((parts == 0) == (y == nullptr) && parts >= 0, "postnorm: parts = %d does not match y", parts);
  const bool route = router != nullptr;
  if (route) {
    MIX_REQUIRE(ids && wts, "postnorm: a router needs ids and wts");
    MIX_REQUIRE(E >= 1 && top >= 1 && top <= E && G >= 1 && E % G == 0 && keep >= 1 && keep <= G && top <= keep * (E / G),
                "postnorm: bad router sizes E %d top %d groups %d keep %d", E, top, G, keep);
  }
  if (rows == 0) return MSGL_MIX_OK;
  const size_t lds = (size_t)(W + 4 + (route ? 2 * E + G + top : 0)) * sizeof(float);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define PN_LAUNCH(ROUTE)                                                                                                                \
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)postnorm_kernel<T, ROUTE>, lds) == 0, "postnorm: row of %d does not fit LDS", W); \
             hipLaunchKernelGGL((postnorm_kernel<T, ROUTE>), dim3(rows), dim3(256), lds, s, x_in, x_out, mp<T>(h_out), cp<T>(y), parts,   \
                                gate, cp<T>(w), alpha, eps, W, cp<T>(router), cp<T>(bias), E, top, G, keep, ids, wts);)
  if (route) {
    PN_LAUNCH(true)
  } else {
    PN_LAUNCH(false)
  }
#undef PN_LAUNCH
  MIX_LAUNCHED("postnorm");
  return MSGL_MIX_OK;
}

int msgl_mix_latent_prep(const void* proj, int64_t ld_proj, float* q_abs, void* cache, const int* out_loc, const int* positions,
                         const float* cos_sin, const void* c_norm_w, float eps, int tokens, int H, int d, int r, int rot_dims, int R,
                         int has_kv, int interleaved, int dtype, void* stream) {
  MIX_REQUIRE(proj && q_abs && positions && cos_sin && dtype_ok(dtype), "latent_prep: null pointer / dtype");
  MIX_REQUIRE(H >= 1 && d >= 0 && r >= 0 && R >= 1 && rot_dims >= 0 && rot_dims <= r && rot_dims % 2 == 0,
              "latent_prep: bad sizes H %d d %d r %d rot %d R %d", H, d, r, rot_dims, R);
  MIX_REQUIRE(!has_kv || (cache && out_loc && c_norm_w), "latent_prep: a layer with its own latent needs cache, out_loc and norm weight");
  MIX_REQUIRE(ld_proj >= (int64_t)H * (d + r) + (has_kv ? R + r : 0), "latent_prep: projection row too short");
  if (tokens == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(latent_prep_kernel<T>, dim3(tokens), dim3(256), 0, s, cp<T>(proj), ld_proj, q_abs, mp<T>(cache),
                                       out_loc, positions, cos_sin, cp<T>(c_norm_w), eps, H, d, r, rot_dims, R, has_kv, interleaved);)
  MIX_LAUNCHED("latent_prep");
  return MSGL_MIX_OK;
}

int msgl_mix_latent_attn_workspace_floats(int total_q, int H, int dv, int splits) {
  return splits > 1 ? total_q * H * splits * (dv + 2) : 0;
}

int msgl_mix_latent_attn(float* out, const float* q_abs, const void* cache, const int* table, int64_t table_stride, const int* req_rows,
                         const int* seq_lens, const int* cu_q, int batch, int total_q, int H, int dk, int dv, float scale,
                         const float* sink, int dtype, int splits, float* workspace, void* stream) {
  MIX_REQUIRE(out && q_abs && cache && table && req_rows && seq_lens && cu_q && dtype_ok(dtype), "latent_attn: null pointer / dtype");
  MIX_REQUIRE(batch >= 1 && total_q >= 0 && H >= 1 && dv >= 1 && dk >= dv, "latent_attn: bad sizes");
  MIX_REQUIRE(splits >= 1 && splits <= 1024 && (splits == 1 || workspace), "latent_attn: %d splits need a workspace", splits);
  if (total_q == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MSGL_MIX_BF16 && dk <= 18 * 32 && dv <= 32 * 16) {
    // matrix-core kernel: the smallest (KC, VC) instance that holds dk <= 32 KC and dv <= 16 VC (and 16 VC <= 32 KC)
    const int HB = H < 64 ? H : 64;
    const int QT = 64 / HB;
    const int groups = (total_q + QT - 1) / QT + batch;
    const dim3 grid(groups, (H + HB - 1) / HB, splits);
    MIX_REQUIRE(grid.y <= 65535, "latent_attn: too many heads");
    float* part_o = workspace;
    float* part_ml = workspace ? workspace + (size_t)total_q * H * splits * dv : nullptr;
    const int vec = (((uintptr_t)cache & 15u) == 0 && dk % 8 == 0) ? 1 : 0;
#define ATTN_CASE(KC, VC)                                                                                                              \
  if (dk <= KC * 32 && dv <= VC * 16) {                                                                                                \
    const size_t lds = (size_t)kAKT * (KC * 32 + 8) * sizeof(uint16_t);                                                                \
    MIX_REQUIRE(ensure_lds((const void*)latent_attn_mfma_kernel<KC, VC>, lds) == 0, "latent_attn: LDS request refused");               \
    hipLaunchKernelGGL((latent_attn_mfma_kernel<KC, VC>), grid, dim3(256), lds, s, out, part_o, part_ml, q_abs, cp<bf16_t>(cache), table, \
                       table_stride, req_rows, seq_lens, cu_q, batch, H, dk, dv, scale, QT, HB, splits, vec, sink);                    \
    MIX_LAUNCHED("latent_attn (matrix cores)");                                                                                        \
    if (splits > 1) {                                                                                                                  \
      hipLaunchKernelGGL(latent_attn_merge_kernel, dim3(total_q * H), dim3(64), 0, s, out, part_o, part_ml, splits, dv, sink, H);       \
      MIX_LAUNCHED("latent_attn merge");                                                                                               \
    }                                                                                                                                  \
    return MSGL_MIX_OK;                                                                                                                \
  }
    ATTN_CASE(2, 4)
    ATTN_CASE(4, 8)
    ATTN_CASE(6, 8)
    ATTN_CASE(10, 16)
    ATTN_CASE(12, 20)
    ATTN_CASE(18, 32)
#undef ATTN_CASE
  }
  MIX_REQUIRE(dv <= 16 * kAttnMaxC, "latent_attn: value width %d above %d", dv, 16 * kAttnMaxC);
  const int HB = H < kAttnRows ? H : kAttnRows;
  const int QT = kAttnRows / HB;
  int KT = 64;
  auto need = [&](int kt) { return (size_t)((kAttnRows + kt) * (dk + 1) + kAttnRows * kt) * sizeof(float); };
  while (KT > 8 && need(KT) > 160 * 1024) KT >>= 1;
  const size_t lds = need(KT);
  MIX_REQUIRE(lds <= 160 * 1024, "latent_attn: key width %d does not fit LDS", dk);
  const int groups = (total_q + QT - 1) / QT + batch;  // every request may end with one partial group
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)latent_attn_kernel<T>, lds) == 0, "latent_attn: LDS request refused");
             hipLaunchKernelGGL(latent_attn_kernel<T>, dim3(groups, (H + HB - 1) / HB), dim3(256), lds, s, out, q_abs, cp<T>(cache), table,
                                table_stride, req_rows, seq_lens, cu_q, batch, H, dk, dv, scale, QT, HB, KT, sink);)
  MIX_LAUNCHED("latent_attn");
  return MSGL_MIX_OK;
}

int msgl_mix_lightning(float* out, const void* qkv, int64_t ld_qkv, float* state, const float* decay, const int* cu_q, const int* seq_lens,
                       const int* slots, int batch, int H, int d, int dv, int dtype, int n_items, const int* items, const int* item_first,
                       float* scratch, void* stream) {
  MIX_REQUIRE(out && qkv && state && decay && cu_q && seq_lens && slots && dtype_ok(dtype), "lightning: null pointer / dtype");
  MIX_REQUIRE(batch >= 1 && batch <= 65535 && H >= 1 && d >= 1 && dv >= 1, "lightning: bad sizes");
  MIX_REQUIRE(ld_qkv >= (int64_t)H * (2 * d + dv), "lightning: projection row too short");
  MIX_REQUIRE(n_items == 0 || (items && item_first && scratch && n_items <= 65535), "lightning: chunk list without its arrays");
  const int CB = dv < kLtMaxCols ? dv : kLtMaxCols;
  const int NS = 256 / CB;
  const int need = (d + NS - 1) / NS;
  MIX_REQUIRE(need <= kLtMaxRows, "lightning: key size %d needs more than %d state rows per thread", d, kLtMaxRows);
  const int col_blocks = (dv + CB - 1) / CB;
  MIX_REQUIRE(col_blocks <= 65535, "lightning: value width %d", dv);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define LT_LAUNCH(RR, ROWS, MODE)                                                                                                      \
  hipLaunchKernelGGL((lightning_kernel<T, RR>), dim3(H, ROWS, col_blocks), dim3(256), lds, s, out, cp<T>(qkv), ld_qkv, state, decay,   \
                     cu_q, seq_lens, slots, H, d, dv, CB, NS, items, scratch, MODE);                                                   \
  MIX_LAUNCHED("lightning");
#define LT_CASE(RR)                                                                                                                    \
  if (need <= RR) {                                                                                                                    \
    const size_t lds = (size_t)(kLtTok * (2 * NS * RR + CB) + kLtTok * NS * CB) * sizeof(float);                                       \
    DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)lightning_kernel<T, RR>, lds) == 0, "lightning: LDS request refused");       \
               if (n_items == 0) { LT_LAUNCH(RR, batch, 0) } else {                                                                    \
                 LT_LAUNCH(RR, n_items, 1)                                                                                             \
                 hipLaunchKernelGGL(lightning_scan_kernel, dim3(H, batch, (d * dv + 255) / 256), dim3(256), 0, s, state, scratch,      \
                                    decay, cu_q, seq_lens, slots, items, item_first, H, d * dv);                                       \
                 MIX_LAUNCHED("lightning scan");                                                                                       \
                 LT_LAUNCH(RR, n_items, 2)                                                                                             \
               })                                                                                                                      \
    return MSGL_MIX_OK;                                                                                                                \
  }
  LT_CASE(4)
  LT_CASE(8)
  LT_CASE(16)
  LT_CASE(32)
  LT_CASE(64)
#undef LT_CASE
#undef LT_LAUNCH
  return MSGL_MIX_EINVAL;
}

int msgl_mix_gated_norm(void* out, const float* o, const void* gate, int64_t ld_gate, const void* w, float eps, int rows, int N, int dtype,
                        void* stream) {
  MIX_REQUIRE(out && o && gate && w && rows >= 0 && N >= 1 && ld_gate >= N && dtype_ok(dtype), "gated_norm: bad arguments");
  if (rows == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(gated_norm_kernel<T>, dim3(rows), dim3(256), 0, s, mp<T>(out), o, cp<T>(gate), ld_gate, cp<T>(w), eps, N);)
  MIX_LAUNCHED("gated_norm");
  return MSGL_MIX_OK;
}

int msgl_mix_route(int* ids, float* wts, const float* z, const void* bias, int tokens, int E, int top, int G, int keep, int dtype,
                   void* stream) {
  MIX_REQUIRE(ids && wts && z && dtype_ok(dtype), "route: null pointer / dtype");
  MIX_REQUIRE(E >= 1 && top >= 1 && top <= E && G >= 1 && E % G == 0 && keep >= 1 && keep <= G && top <= keep * (E / G),
              "route: bad sizes E %d top %d groups %d keep %d", E, top, G, keep);
  if (tokens == 0) return MSGL_MIX_OK;
  int tpb = 64;
  while (tpb > 1 && (size_t)(2 * E + G) * tpb * sizeof(float) > 64 * 1024) tpb >>= 1;
  const size_t lds = (size_t)(2 * E + G) * tpb * sizeof(float);
  MIX_REQUIRE(lds <= 64 * 1024, "route: too many experts");
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(route_kernel<T>, dim3((tokens + tpb - 1) / tpb), dim3(64), lds, s, ids, wts, z, cp<T>(bias), tokens, E,
                                       top, G, keep, tpb);)
  MIX_LAUNCHED("route");
  return MSGL_MIX_OK;
}

int msgl_mix_moe_sort(int* seg, int* perm, int* counts, const int* ids, int n, int E, void* stream) {
  MIX_REQUIRE(seg && perm && counts && ids && n >= 0 && E >= 1 && E <= 65535, "moe_sort: bad arguments");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(moe_count_kernel, dim3(E), dim3(256), 0, s, counts, ids, n);
  MIX_LAUNCHED("moe_sort (count)");
  hipLaunchKernelGGL(moe_place_kernel, dim3(E), dim3(256), 0, s, seg, perm, counts, ids, n, E);
  MIX_LAUNCHED("moe_sort (place)");
  return MSGL_MIX_OK;
}

int msgl_mix_gemm_nt(void* C, const void* A, const void* B, int M, int N, int K, int64_t lda, int64_t ldb, int64_t ldc, int groups,
                     int64_t a_gs, int64_t b_gs, int64_t c_gs, const int* seg, const int* a_rows, int a_div, const int* c_rows, int act,
                     int ta, int tb, int tc, void* stream) {
  MIX_REQUIRE(C && A && B && M >= 0 && N >= 1 && K >= 1 && groups >= 1 && groups <= 65535, "gemm_nt: bad arguments");
  MIX_REQUIRE(dtype_ok(ta) && dtype_ok(tb) && dtype_ok(tc), "gemm_nt: dtype codes");
  MIX_REQUIRE(lda >= K && ldb >= K && a_div >= 1, "gemm_nt: leading dimensions");
  MIX_REQUIRE(act == MSGL_MIX_ACT_NONE || act == MSGL_MIX_ACT_RELU2, "gemm_nt: activation code %d", act);
  if (M == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (tb == MSGL_MIX_BF16) {  // 16-bit weights: the matrix-core kernel
    const int row_tiles = (M + kMT - 1) / kMT;
    MIX_REQUIRE(row_tiles <= 65535, "gemm_nt: too many rows");
    const dim3 grid((N + kMT - 1) / kMT, row_tiles, groups);
    auto al = [](const void* p, int64_t ld, int64_t gs, int elems) {
      return ((uintptr_t)p & 15u) == 0 && ld % elems == 0 && gs % elems == 0;
    };
    const int b_vec = al(B, ldb, b_gs, 8);
    const int a_vec = ta == MSGL_MIX_BF16 ? al(A, lda, a_gs, 8) : al(A, lda, a_gs, 4);
#define MFMA_CASE(CA, CC, TA, TC)                                                                                                   \
  if (ta == CA && tc == CC) {                                                                                                       \
    hipLaunchKernelGGL((gemm_nt_mfma_kernel<TA, TC>), grid, dim3(256), 0, s, mp<TC>(C), cp<TA>(A), cp<bf16_t>(B), M, N, K, lda, ldb, \
                       ldc, a_gs, b_gs, c_gs, seg, a_rows, a_div, c_rows, act, a_vec, b_vec);                                       \
    MIX_LAUNCHED("gemm_nt (matrix cores)");                                                                                         \
    return MSGL_MIX_OK;                                                                                                             \
  }
    MFMA_CASE(MSGL_MIX_BF16, MSGL_MIX_BF16, bf16_t, bf16_t)
    MFMA_CASE(MSGL_MIX_BF16, MSGL_MIX_F32, bf16_t, float)
    MFMA_CASE(MSGL_MIX_F32, MSGL_MIX_BF16, float, bf16_t)
    MFMA_CASE(MSGL_MIX_F32, MSGL_MIX_F32, float, float)
#undef MFMA_CASE
  }
  const int row_tiles = (M + kTile - 1) / kTile;
  MIX_REQUIRE(row_tiles <= 65535, "gemm_nt: too many rows");
  const dim3 grid((N + kTile - 1) / kTile, row_tiles, groups);
#define GEMM_CASE(CA, CB, CC, TA, TB, TC)                                                                                            \
  if (ta == CA && tb == CB && tc == CC) {                                                                                            \
    hipLaunchKernelGGL((gemm_nt_kernel<TA, TB, TC>), grid, dim3(256), 0, s, mp<TC>(C), cp<TA>(A), cp<TB>(B), M, N, K, lda, ldb, ldc, \
                       a_gs, b_gs, c_gs, seg, a_rows, a_div, c_rows, act);                                                           \
    MIX_LAUNCHED("gemm_nt");                                                                                                         \
    return MSGL_MIX_OK;                                                                                                              \
  }
  GEMM_CASE(MSGL_MIX_F32, MSGL_MIX_F32, MSGL_MIX_F32, float, float, float)
#undef GEMM_CASE
  set_err("gemm_nt: no kernel for dtype codes (%d, %d, %d)", ta, tb, tc);
  return MSGL_MIX_EINVAL;
}

}  // extern "C"
