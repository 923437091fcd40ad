// Kernels of the parallel-residual hybrid decoders (one norm per layer feeding a token-shifted mixer and a feed-forward side
// by side; mixers: latent attention with a sink, or sigmoid attention beside a state-space layer), gfx950, wave = 64 lanes.
// Third translation unit of libmsgl_mix.so; C ABI in include/msgl_mix.h.
//
// Precision rules (as in seqmix.hip): the residual stream, every norm, rotary angles, attention scores and weights, step
// sizes, decays and the recurrent state are fp32 in registers and in memory; tensors that feed a matrix product are stored in
// the model dtype T (bf16 or fp32).  With T = float every kernel here is true 32-bit.
//
//   embed_scaled_kernel     x[t] = scale * table[id] + pair_table[hash(previous id, id)]       (fp32)
//   shift_norm_kernel       closes a layer and opens the next: x' = x + bias + v0 * y0 + v1 * y1;  h = rms(x') * w;
//                           g = h + (h_prev - h) * shift with h_prev the previous token's h (same launch: recomputed from the
//                           previous row; first token of a portion: the request's state row; position 0: zero)
//   commit_rows_kernel      after the forward: every request's last h of every layer -> its state row; its last token id
//   qk_prep_kernel          q, k (+ bias), rotation of the leading entries of each head, unit-RMS q and k; k, v -> cache rows
//   sigmoid_attn_mfma_kernel  o[t, h] = sum_{j <= t} sigmoid(cap(scale q . k_j) + b_h) v_j, no normalisation over keys; bf16 caches,
//                           both products on the matrix cores, weights in fp32; key ranges are plain partial sums
//                           (sigmoid_merge_kernel adds them)
//   sigmoid_attn_kernel     the same in plain fp32 (fp32 caches, heads past the matrix-core instances)
//   ssd_kernel              S <- exp(rate dt) S + dt B x^T,  y = S^T C + D x per (request, head); four waves share the rows of a
//                           state column; long portions as parallel chunks joined by ssd_scan_kernel
//   gate_group_norm_kernel  (y * silu(z)) normed in equal groups of the row, times w
//   xielu_kernel            z > 0: a z^2 + z / 2;  z <= 0: b (exp(z) - 1 - z) + z / 2
#include "mix_common.h"

namespace {

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

// ------------------------------------------------------------------------------------------------ embedding
// pair != null: the row (prev * mul_prev + id * mul_cur) mod buckets of `pair` is added; a sequence's first token takes row
// `buckets`.  The previous id of a portion's first token is the request's entry of prev_tok.
template <typename T>
__global__ __launch_bounds__(256) void embed_scaled_kernel(float* __restrict__ x32, const T* __restrict__ table, const T* __restrict__ pair,
                                                           const int* __restrict__ ids, const int* __restrict__ positions,
                                                           const int* __restrict__ cu_q, const int* __restrict__ req_rows, int batch,
                                                           const int* __restrict__ prev_tok, float scale, int buckets, int mul_prev,
                                                           int mul_cur, int W) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const T* row = table + (size_t)id * W;
  const T* prow = nullptr;
  if (pair) {
    int64_t r = buckets;
    if (positions[t] != 0) {
      const int b = request_of(cu_q, batch, t);
      const int prev = t > cu_q[b] ? ids[t - 1] : prev_tok[req_rows[b]];
      r = ((int64_t)prev * mul_prev + (int64_t)id * mul_cur) % buckets;
    }
    prow = pair + (size_t)r * W;
  }
  for (int i = threadIdx.x; i < W; i += 256) x32[(size_t)t * W + i] = ld(row + i) * scale + (prow ? ld(prow + i) : 0.f);
}

// ------------------------------------------------------------------------------------------------ residual sum + norm + token shift
// One workgroup per token.  row(t) = x_in[t] + bias + v0 * y0[t] + v1 * y1[t] (v: fp32 per column, null = ones) -> x_out;
// h = row * rsqrt(mean(row^2) + eps) * (w + w_off) -> h_out (T).  With `shift`: g = h + (h_prev - h) * shift -> g_out (T), h_prev = the h of
// the token before (fp32, not rounded): recomputed here from row(t - 1) inside a portion (the same arithmetic in the same order,
// so it equals what that token's own workgroup computes), state[req_rows[b]] for a portion's first token, zero at position 0.
// The last token of every request leaves its h in staging[b]; commit_rows_kernel moves it to the state row after the forward
// (a portion's first and last token run in different workgroups of this launch, so the state row cannot be replaced here).
// A workgroup takes TT consecutive tokens; only the first of them has to rebuild the row before it.
// VEC: W is a multiple of 8 and every row is 16-byte aligned -- a thread takes 8 consecutive columns at a time with 16-byte loads
// and stores; otherwise one column at a time.  Either way a thread only ever touches its own columns of the LDS rows.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void shift_norm_kernel(const float* __restrict__ x_in, float* __restrict__ x_out, const T* __restrict__ y0,
                                                         int64_t ld0, const float* __restrict__ v0, const T* __restrict__ y1, int64_t ld1,
                                                         const float* __restrict__ v1, const float* __restrict__ bias,
                                                         const float* __restrict__ w, float w_off, const float* __restrict__ shift, T* __restrict__ h_out,
                                                         T* __restrict__ g_out, const float* __restrict__ state, float* __restrict__ staging,
                                                         const int* __restrict__ positions, const int* __restrict__ cu_q,
                                                         const int* __restrict__ req_rows, int batch, float eps, int W, int rows, int TT) {
  extern __shared__ __attribute__((aligned(16))) float srow[];  // two rows of W: this token's and the one before it
  __shared__ float red[4];
  constexpr int kStep = VEC ? 8 : 1;
  auto vec_of = [](const float* __restrict__ p, int c, float (&f)[kStep]) {  // kStep columns of a per-column fp32 vector
    if constexpr (VEC) {
      read8(p + c, f);
    } else {
      f[0] = p[c];
    }
  };
  auto row_of = [&](int tt, float* dst, bool store) {
    float ss = 0.f;
    for (int c = threadIdx.x * kStep; c < W; c += 256 * kStep) {
      float s[kStep], a[kStep], m[kStep];
      if constexpr (VEC) {
        read8(x_in + (size_t)tt * W + c, s);
      } else {
        s[0] = x_in[(size_t)tt * W + c];
      }
      if (bias) {
        vec_of(bias, c, a);
#pragma unroll
        for (int u = 0; u < kStep; ++u) s[u] += a[u];
      }
      if (y0) {
        if constexpr (VEC) read8(y0 + (size_t)tt * ld0 + c, a); else a[0] = ld(y0 + (size_t)tt * ld0 + c);
#pragma unroll
        for (int u = 0; u < kStep; ++u) m[u] = 1.f;
        if (v0) vec_of(v0, c, m);
#pragma unroll
        for (int u = 0; u < kStep; ++u) s[u] = fmaf(m[u], a[u], s[u]);
      }
      if (y1) {
        if constexpr (VEC) read8(y1 + (size_t)tt * ld1 + c, a); else a[0] = ld(y1 + (size_t)tt * ld1 + c);
#pragma unroll
        for (int u = 0; u < kStep; ++u) m[u] = 1.f;
        if (v1) vec_of(v1, c, m);
#pragma unroll
        for (int u = 0; u < kStep; ++u) s[u] = fmaf(m[u], a[u], s[u]);
      }
      if (store) {
        if constexpr (VEC) write8(x_out + (size_t)tt * W + c, s); else x_out[(size_t)tt * W + c] = s[0];
      }
#pragma unroll
      for (int u = 0; u < kStep; ++u) {
        dst[c + u] = s[u];
        ss += s[u] * s[u];
      }
    }
    return 1.0f / sqrtf(block_sum256(ss, red) / (float)W + eps);
  };
  // a workgroup walks TT consecutive tokens: from the second on, the row before is still in LDS and is not read again
  float inv_before = 0.f;
  for (int k = 0; k < TT; ++k) {
    const int t = blockIdx.x * TT + k;
    if (t >= rows) break;
    float* cur = srow + (k & 1) * W;
    float* prv = srow + ((k & 1) ^ 1) * W;
    const float inv = row_of(t, cur, x_out != nullptr);
    if (!shift) {
      for (int c = threadIdx.x * kStep; c < W; c += 256 * kStep) {
        float h[kStep], wv[kStep];
        vec_of(w, c, wv);
#pragma unroll
        for (int u = 0; u < kStep; ++u) h[u] = cur[c + u] * inv * (wv[u] + w_off);
        if constexpr (VEC) write8(h_out + (size_t)t * W + c, h); else st(h_out + (size_t)t * W + c, h[0]);
      }
      continue;
    }
    const int b = request_of(cu_q, batch, t);
    const bool last = t == cu_q[b + 1] - 1;
    const int mode = positions[t] == 0 ? 0 : (t > cu_q[b] ? 1 : 2);  // uniform over the workgroup
    float inv_p = inv_before;
    if (mode == 1 && k == 0) inv_p = row_of(t - 1, prv, false);
    const float* srow_state = state + (size_t)req_rows[b] * W;
    for (int c = threadIdx.x * kStep; c < W; c += 256 * kStep) {
      float h[kStep], g[kStep], wv[kStep], sv[kStep], pv[kStep];
      vec_of(w, c, wv);
      vec_of(shift, c, sv);
      if (mode == 2) vec_of(srow_state, c, pv);
#pragma unroll
      for (int u = 0; u < kStep; ++u) {
        const float wi = wv[u] + w_off;
        h[u] = cur[c + u] * inv * wi;
        const float hp = mode == 0 ? 0.f : (mode == 1 ? prv[c + u] * inv_p * wi : pv[u]);
        g[u] = h[u] + (hp - h[u]) * sv[u];
      }
      if constexpr (VEC) {
        if (h_out) write8(h_out + (size_t)t * W + c, h);
        write8(g_out + (size_t)t * W + c, g);
        if (last) write8(staging + (size_t)b * W + c, h);
      } else {
        if (h_out) st(h_out + (size_t)t * W + c, h[0]);
        st(g_out + (size_t)t * W + c, g[0]);
        if (last) staging[(size_t)b * W + c] = h[0];
      }
    }
    inv_before = inv;
  }
}

// dst[l][slots[b]] = src[l][b] for every layer l (grid.y) and request b (grid.x); prev_tok[slots[b]] = the request's last id.
__global__ __launch_bounds__(256) void commit_rows_kernel(float* __restrict__ dst, int64_t dst_stride, const float* __restrict__ src,
                                                          int64_t src_stride, const int* __restrict__ slots, int W, int* __restrict__ prev_tok,
                                                          const int* __restrict__ ids, const int* __restrict__ cu_q) {
  const int b = blockIdx.x, l = blockIdx.y;
  if (cu_q[b + 1] <= cu_q[b]) return;
  const size_t slot = (size_t)slots[b];
  if (dst) {
    const float* s = src + (size_t)l * src_stride + (size_t)b * W;
    float* d = dst + (size_t)l * dst_stride + slot * W;
    for (int i = threadIdx.x; i < W; i += 256) d[i] = s[i];
  }
  if (prev_tok && l == 0 && threadIdx.x == 0) prev_tok[slot] = ids[cu_q[b + 1] - 1];
}

// ------------------------------------------------------------------------------------------------ q / k preparation of grouped attention
// One workgroup per token.  proj row = [q: H x d | k: G x d | v: G x dv | ...] (+ bias, fp32, same layout, may be null).  The first
// rd entries of every q and k head turn by the token's angles (cos_sin row = cos | sin halves of rd / 2; pairs (2i, 2i + 1) when
// `interleaved`, else (i, i + rd / 2)); with bit 0 of `unit` every q and k head is then divided by its root mean square (eps inside
// the root), with bit 1 every v head.
// q -> q_out (fp32 [tokens, H * d]); k, v -> the cache rows at out_loc (T).
template <typename T>
__global__ __launch_bounds__(256) void qk_prep_kernel(const T* __restrict__ proj, int64_t ld_proj, const float* __restrict__ bias,
                                                      float* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                      const int* __restrict__ out_loc, const int* __restrict__ positions,
                                                      const float* __restrict__ cos_sin, int rd, int interleaved, int unit, float eps, int H,
                                                      int G, int d, int dv) {
  extern __shared__ float row[];  // (H + G) * d
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const T* src = proj + (size_t)t * ld_proj;
  const float* cs = cos_sin ? cos_sin + (size_t)positions[t] * rd : nullptr;
  const int half = rd >> 1, n = (H + G) * d;
  for (int e = threadIdx.x; e < n; e += 256) {
    const int hh = e / d, j = e - hh * d;
    auto in = [&](int jj) { return ld(src + (size_t)hh * d + jj) + (bias ? bias[(size_t)hh * d + jj] : 0.f); };
    float v = in(j);
    if (j < rd) {
      if (interleaved) {
        const int i = j >> 1;
        const float c = cs[i], s = cs[half + i], o = in(j ^ 1);
        v = (j & 1) ? v * c + o * s : v * c - o * s;
      } else {
        const int i = j < half ? j : j - half;
        const float c = cs[i], s = cs[half + i], o = in(j < half ? j + half : j - half);
        v = j < half ? v * c - o * s : v * c + o * s;
      }
    }
    row[e] = v;
  }
  __syncthreads();
  if (unit & 1) {
    for (int hh = wave; hh < H + G; hh += 4) {
      float ss = 0.f;
      for (int i = lane; i < d; i += 64) ss = fmaf(row[hh * d + i], row[hh * d + i], ss);
      const float f = 1.0f / sqrtf(wave_sum(ss) / (float)d + eps);
      for (int i = lane; i < d; i += 64) row[hh * d + i] *= f;
    }
    __syncthreads();
  }
  const size_t slot = (size_t)out_loc[t];
  for (int e = threadIdx.x; e < H * d; e += 256) q_out[(size_t)t * H * d + e] = row[e];
  for (int e = threadIdx.x; e < G * d; e += 256) st(k_cache + slot * G * d + e, row[H * d + e]);
  const size_t vo = (size_t)(H + G) * d;
  if (unit & 2) {  // every value head divided by its root mean square
    for (int g = wave; g < G; g += 4) {
      float ss = 0.f;
      for (int i = lane; i < dv; i += 64) {
        const float v = ld(src + vo + (size_t)g * dv + i) + (bias ? bias[vo + (size_t)g * dv + i] : 0.f);
        ss = fmaf(v, v, ss);
      }
      const float f = 1.0f / sqrtf(wave_sum(ss) / (float)dv + eps);
      for (int i = lane; i < dv; i += 64)
        st(v_cache + slot * G * dv + (size_t)g * dv + i, (ld(src + vo + (size_t)g * dv + i) + (bias ? bias[vo + (size_t)g * dv + i] : 0.f)) * f);
    }
    return;
  }
  for (int e = threadIdx.x; e < G * dv; e += 256) st(v_cache + slot * G * dv + e, ld(src + vo + e) + (bias ? bias[vo + e] : 0.f));
}

// ------------------------------------------------------------------------------------------------ sigmoid attention
// A workgroup = 16 query rows (QT tokens of one request x HB query heads of ONE key/value head) x 16 lanes, one range of the keys.
// Keys and values of the tile go through LDS as fp32; weight of a visible key = sigmoid(cap * tanh(scale q.k / cap) + pb[h])
// (cap <= 0: no soft cap), no normalisation: the output is the plain weighted sum of values, so key ranges add up.
constexpr int kSigRows = 16;
constexpr int kSigMaxC = 16;  // value columns per lane: dv <= 256

template <typename T>
__global__ __launch_bounds__(256) void sigmoid_attn_kernel(T* __restrict__ out, int64_t ld_out, float* __restrict__ part,
                                                           const float* __restrict__ q, const T* __restrict__ k_cache,
                                                           const T* __restrict__ v_cache, const int* __restrict__ table, int64_t table_stride,
                                                           const int* __restrict__ req_rows, const int* __restrict__ seq_lens,
                                                           const int* __restrict__ cu_q, int B, int total_q, int H, int G, int d, int dv,
                                                           float scale, float cap, const float* __restrict__ pb, float out_scale, int QT,
                                                           int HB, int KT, int splits) {
  extern __shared__ float lds[];
  const int qs = d + 1, vs = dv + 1;
  float* sq = lds;                      // [16][d + 1]
  float* sk = sq + kSigRows * qs;       // [KT][d + 1]
  float* sv = sk + KT * qs;             // [KT][dv + 1]
  float* sp = sv + KT * vs;             // [16][KT]
  __shared__ int s_req, s_tok0, s_cnt[256];
  find_group(cu_q, B, QT, s_cnt, &s_req, &s_tok0);
  const int b = s_req;
  if (b < 0) return;
  const int rep = H / G, hblocks = (rep + HB - 1) / HB;
  const int kvh = blockIdx.y / hblocks, h0 = kvh * rep + (blockIdx.y % hblocks) * HB;
  const int q_len = cu_q[b + 1] - cu_q[b];
  const int start = seq_lens[b] - q_len;  // position of the request's first new token
  const int r = threadIdx.x >> 4, l = threadIdx.x & 15;
  const int tl = s_tok0 + r / HB, hh = h0 + r % HB;
  const bool valid = r < QT * HB && tl < q_len && hh < (kvh + 1) * rep;
  const int tok = cu_q[b] + (valid ? tl : s_tok0);
  const int head = valid ? hh : h0;
  const int limit = valid ? start + tl : -1;  // last visible key
  const int last_tok = min(s_tok0 + QT, q_len) - 1;
  const int n_keys = start + last_tok + 1;
  const int per = ((n_keys + splits - 1) / splits + KT - 1) / KT * KT;
  const int k_begin = blockIdx.z * per, k_end = min(n_keys, k_begin + per);
  for (int i = l; i < d; i += 16) sq[r * qs + i] = q[((size_t)tok * H + head) * d + i];
  const int* trow = table + (size_t)req_rows[b] * table_stride;
  const float bias_h = pb ? pb[head] : 0.f;
  const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
  float o[kSigMaxC];
#pragma unroll
  for (int i = 0; i < kSigMaxC; ++i) o[i] = 0.f;
  const int nkd = G * d, nvd = G * dv;
  for (int j0 = k_begin; j0 < k_end; j0 += KT) {
    __syncthreads();
    const int nk = min(KT, k_end - j0);
    for (int e = threadIdx.x; e < nk * d; e += 256) {
      const int j = e / d, i = e - j * d;
      sk[j * qs + i] = ld(k_cache + (size_t)trow[j0 + j] * nkd + (size_t)kvh * d + i);
    }
    for (int e = threadIdx.x; e < nk * dv; e += 256) {
      const int j = e / dv, i = e - j * dv;
      sv[j * vs + i] = ld(v_cache + (size_t)trow[j0 + j] * nvd + (size_t)kvh * dv + i);
    }
    __syncthreads();
    for (int j = l; j < KT; j += 16) {
      float p = 0.f;
      if (j < nk && j0 + j <= limit) {
        float acc = 0.f;
        const float* qp = sq + r * qs;
        const float* kp = sk + j * qs;
        for (int i = 0; i < d; ++i) acc = fmaf(qp[i], kp[i], acc);
        float s = acc * scale;
        if (cap > 0.f) s = cap * tanhf(s * inv_cap);
        p = sigmoidf_(s + bias_h);
      }
      sp[r * KT + j] = p;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kSigMaxC; ++i) {
      const int c = l + 16 * i;
      if (c < dv) {
        float acc = o[i];
        for (int j = 0; j < nk; ++j) acc = fmaf(sp[r * KT + j], sv[j * vs + c], acc);
        o[i] = acc;
      }
    }
  }
  if (!valid) return;
#pragma unroll
  for (int i = 0; i < kSigMaxC; ++i) {
    const int c = l + 16 * i;
    if (c >= dv) continue;
    if (splits == 1)
      st(out + (size_t)tok * ld_out + (size_t)head * dv + c, o[i] * out_scale);
    else
      part[((size_t)blockIdx.z * total_q + tok) * H * dv + (size_t)head * dv + c] = o[i];
  }
}

// The same on the matrix cores, for bf16 caches.  A workgroup = 64 query rows ((token, head) pairs of one request and ONE key/value
// head: QT tokens x HB heads) in 4 waves of 16 rows, one key range.  Keys and values come through LDS in tiles of 64 rows, row-major,
// 16-byte padded.  Per 16-key subtile and wave:
//   S^T[16 keys x 16 rows] = K . Q^T     KC x v_mfma_f32_16x16x32_bf16   (Q fragments live in registers, rounded to bf16 once)
//   weights in fp32 in the lane that holds the score (one query row, four keys): the B-operand layout of the second product;
//   O^T[16 v x 16 rows] += V^T . P^T     VC x v_mfma_f32_16x16x16_bf16, V^T fragments read TRANSPOSED out of the row-major value
//   tile (ds_read_b64_tr_b16).  There is no running maximum and nothing to rescale: weights are independent of each other.
constexpr int kSKT = 64;

__device__ __forceinline__ float capped_sigmoid(float s, float cap, float inv_cap, float bias) {
  if (cap > 0.f) s = cap * (1.0f - 2.0f / (1.0f + __expf(2.0f * s * inv_cap)));  // cap * tanh(s / cap)
  return 1.0f / (1.0f + __expf(-(s + bias)));
}

template <int KC, int VC>
__global__ __launch_bounds__(256) void sigmoid_attn_mfma_kernel(bf16_t* __restrict__ out, int64_t ld_out, float* __restrict__ part,
                                                                const float* __restrict__ q, const bf16_t* __restrict__ k_cache,
                                                                const bf16_t* __restrict__ v_cache, const int* __restrict__ table,
                                                                int64_t table_stride, const int* __restrict__ req_rows,
                                                                const int* __restrict__ seq_lens, const int* __restrict__ cu_q, int B,
                                                                int total_q, int H, int G, int d, int dv, float scale, float cap,
                                                                const float* __restrict__ pb, float out_scale, int QT, int HB, int splits,
                                                                int kvec, int vvec) {
  constexpr int KS = KC * 32 + 8, VS = VC * 16 + 8;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* sk = smem;               // [kSKT][KS]
  uint16_t* sv = smem + kSKT * KS;   // [kSKT][VS]
  __shared__ int s_req, s_tok0, s_cnt[256];
  __shared__ int s_slot[2][kSKT];
  find_group(cu_q, B, QT, s_cnt, &s_req, &s_tok0);
  const int b = s_req;
  if (b < 0) return;
  const int rep = H / G, hblocks = (rep + HB - 1) / HB;
  const int kvh = blockIdx.y / hblocks, h0 = kvh * rep + (blockIdx.y % hblocks) * HB, z = blockIdx.z;
  const int q_len = cu_q[b + 1] - cu_q[b];
  const int start = seq_lens[b] - q_len;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int r = wave * 16 + lr;
  const int tl = s_tok0 + r / HB, hh = h0 + r % HB;
  const bool valid = r < QT * HB && tl < q_len && hh < (kvh + 1) * rep;
  const int tok = cu_q[b] + (valid ? tl : s_tok0);
  const int head = valid ? hh : h0;
  const int limit = valid ? start + tl : -1;
  const int last_tok = min(s_tok0 + QT, q_len) - 1;
  const int n_keys = start + last_tok + 1;
  const int per = ((n_keys + splits - 1) / splits + kSKT - 1) / kSKT * kSKT;
  const int k_begin = z * per, k_end = min(n_keys, k_begin + per);
  const bool wave_live = __builtin_amdgcn_ballot_w64(valid) != 0;
  bf16x8_t qf[KC];
  {
    const float* qrow = q + ((size_t)tok * H + head) * d;
#pragma unroll
    for (int kc = 0; kc < KC; ++kc) {
      const int k = kc * 32 + lg * 8;
      Q4 v = (valid && k < d) ? load8(qrow + k, d - k, (d & 3) == 0) : Q4{0u, 0u, 0u, 0u};
      qf[kc] = __builtin_bit_cast(bf16x8_t, v);
    }
  }
  f32x4_t o[VC];
#pragma unroll
  for (int vt = 0; vt < VC; ++vt) o[vt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const float bias_h = pb ? pb[head] : 0.f, inv_cap = cap > 0.f ? 1.0f / cap : 0.f;
  const int* trow = table + (size_t)req_rows[b] * table_stride;
  const size_t nkd = (size_t)G * d, nvd = (size_t)G * dv, ko = (size_t)kvh * d, vo = (size_t)kvh * dv;
  // the next tile's rows are requested before the current tile's products: their latency hides under the MFMAs
  constexpr int NK = (kSKT * KC * 4 + 255) / 256, NV = (kSKT * VC * 2 + 255) / 256;
  Q4 pre_k[NK], pre_v[NV];
  auto request = [&](int j0, int buf) {
#pragma unroll
    for (int u = 0; u < NK; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (KC * 4), k = (e - key * (KC * 4)) * 8;
      pre_k[u] = Q4{0u, 0u, 0u, 0u};
      if (e < kSKT * KC * 4 && j0 + key < k_end && k < d) pre_k[u] = load8(k_cache + (size_t)s_slot[buf][key] * nkd + ko + k, d - k, kvec != 0);
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (VC * 2), c = (e - key * (VC * 2)) * 8;
      pre_v[u] = Q4{0u, 0u, 0u, 0u};
      if (e < kSKT * VC * 2 && j0 + key < k_end && c < dv) pre_v[u] = load8(v_cache + (size_t)s_slot[buf][key] * nvd + vo + c, dv - c, vvec != 0);
    }
  };
  if (threadIdx.x < kSKT && k_begin + (int)threadIdx.x < k_end) s_slot[0][threadIdx.x] = trow[k_begin + threadIdx.x];
  __syncthreads();
  if (k_begin < k_end) request(k_begin, 0);
  int buf = 0;
  for (int j0 = k_begin; j0 < k_end; j0 += kSKT, buf ^= 1) {
    __syncthreads();
    if (threadIdx.x < kSKT && j0 + kSKT + (int)threadIdx.x < k_end) s_slot[buf ^ 1][threadIdx.x] = trow[j0 + kSKT + threadIdx.x];
#pragma unroll
    for (int u = 0; u < NK; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (KC * 4), ch = e - key * (KC * 4);
      if (e < kSKT * KC * 4) *reinterpret_cast<Q4*>(&sk[key * KS + ch * 8]) = pre_k[u];
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (VC * 2), ch = e - key * (VC * 2);
      if (e < kSKT * VC * 2) *reinterpret_cast<Q4*>(&sv[key * VS + ch * 8]) = pre_v[u];
    }
    __syncthreads();
    if (j0 + kSKT < k_end) request(j0 + kSKT, buf ^ 1);
    if (!wave_live) continue;
    constexpr int NKS = kSKT / 16;
    s16x4_t pf[NKS];
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      f32x4_t sacc{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) {
        const bf16x8_t kf = *reinterpret_cast<const bf16x8_t*>(&sk[(ks * 16 + lr) * KS + kc * 32 + lg * 8]);
        sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[kc], sacc, 0, 0, 0);
      }
      float pe[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int j = j0 + ks * 16 + 4 * lg + c;
        pe[c] = (j <= limit && j < k_end) ? capped_sigmoid(sacc[c] * scale, cap, inv_cap, bias_h) : 0.f;
      }
      const uint32_t p01 = bf16_bits(pe[0]) | (bf16_bits(pe[1]) << 16), p23 = bf16_bits(pe[2]) | (bf16_bits(pe[3]) << 16);
      pf[ks] = __builtin_bit_cast(s16x4_t, uint2{p01, p23});
    }
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (j0 + ks * 16 >= k_end) break;
      const uint16_t* vbase = &sv[(ks * 16 + 4 * lg + (lr >> 2)) * VS + 4 * (lr & 3)];
#pragma unroll
      for (int vt = 0; vt < VC; ++vt) {
        const s16x4_t vf = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(vbase + vt * 16));
        o[vt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vf, pf[ks], o[vt], 0, 0, 0);
      }
    }
  }
  if (!valid) return;
#pragma unroll
  for (int vt = 0; vt < VC; ++vt)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int v = vt * 16 + 4 * lg + c;
      if (v >= dv) continue;
      if (splits == 1)
        st(out + (size_t)tok * ld_out + (size_t)head * dv + v, o[vt][c] * out_scale);
      else
        part[((size_t)z * total_q + tok) * H * dv + (size_t)head * dv + v] = o[vt][c];
    }
}

template <typename T>
__global__ __launch_bounds__(256) void sigmoid_merge_kernel(T* __restrict__ out, int64_t ld_out, const float* __restrict__ part, int total_q,
                                                            int no, int splits, float out_scale) {
  const size_t t = blockIdx.x;
  for (int o = threadIdx.x; o < no; o += 256) {
    float v = 0.f;
    for (int s = 0; s < splits; ++s) v += part[((size_t)s * total_q + t) * no + o];
    st(out + t * ld_out + o, v * out_scale);
  }
}

// ------------------------------------------------------------------------------------------------ state-space recurrence
// Workgroup = (block of 64 value columns, head, request or chunk), 4 waves; lane = column e of the head's state S [N, P], wave w
// owns rows w R .. w R + R - 1 of that column in registers (4 R >= N, the tail zero).  Per token:
//   dt = softplus(dt_raw + dt_bias[h]);  a = exp(rate[h] dt);  S <- a S + (dt x_e) B;  y_e = S . C + D[h] x_e
// (the four waves' partial dot products are added in wave order).  Rows xbc = [x: H x P | B: G x N | C: G x N] (fp32); the B and C
// entries a wave needs are the same for all its lanes and are read through uniform addresses.  16 tokens are staged at a time.
// MODE 0  a request's whole portion from its state row (zero when the portion starts at position 0), state row written back.
// Long portions are cut into chunks that run in parallel; over a chunk S_end = A S_start + L with A = exp(rate * sum of dt).
// MODE 1  a chunk's L from zero and its sum of dt -> scratch[item], chunk_dt[item, h]; no outputs; the last chunk of a request is
//         skipped (nothing follows it).  ssd_scan_kernel then walks a request's chunks: start[c + 1] = A_c start[c] + L_c.
// MODE 2  a chunk's outputs from its start state (scratch[item] after the scan); the last chunk writes the state row.
template <typename T, int R, int MODE>
__global__ __launch_bounds__(256) void ssd_kernel(float* __restrict__ out, const float* __restrict__ xbc, int64_t ld_x, const T* __restrict__ dt_raw,
                                                  int64_t ld_dt, float* __restrict__ state, const float* __restrict__ rate,
                                                  const float* __restrict__ dt_bias, const float* __restrict__ Dv, const int* __restrict__ cu_q,
                                                  const int* __restrict__ seq_lens, const int* __restrict__ slots, int H, int G, int N, int P,
                                                  const int* __restrict__ items, const int* __restrict__ item_first, float* __restrict__ scratch,
                                                  float* __restrict__ chunk_dt) {
  constexpr int kStage = 16;
  __shared__ float sx[kStage][64], sdt[kStage], sa[kStage], part[kStage][4][64];
  const int h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, e = blockIdx.x * 64 + lane;
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
  const int grp = h / (H / G), row0 = wave * R;
  const bool live = e < P;
  float S[R];
  if (MODE == 1) {
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = 0.f;
  } else {
    const bool fresh = MODE == 0 && seq_lens[b] == n_new;
    const float* Srow = MODE == 0 ? state + ((size_t)slots[b] * H + h) * N * P : scratch + ((size_t)blockIdx.z * H + h) * N * P;
#pragma unroll
    for (int i = 0; i < R; ++i) S[i] = (!fresh && live && row0 + i < N) ? Srow[(size_t)(row0 + i) * P + e] : 0.f;
  }
  const float r = rate[h], dskip = Dv[h], db = dt_bias[h];
  const size_t no = (size_t)H * P;
  const bool full = row0 + R <= N;  // uniform over the wave
  float dt_sum = 0.f;
  for (int t0 = 0; t0 < n_new; t0 += kStage) {
    const int nt = n_new - t0 < kStage ? n_new - t0 : kStage;
    __syncthreads();
    if (threadIdx.x < nt) {
      const float dt = softplusf_(ld(dt_raw + (size_t)(first + t0 + threadIdx.x) * ld_dt + h) + db);
      sdt[threadIdx.x] = dt;
      sa[threadIdx.x] = expf(r * dt);
    }
    for (int tt = wave; tt < nt; tt += 4) sx[tt][lane] = live ? xbc[(size_t)(first + t0 + tt) * ld_x + (size_t)h * P + e] : 0.f;
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float* __restrict__ Bp = xbc + (size_t)(first + t0 + tt) * ld_x + (size_t)H * P + (size_t)grp * N + row0;
      const float* __restrict__ Cp = Bp + (size_t)G * N;
      const float a = sa[tt], u = sdt[tt] * sx[tt][lane];
      if (MODE == 1) dt_sum += sdt[tt];
      float y = 0.f;
      if (full) {
#pragma unroll
        for (int i = 0; i < R; ++i) {
          S[i] = fmaf(a, S[i], u * Bp[i]);
          if (MODE != 1) y = fmaf(S[i], Cp[i], y);
        }
      } else {
#pragma unroll
        for (int i = 0; i < R; ++i) {
          if (row0 + i < N) {
            S[i] = fmaf(a, S[i], u * Bp[i]);
            if (MODE != 1) y = fmaf(S[i], Cp[i], y);
          }
        }
      }
      if (MODE != 1) part[tt][wave][lane] = y;
    }
    if (MODE == 1) continue;
    __syncthreads();
    for (int tt = wave; tt < nt; tt += 4) {
      const float y = ((part[tt][0][lane] + part[tt][1][lane]) + part[tt][2][lane]) + part[tt][3][lane];
      if (live) out[(size_t)(first + t0 + tt) * no + (size_t)h * P + e] = fmaf(dskip, sx[tt][lane], y);
    }
  }
  if (MODE == 1) {
    float* L = scratch + ((size_t)blockIdx.z * H + h) * N * P;
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (live && row0 + i < N) L[(size_t)(row0 + i) * P + e] = S[i];
    if (blockIdx.x == 0 && threadIdx.x == 0) chunk_dt[(size_t)blockIdx.z * H + h] = dt_sum;
  } else if (last_chunk) {
    float* Srow = state + ((size_t)slots[b] * H + h) * N * P;
#pragma unroll
    for (int i = 0; i < R; ++i)
      if (live && row0 + i < N) Srow[(size_t)(row0 + i) * P + e] = S[i];
  }
}

// Per state element, walk a request's chunks in order: scratch[item] holds the chunk's own contribution L on entry (nothing for
// the last chunk) and the state BEFORE the chunk on exit.
__global__ __launch_bounds__(256) void ssd_scan_kernel(const float* __restrict__ state, float* __restrict__ scratch,
                                                       const float* __restrict__ chunk_dt, const float* __restrict__ rate,
                                                       const int* __restrict__ cu_q, const int* __restrict__ seq_lens,
                                                       const int* __restrict__ slots, const int* __restrict__ item_first, int H, int dd) {
  const int hh = blockIdx.x, b = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  const int i0 = item_first[b], i1 = item_first[b + 1];
  if (e >= dd || i0 >= i1) return;
  const int n = cu_q[b + 1] - cu_q[b];
  float cur = (seq_lens[b] - n == 0) ? 0.f : state[((size_t)slots[b] * H + hh) * dd + e];
  const float r = rate[hh];
  for (int i = i0; i < i1; ++i) {
    float* u = scratch + ((size_t)i * H + hh) * dd + e;
    const float add = i + 1 < i1 ? *u : 0.f;
    *u = cur;
    if (i + 1 < i1) cur = fmaf(expf(r * chunk_dt[(size_t)i * H + hh]), cur, add);
  }
}

// ------------------------------------------------------------------------------------------------ gate, then grouped norm
// One workgroup per token: v = y * silu(z); every one of `groups` equal parts of the row is divided by its own root mean square;
// out = v * w * out_scale in T (rows `ld_out` apart: the output may be a column block of a wider buffer).
template <typename T>
__global__ __launch_bounds__(256) void gate_group_norm_kernel(T* __restrict__ out, int64_t ld_out, const float* __restrict__ y,
                                                              const T* __restrict__ z, int64_t ld_z, const float* __restrict__ w, float eps,
                                                              int N, int groups, float out_scale) {
  extern __shared__ float v[];  // N + groups
  float* inv = v + N;
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < N; i += 256) v[i] = y[(size_t)t * N + i] * siluf_(ld(z + (size_t)t * ld_z + i));
  __syncthreads();
  const int per = N / groups;
  for (int g = wave; g < groups; g += 4) {
    float ss = 0.f;
    for (int i = lane; i < per; i += 64) ss = fmaf(v[g * per + i], v[g * per + i], ss);
    ss = wave_sum(ss);
    if (lane == 0) inv[g] = out_scale / sqrtf(ss / (float)per + eps);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < N; i += 256) st(out + (size_t)t * ld_out + i, v[i] * inv[i / per] * w[i]);
}

// ------------------------------------------------------------------------------------------------ activation
// A thread takes 8 consecutive elements of a row (16-byte loads when `vec`), so the two softplus of the layer's numbers are paid once
// per 8 elements.
template <typename T>
__global__ __launch_bounds__(256) void xielu_kernel(T* __restrict__ out, const T* __restrict__ z, int64_t ldz, const float* __restrict__ pq,
                                                    int64_t groups, int N, int vec) {
  const int64_t gi = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (gi >= groups) return;
  const int per_row = (N + 7) >> 3;
  const int64_t r = gi / per_row;
  const int c0 = (int)(gi - r * per_row) << 3, n = N - c0 < 8 ? N - c0 : 8;
  const float a = softplusf_(pq[0]), bneg = 0.5f + softplusf_(pq[1]);
  const T* src = z + r * ldz + c0;
  T* dst = out + r * N + c0;
  float x[8];
  if (vec && n == 8) {
    read8(src, x);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = i < n ? ld(src + i) : 0.f;
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float v = x[i] > 0.f ? fmaf(a * x[i], x[i], 0.5f * x[i]) : fmaf(bneg, expm1f(x[i]) - x[i], 0.5f * x[i]);
    if (i < n) st(dst + i, v);
  }
}

}  // namespace

extern "C" {

int msgl_mix_embed_scaled(float* x32, const void* table, const void* pair, const int* ids, const int* positions, const int* cu_q,
                          const int* req_rows, int batch, const int* prev_tok, float scale, int buckets, int mul_prev, int mul_cur,
                          int tokens, int W, int dtype, void* stream) {
  MIX_REQUIRE(x32 && table && ids && tokens >= 0 && W >= 1 && dtype_ok(dtype), "embed_scaled: bad arguments");
  MIX_REQUIRE(!pair || (positions && cu_q && req_rows && prev_tok && batch >= 1 && buckets >= 1),
              "embed_scaled: a pair table needs positions, requests, the previous-token rows and buckets >= 1");
  if (tokens == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(embed_scaled_kernel<T>, dim3(tokens), dim3(256), 0, s, x32, cp<T>(table), cp<T>(pair), ids, positions,
                                       cu_q, req_rows, batch, prev_tok, scale, buckets, mul_prev, mul_cur, W);)
  MIX_LAUNCHED("embed_scaled");
  return MSGL_MIX_OK;
}

int msgl_mix_shift_norm(const float* x_in, float* x_out, const void* y0, int64_t ld0, const float* v0, const void* y1, int64_t ld1,
                        const float* v1, const float* bias, const float* w, float w_off, const float* shift, void* h_out, void* g_out,
                        const float* state, float* staging, const int* positions, const int* cu_q, const int* req_rows, int batch,
                        float eps, int rows, int W, int dtype, void* stream) {
  MIX_REQUIRE(x_in && w && rows >= 0 && W >= 1 && dtype_ok(dtype), "shift_norm: bad arguments");
  MIX_REQUIRE(x_out != x_in, "shift_norm: the summed rows may not replace their input (a token re-reads the row before it)");
  MIX_REQUIRE((!y0 || ld0 >= W) && (!y1 || ld1 >= W), "shift_norm: part rows shorter than the width");
  MIX_REQUIRE(x_out || (!y0 && !y1 && !bias), "shift_norm: parts without a place for the sum");
  if (shift) {
    MIX_REQUIRE(g_out && state && staging && positions && cu_q && req_rows && batch >= 1, "shift_norm: a shift needs g_out, state and requests");
  } else {
    MIX_REQUIRE(h_out, "shift_norm: nothing to write");
  }
  if (rows == 0) return MSGL_MIX_OK;
  const size_t lds = (size_t)2 * W * sizeof(float);
  // long batches: a workgroup takes 2 consecutive tokens and re-reads one row in two instead of every row (measured: 4 and 8
  // tokens per workgroup gain nothing more, the serial walk costs what the saved reads give); short ones keep a workgroup per
  // token (the arithmetic of a token is the same either way)
  const int TT = (shift && rows >= 1024) ? 2 : 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto al16 = [](const void* p) { return ((uintptr_t)p & 15u) == 0; };
  const int es = dtype == MSGL_MIX_BF16 ? 2 : 4;
  const bool vec = W % 8 == 0 && al16(w) && al16(shift) && al16(bias) && al16(v0) && al16(v1) && al16(state) && al16(x_in) && al16(x_out) && al16(h_out) && al16(g_out) && al16(staging) && al16(y0) && al16(y1) &&
                   (!y0 || (ld0 * es) % 16 == 0) && (!y1 || (ld1 * es) % 16 == 0);
#define SN_LAUNCH(VEC)                                                                                                                          \
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)shift_norm_kernel<T, VEC>, lds) == 0, "shift_norm: two rows of %d do not fit LDS", W); \
             hipLaunchKernelGGL((shift_norm_kernel<T, VEC>), dim3((rows + TT - 1) / TT), dim3(256), lds, s, x_in, x_out, cp<T>(y0), ld0, v0,    \
                                cp<T>(y1), ld1, v1, bias, w, w_off, shift, mp<T>(h_out), mp<T>(g_out), state, staging, positions, cu_q,         \
                                req_rows, batch, eps, W, rows, TT);)
  if (vec) {
    SN_LAUNCH(true)
  } else {
    SN_LAUNCH(false)
  }
#undef SN_LAUNCH
  MIX_LAUNCHED("shift_norm");
  return MSGL_MIX_OK;
}

int msgl_mix_commit_rows(float* dst, int64_t dst_stride, const float* src, int64_t src_stride, int layers, const int* slots, int batch, int W,
                         int* prev_tok, const int* ids, const int* cu_q, void* stream) {
  MIX_REQUIRE(slots && cu_q && batch >= 0 && layers >= 0 && (layers == 0 || (dst && src && W >= 1)) && (!prev_tok || ids),
              "commit_rows: bad arguments");
  if (batch == 0 || (layers == 0 && !prev_tok)) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(commit_rows_kernel, dim3(batch, layers > 0 ? layers : 1), dim3(256), 0, s, layers > 0 ? dst : nullptr, dst_stride, src,
                     src_stride, slots, W, prev_tok, ids, cu_q);
  MIX_LAUNCHED("commit_rows");
  return MSGL_MIX_OK;
}

int msgl_mix_qk_prep(const void* proj, int64_t ld_proj, const float* bias, float* q_out, void* k_cache, void* v_cache, const int* out_loc,
                     const int* positions, const float* cos_sin, int rot_dims, int interleaved, int unit, float eps, int tokens, int H,
                     int G, int d, int dv, int dtype, void* stream) {
  MIX_REQUIRE(proj && q_out && k_cache && v_cache && out_loc && dtype_ok(dtype), "qk_prep: null pointer / dtype");
  MIX_REQUIRE(H >= 1 && G >= 1 && H % G == 0 && d >= 1 && dv >= 1 && rot_dims >= 0 && rot_dims <= d && rot_dims % 2 == 0,
              "qk_prep: bad sizes H %d G %d d %d dv %d rot %d", H, G, d, dv, rot_dims);
  MIX_REQUIRE(rot_dims == 0 || (cos_sin && positions), "qk_prep: a rotation needs its table and positions");
  MIX_REQUIRE(ld_proj >= (int64_t)(H + G) * d + (int64_t)G * dv, "qk_prep: projection row too short");
  if (tokens == 0) return MSGL_MIX_OK;
  const size_t lds = (size_t)(H + G) * d * sizeof(float);
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)qk_prep_kernel<T>, lds) == 0, "qk_prep: heads do not fit LDS");
             hipLaunchKernelGGL(qk_prep_kernel<T>, dim3(tokens), dim3(256), lds, s, cp<T>(proj), ld_proj, bias, q_out, mp<T>(k_cache),
                                mp<T>(v_cache), out_loc, positions, cos_sin, rot_dims, interleaved, unit, eps, H, G, d, dv);)
  MIX_LAUNCHED("qk_prep");
  return MSGL_MIX_OK;
}

int msgl_mix_sigmoid_attn_workspace_floats(int total_q, int H, int dv, int splits) { return splits > 1 ? total_q * H * dv * splits : 0; }

int msgl_mix_sigmoid_attn(void* out, int64_t ld_out, const float* q, const void* k_cache, const void* v_cache, const int* table,
                          int64_t table_stride, const int* req_rows, const int* seq_lens, const int* cu_q, int batch, int total_q, int H,
                          int G, int d, int dv, float scale, float softcap, const float* pb, float out_scale, int dtype, int splits,
                          float* workspace, void* stream) {
  MIX_REQUIRE(out && q && k_cache && v_cache && table && req_rows && seq_lens && cu_q && dtype_ok(dtype), "sigmoid_attn: null pointer / dtype");
  MIX_REQUIRE(batch >= 1 && total_q >= 0 && H >= 1 && G >= 1 && H % G == 0 && d >= 1 && dv >= 1 && dv <= 16 * kSigMaxC &&
                  ld_out >= (int64_t)H * dv,
              "sigmoid_attn: bad sizes H %d G %d d %d dv %d", H, G, d, dv);
  MIX_REQUIRE(splits >= 1 && splits <= 1024 && (splits == 1 || workspace), "sigmoid_attn: %d splits need a workspace", splits);
  if (total_q == 0) return MSGL_MIX_OK;
  const int rep = H / G;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == MSGL_MIX_BF16 && d <= 256 && dv <= 256) {
    // matrix-core kernel: the smallest (KC, VC) instance that holds d <= 32 KC and dv <= 16 VC
    int HBm = 1;
    while (HBm * 2 <= rep && HBm * 2 <= 64) HBm *= 2;
    const int QTm = 64 / HBm, hbl = (rep + HBm - 1) / HBm;
    const int groups_m = (total_q + QTm - 1) / QTm + batch;
    MIX_REQUIRE((int64_t)G * hbl <= 65535, "sigmoid_attn: too many heads");
    const dim3 grid(groups_m, G * hbl, splits);
    const int kvec = (((uintptr_t)k_cache & 15u) == 0 && d % 8 == 0) ? 1 : 0, vvec = (((uintptr_t)v_cache & 15u) == 0 && dv % 8 == 0) ? 1 : 0;
#define SIG_CASE(KC, VC)                                                                                                                  \
  if (d <= KC * 32 && dv <= VC * 16) {                                                                                                    \
    const size_t lds_m = (size_t)kSKT * ((KC * 32 + 8) + (VC * 16 + 8)) * sizeof(uint16_t);                                               \
    MIX_REQUIRE(ensure_lds((const void*)sigmoid_attn_mfma_kernel<KC, VC>, lds_m) == 0, "sigmoid_attn: LDS request refused");              \
    hipLaunchKernelGGL((sigmoid_attn_mfma_kernel<KC, VC>), grid, dim3(256), lds_m, s, mp<bf16_t>(out), ld_out, workspace, q,              \
                       cp<bf16_t>(k_cache), cp<bf16_t>(v_cache), table, table_stride, req_rows, seq_lens, cu_q, batch, total_q, H, G, d,  \
                       dv, scale, softcap, pb, out_scale, QTm, HBm, splits, kvec, vvec);                                                  \
    MIX_LAUNCHED("sigmoid_attn (matrix cores)");                                                                                          \
    if (splits > 1) {                                                                                                                     \
      hipLaunchKernelGGL(sigmoid_merge_kernel<bf16_t>, dim3(total_q), dim3(256), 0, s, mp<bf16_t>(out), ld_out, workspace, total_q,       \
                         H * dv, splits, out_scale);                                                                                      \
      MIX_LAUNCHED("sigmoid_attn merge");                                                                                                 \
    }                                                                                                                                     \
    return MSGL_MIX_OK;                                                                                                                   \
  }
    SIG_CASE(2, 4)
    SIG_CASE(3, 6)
    SIG_CASE(4, 8)
    SIG_CASE(6, 12)
    SIG_CASE(8, 16)
#undef SIG_CASE
  }
  int HB = 1;
  while (HB * 2 <= rep && HB * 2 <= kSigRows) HB *= 2;
  const int QT = kSigRows / HB, hblocks = (rep + HB - 1) / HB;
  int KT = 64;
  auto need = [&](int kt) { return (size_t)((kSigRows + kt) * (d + 1) + kt * (dv + 1) + kSigRows * kt) * sizeof(float); };
  while (KT > 8 && need(KT) > 160 * 1024) KT >>= 1;
  const size_t lds = need(KT);
  MIX_REQUIRE(lds <= 160 * 1024, "sigmoid_attn: heads of %d / %d do not fit LDS", d, dv);
  const int groups = (total_q + QT - 1) / QT + batch;  // every request may end with one partial group
  MIX_REQUIRE((int64_t)G * hblocks <= 65535, "sigmoid_attn: too many heads");
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)sigmoid_attn_kernel<T>, lds) == 0, "sigmoid_attn: LDS request refused");
             hipLaunchKernelGGL(sigmoid_attn_kernel<T>, dim3(groups, G * hblocks, splits), dim3(256), lds, s, mp<T>(out), ld_out, workspace, q,
                                cp<T>(k_cache), cp<T>(v_cache), table, table_stride, req_rows, seq_lens, cu_q, batch, total_q, H, G, d, dv,
                                scale, softcap, pb, out_scale, QT, HB, KT, splits);
             if (splits > 1) hipLaunchKernelGGL(sigmoid_merge_kernel<T>, dim3(total_q), dim3(256), 0, s, mp<T>(out), ld_out, workspace, total_q,
                                                H * dv, splits, out_scale);)
  MIX_LAUNCHED("sigmoid_attn");
  return MSGL_MIX_OK;
}

int msgl_mix_ssd(float* out, const float* xbc, int64_t ld_x, const void* dt_raw, int64_t ld_dt, float* state, const float* rate,
                 const float* dt_bias, const float* D, const int* cu_q, const int* seq_lens, const int* slots, int batch, int H, int G, int N,
                 int P, int dtype, int n_items, const int* items, const int* item_first, float* scratch, void* stream) {
  MIX_REQUIRE(out && xbc && dt_raw && state && rate && dt_bias && D && cu_q && seq_lens && slots && dtype_ok(dtype), "ssd: null pointer / dtype");
  MIX_REQUIRE(batch >= 0 && H >= 1 && G >= 1 && H % G == 0 && N >= 1 && N <= 256 && P >= 1, "ssd: bad sizes H %d G %d N %d P %d", H, G, N, P);
  MIX_REQUIRE(ld_x >= (int64_t)H * P + 2 * (int64_t)G * N && ld_dt >= H, "ssd: rows shorter than their heads");
  MIX_REQUIRE(n_items >= 0 && (n_items == 0 || (items && item_first && scratch)), "ssd: chunks without their lists / scratch");
  if (batch == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* chunk_dt = scratch ? scratch + (size_t)n_items * H * N * P : nullptr;
  const int cb = (P + 63) / 64;
#define SSD_GO(DP)                                                                                                                        \
  if (N <= DP) {                                                                                                                          \
    DISPATCH_T(dtype, if (n_items == 0) {                                                                                                 \
      hipLaunchKernelGGL((ssd_kernel<T, DP / 4, 0>), dim3(cb, H, batch), dim3(256), 0, s, out, xbc, ld_x, cp<T>(dt_raw), ld_dt, state, rate,   \
                         dt_bias, D, cu_q, seq_lens, slots, H, G, N, P, items, item_first, scratch, chunk_dt);                            \
    } else {                                                                                                                              \
      hipLaunchKernelGGL((ssd_kernel<T, DP / 4, 1>), dim3(cb, H, n_items), dim3(256), 0, s, out, xbc, ld_x, cp<T>(dt_raw), ld_dt, state, rate, \
                         dt_bias, D, cu_q, seq_lens, slots, H, G, N, P, items, item_first, scratch, chunk_dt);                            \
      hipLaunchKernelGGL(ssd_scan_kernel, dim3(H, batch, (N * P + 255) / 256), dim3(256), 0, s, state, scratch, chunk_dt, rate, cu_q,     \
                         seq_lens, slots, item_first, H, N * P);                                                                          \
      hipLaunchKernelGGL((ssd_kernel<T, DP / 4, 2>), dim3(cb, H, n_items), dim3(256), 0, s, out, xbc, ld_x, cp<T>(dt_raw), ld_dt, state, rate, \
                         dt_bias, D, cu_q, seq_lens, slots, H, G, N, P, items, item_first, scratch, chunk_dt);                            \
    })                                                                                                                                    \
    MIX_LAUNCHED("ssd");                                                                                                                  \
    return MSGL_MIX_OK;                                                                                                                   \
  }
  SSD_GO(16)
  SSD_GO(32)
  SSD_GO(64)
  SSD_GO(128)
  SSD_GO(256)
#undef SSD_GO
  return MSGL_MIX_EINVAL;
}

int msgl_mix_gate_group_norm(void* out, int64_t ld_out, const float* y, const void* z, int64_t ld_z, const float* w, float eps, int rows,
                             int N, int groups, float out_scale, int dtype, void* stream) {
  MIX_REQUIRE(out && y && z && w && rows >= 0 && N >= 1 && groups >= 1 && N % groups == 0 && ld_out >= N && ld_z >= N && dtype_ok(dtype),
              "gate_group_norm: bad arguments (N %d groups %d)", N, groups);
  if (rows == 0) return MSGL_MIX_OK;
  const size_t lds = (size_t)(N + groups) * sizeof(float);
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)gate_group_norm_kernel<T>, lds) == 0, "gate_group_norm: row of %d does not fit LDS", N);
             hipLaunchKernelGGL(gate_group_norm_kernel<T>, dim3(rows), dim3(256), lds, s, mp<T>(out), ld_out, y, cp<T>(z), ld_z, w, eps, N,
                                groups, out_scale);)
  MIX_LAUNCHED("gate_group_norm");
  return MSGL_MIX_OK;
}

int msgl_mix_xielu(void* out, const void* z, int64_t ldz, const float* pq, int rows, int N, int dtype, void* stream) {
  MIX_REQUIRE(out && z && pq && rows >= 0 && N >= 1 && ldz >= N && dtype_ok(dtype), "xielu: bad arguments");
  if (rows == 0) return MSGL_MIX_OK;
  const int64_t groups = (int64_t)rows * ((N + 7) / 8);
  const int es = dtype == MSGL_MIX_BF16 ? 2 : 4;
  const int vec = (N % 8 == 0 && ldz % 8 == 0 && ((uintptr_t)z & 15u) == 0 && (es == 2 || ((uintptr_t)z & 31u) == 0)) ? 1 : 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  DISPATCH_T(dtype, hipLaunchKernelGGL(xielu_kernel<T>, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s, mp<T>(out), cp<T>(z), ldz, pq,
                                       groups, N, vec);)
  MIX_LAUNCHED("xielu");
  return MSGL_MIX_OK;
}

}  // extern "C"
