// Kernels of the looped pre-norm hybrid decoders (grouped norms, a short causal convolution in front of every sublayer,
// mixers: gated latent attention, a selective-scan state-space layer, windowed attention with a sink and normed values;
// experts that are weighted on their input), gfx950, wave = 64 lanes.  Fourth translation unit of libmsgl_mix.so; C ABI in
// include/msgl_mix.h.
//
// Precision rules (as in seqmix.hip): the residual stream, every norm, rotary angles, attention scores and weights, step
// sizes, decays and the recurrent state are fp32 in registers and in memory; tensors that feed a matrix product are stored in
// the model dtype T (bf16 or fp32).  With T = float every kernel here is true 32-bit.
//
//   norm_conv_kernel        closes a sublayer and opens the next: x' = x + mult * sum of parts (+ a vector); h = x' normed in equal
//                           groups of the row, times w; out = h + sum_j taps[., j] h[t - (n - 1) + j] (inputs before the portion from
//                           the request's state rows, inside the portion recomputed by the workgroup that needs them); the last
//                           n - 1 inputs of every request -> staging rows (msgl_mix_commit_rows moves them after the forward)
//   selective_scan_kernel   S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;  y_c = sum_n S[c, n] C_n + D_c x_c;  out = y silu(z);
//                           a thread owns one channel's state row in registers; long portions as parallel chunks joined by
//                           selective_join_kernel
//   sink_attn_mfma_kernel   softmax attention over the last `window` keys with one more term exp(sink_h) in the denominator; bf16
//                           caches, both products on the matrix cores, fp32 online softmax; key ranges + sink_merge_kernel
//   sink_attn_kernel        the same in plain fp32 (fp32 caches, heads past the matrix-core instances)
//   route_sigmoid_kernel    the `top` largest router logits win, weights = sigmoid(logit)
//   scale_rows_kernel       one copy of a token's row per chosen expert, multiplied by that choice's weight
//   route_scale_kernel      logits, choice and scaled rows of a token in one launch (steps with few tokens)
//   sigmoid_gate_kernel     out = o * sigmoid(g)
//   softcap_kernel          x <- cap tanh(x / cap)
#include "mix_common.h"

namespace {

__device__ __forceinline__ float sigmoidf_(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplusf_(float z) { return z > 20.0f ? z : log1pf(expf(z)); }
// the decay of a state element: the library's exponential in a 32-bit engine, the hardware's in a 16-bit one
__device__ __forceinline__ float decay_exp(float z, const float*) { return expf(z); }
__device__ __forceinline__ float decay_exp(float z, const bf16_t*) { return __expf(z); }
// the same split for the scan's step size and gate (once per token and channel, but inside the serial walk)
__device__ __forceinline__ float scan_softplus(float z, const float*) { return softplusf_(z); }
__device__ __forceinline__ float scan_softplus(float z, const bf16_t*) {
  return z > 20.0f ? z : (z < -15.0f ? __expf(z) : __logf(1.0f + __expf(z)));
}
__device__ __forceinline__ float scan_silu(float z, const float*) { return siluf_(z); }
__device__ __forceinline__ float scan_silu(float z, const bf16_t*) { return z * __builtin_amdgcn_rcpf(1.0f + __expf(-z)); }

// ------------------------------------------------------------------------------------------------ residual sum + grouped norm + input convolution
// A workgroup owns TB consecutive new tokens of ONE request (cu_q given) or TB consecutive rows (cu_q null: no convolution over
// time, n = 1).  It walks them in order and keeps the last n normed rows in LDS; a thread owns the columns c = tid + 256 k of
// every row, so the rows of the ring are private to it and only the group statistics need the workgroup.  Rows before the
// workgroup's first token: inside the portion they are recomputed (same arithmetic, same order: bit-equal to what their own
// workgroup stores), before the portion they are the request's state rows (state[slot][s] = the normed row at position start -
// (n - 1) + s), before position 0 they are zero.  The workgroup that holds a request's last new token leaves the request's
// new state rows in staging[b]; the state itself is replaced after the forward, because first and last tokens of a portion run
// concurrently.
template <typename T>
__global__ __launch_bounds__(256) void norm_conv_kernel(const float* __restrict__ x_in, float* __restrict__ x_out, const T* __restrict__ y0,
                                                        int p0, const T* __restrict__ y1, int p1, float mult, const float* __restrict__ add,
                                                        const T* __restrict__ w, int groups, float eps, const T* __restrict__ taps, int n,
                                                        const float* __restrict__ state, float* __restrict__ staging, T* __restrict__ h_out,
                                                        const int* __restrict__ cu_q, const int* __restrict__ seq_lens,
                                                        const int* __restrict__ slots, int B, int rows, int W, int TB) {
  extern __shared__ float lds[];
  float* ring = lds;                       // [n][W]
  float* inv = lds + (size_t)n * W;        // [groups]
  __shared__ int s_req, s_tok0, s_cnt[256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int b = 0, tok_first = 0, q_len = rows, start = 0, tl0 = blockIdx.x * TB;
  if (cu_q) {
    find_group(cu_q, B, TB, s_cnt, &s_req, &s_tok0);
    b = s_req;
    if (b < 0) return;
    tok_first = cu_q[b];
    q_len = cu_q[b + 1] - tok_first;
    start = seq_lens[b] - q_len;
    tl0 = s_tok0;
  }
  const int gw = W / groups;
  const int i_begin = -(n - 1);
  const size_t slot = cu_q && n > 1 ? (size_t)slots[b] : 0;
  for (int i = i_begin; i < TB; ++i) {
    const int tl = tl0 + i;
    if (tl >= q_len) break;
    float* cur = ring + (size_t)((i - i_begin) % n) * W;
    if (tl < 0) {  // before the portion: the request's state rows (zero before the sequence)
      const bool have = start + tl >= 0;
      const float* src = state + (slot * (n - 1) + (size_t)(n - 1 + tl)) * W;
      for (int c = tid; c < W; c += 256) cur[c] = have ? src[c] : 0.f;
      continue;
    }
    const size_t t = (size_t)tok_first + tl;
    for (int c = tid; c < W; c += 256) {
      float acc = 0.f;
      for (int p = 0; p < p0; ++p) acc += ld(y0 + (t * p0 + p) * W + c);
      for (int p = 0; p < p1; ++p) acc += ld(y1 + (t * p1 + p) * W + c);
      float s = x_in[t * W + c];
      if (p0 + p1 > 0) s = fmaf(mult, acc, s);
      if (add) s += add[c];
      if (i >= 0 && x_out) x_out[t * W + c] = s;
      cur[c] = s;
    }
    __syncthreads();
    for (int g = wave; g < groups; g += 4) {
      float ss = 0.f;
      for (int k = lane; k < gw; k += 64) ss = fmaf(cur[g * gw + k], cur[g * gw + k], ss);
      ss = wave_sum(ss);
      if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)gw + eps);
    }
    __syncthreads();
    for (int c = tid; c < W; c += 256) {
      const float h = cur[c] * inv[c / gw] * ld(w + c);
      cur[c] = h;
      if (i < 0) continue;
      float o = h;
      if (taps) {
        for (int j = 0; j < n; ++j) {
          const int back = n - 1 - j;
          o = fmaf(ld(taps + (size_t)c * n + j), ring[(size_t)((i - back - i_begin) % n) * W + c], o);
        }
      }
      st(h_out + t * W + c, o);
    }
    if (staging && n > 1 && tl == q_len - 1) {  // the request's new state rows: the inputs at local indices q_len - (n - 1) + s
      for (int s = 0; s < n - 1; ++s) {
        const int li = q_len - (n - 1) + s;
        const float* src = ring + (size_t)((li - tl0 - i_begin) % n) * W;
        float* dst = staging + ((size_t)b * (n - 1) + s) * W;
        for (int c = tid; c < W; c += 256) dst[c] = src[c];
      }
    }
  }
}

// The same with 16-byte accesses and the ring in registers, for rows whose width and groups are multiples of 8 and at most NT <= 4 taps:
// a thread owns NCH chunks of 8 consecutive columns (chunk j * 256 + tid), ring[NT - 1] is the current row, ring[k] the row NT - 1 - k
// tokens before; LDS only carries the chunks' sums of squares to the waves that add up a group.
template <typename T, int NCH, int NT>
__global__ __launch_bounds__(256) void norm_conv_vec_kernel(const float* __restrict__ x_in, float* __restrict__ x_out, const T* __restrict__ y0,
                                                            int p0, const T* __restrict__ y1, int p1, float mult, const float* __restrict__ add,
                                                            const T* __restrict__ w, int groups, float eps, const T* __restrict__ taps,
                                                            const float* __restrict__ state, float* __restrict__ staging,
                                                            T* __restrict__ h_out, const int* __restrict__ cu_q,
                                                            const int* __restrict__ seq_lens, const int* __restrict__ slots, int B, int rows,
                                                            int W, int TB) {
  extern __shared__ float lds[];
  const int nchunks = W >> 3;
  float* part = lds;            // [W / 8]
  float* inv = lds + nchunks;   // [groups]
  __shared__ int s_req, s_tok0, s_cnt[256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  int b = 0, tok_first = 0, q_len = rows, start = 0, tl0 = blockIdx.x * TB;
  if (cu_q) {
    find_group(cu_q, B, TB, s_cnt, &s_req, &s_tok0);
    b = s_req;
    if (b < 0) return;
    tok_first = cu_q[b];
    q_len = cu_q[b + 1] - tok_first;
    start = seq_lens[b] - q_len;
    tl0 = s_tok0;
  }
  const int cpg = (W / groups) >> 3;  // chunks per group
  const size_t slot = cu_q && NT > 1 ? (size_t)slots[b] : 0;
  float ring[NT][NCH][8];
#pragma unroll
  for (int k = 0; k < NT; ++k)
#pragma unroll
    for (int j = 0; j < NCH; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) ring[k][j][e] = 0.f;
  for (int i = -(NT - 1); i < TB; ++i) {
    const int tl = tl0 + i;
    if (tl >= q_len) break;
#pragma unroll
    for (int k = 0; k + 1 < NT; ++k)
#pragma unroll
      for (int j = 0; j < NCH; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) ring[k][j][e] = ring[k + 1][j][e];
    if (tl < 0) {  // before the portion: the request's state rows (zero before the sequence)
      const bool have = start + tl >= 0;
      const float* src = state + (slot * (NT - 1) + (size_t)(NT - 1 + tl)) * W;
#pragma unroll
      for (int j = 0; j < NCH; ++j) {
        const int ch = j * 256 + tid;
        if (ch < nchunks && have) {
          read8(src + ch * 8, ring[NT - 1][j]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) ring[NT - 1][j][e] = 0.f;
        }
      }
      continue;
    }
    const size_t t = (size_t)tok_first + tl;
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int ch = j * 256 + tid;
      if (ch >= nchunks) continue;
      const size_t c0 = (size_t)ch * 8;
      float acc[8], v[8], s[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = 0.f;
      for (int p = 0; p < p0; ++p) {
        read8(y0 + (t * p0 + p) * W + c0, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += v[e];
      }
      for (int p = 0; p < p1; ++p) {
        read8(y1 + (t * p1 + p) * W + c0, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += v[e];
      }
      read8(x_in + t * W + c0, s);
      if (p0 + p1 > 0) {
#pragma unroll
        for (int e = 0; e < 8; ++e) s[e] = fmaf(mult, acc[e], s[e]);
      }
      if (add) {
        read8(add + c0, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) s[e] += v[e];
      }
      if (i >= 0 && x_out) write8(x_out + t * W + c0, s);
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ss = fmaf(s[e], s[e], ss);
        ring[NT - 1][j][e] = s[e];
      }
      part[ch] = ss;
    }
    __syncthreads();
    for (int g = wave; g < groups; g += 4) {
      float ss = 0.f;
      for (int k = lane; k < cpg; k += 64) ss += part[g * cpg + k];
      ss = wave_sum(ss);
      if (lane == 0) inv[g] = 1.0f / sqrtf(ss / (float)(cpg * 8) + eps);
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NCH; ++j) {
      const int ch = j * 256 + tid;
      if (ch >= nchunks) continue;
      const size_t c0 = (size_t)ch * 8;
      float wv[8], o[8];
      read8(w + c0, wv);
      const float f = inv[ch / cpg];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        ring[NT - 1][j][e] = ring[NT - 1][j][e] * f * wv[e];
        o[e] = ring[NT - 1][j][e];
      }
      if (i < 0) continue;
      if (taps) {
        float tv[NT][8];  // the chunk's taps: element c * NT + k of 8 NT consecutive numbers
#pragma unroll
        for (int k = 0; k < NT; ++k) read8(taps + c0 * NT + k * 8, tv[k]);
#pragma unroll
        for (int e = 0; e < 8; ++e)
#pragma unroll
          for (int k = 0; k < NT; ++k) o[e] = fmaf(tv[(e * NT + k) >> 3][(e * NT + k) & 7], ring[k][j][e], o[e]);
      }
      write8(h_out + t * W + c0, o);
    }
    if (staging && NT > 1 && tl == q_len - 1) {  // the request's new state rows: the rows NT - 1 .. 1 tokens back = ring[1 ..]
#pragma unroll
      for (int s = 0; s + 1 < NT; ++s)
#pragma unroll
        for (int j = 0; j < NCH; ++j) {
          const int ch = j * 256 + tid;
          if (ch < nchunks) write8(staging + ((size_t)b * (NT - 1) + s) * W + (size_t)ch * 8, ring[s + 1][j]);
        }
    }
  }
}

// ------------------------------------------------------------------------------------------------ selective scan
// Thread = channel c, its state row S[c, 0 : N] in NP registers (the tail unused).  Workgroup = 256 channels x (request or chunk).
// Per token: dt = softplus(dt_in[t, c] + dt_bias[c]);  S[n] <- exp(dt A[c, n]) S[n] + dt x[t, c] B[t, n];  y = sum_n S[n] C[t, n] +
// D[c] x[t, c];  out[t, c] = y silu(z[t, c]).  B and C of up to 16 tokens at a time go through LDS (every channel reads the same).
// MODE 0  a request's whole portion from its state row (zero when the portion starts at position 0), state row written back.
// Long portions are cut into chunks that run in parallel; over a chunk S_end = exp(A sum dt) S_start + L:
// MODE 1  a chunk's L (from zero) and sum dt -> scratch, no outputs (a request's last chunk is skipped: nothing follows it);
//         selective_join_kernel walks a request's chunks and leaves every chunk's start state where its L was;
// MODE 2  a chunk's outputs from its start state; the last chunk of a request writes the state row.

template <typename T, int NP, int MODE>
__global__ __launch_bounds__(256) void selective_scan_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t ld_x, const T* __restrict__ z,
                                                             int64_t ld_z, const T* __restrict__ dt_in, int64_t ld_dt,
                                                             const T* __restrict__ bc, int64_t ld_bc, const float* __restrict__ A,
                                                             const float* __restrict__ dt_bias, const float* __restrict__ D,
                                                             float* __restrict__ state, const int* __restrict__ cu_q,
                                                             const int* __restrict__ seq_lens, const int* __restrict__ slots, int C, int N,
                                                             const int* __restrict__ items, const int* __restrict__ item_first,
                                                             float* __restrict__ scratch, int n_items) {
  constexpr int kScanStage = NP <= 32 ? 16 : (NP <= 64 ? 8 : 4);  // tokens staged at a time (the walk over a stage is unrolled)
  __shared__ float sB[kScanStage][NP], sC[kScanStage][NP];
  const int c = blockIdx.x * 256 + threadIdx.x;
  const bool live = c < C;
  int b, first, n_new, it = 0;
  bool last_chunk = true;
  if (MODE == 0) {
    b = blockIdx.y;
    first = cu_q[b];
    n_new = cu_q[b + 1] - first;
  } else {
    it = blockIdx.y;
    b = items[3 * it];
    first = cu_q[b] + items[3 * it + 1];
    n_new = items[3 * it + 2] - items[3 * it + 1];
    last_chunk = it == item_first[b + 1] - 1;
    if (MODE == 1 && last_chunk) return;
  }
  if (n_new <= 0) return;
  const int q_len = cu_q[b + 1] - cu_q[b];
  const bool from_zero = seq_lens[b] - q_len == 0;
  float S[NP], a[NP];
  float* srow = state + ((size_t)slots[b] * C + (live ? c : 0)) * N;
  float* lrow = scratch + ((size_t)it * C + (live ? c : 0)) * N;
  const float* init = MODE == 2 ? lrow : ((MODE == 0 && !from_zero) ? srow : nullptr);
  if (N == NP && live) {  // whole rows: 16-byte loads
#pragma unroll
    for (int k = 0; k < NP; k += 4) {
      const float4 av = *reinterpret_cast<const float4*>(A + (size_t)c * N + k);
      const float4 sv = init ? *reinterpret_cast<const float4*>(init + k) : float4{0.f, 0.f, 0.f, 0.f};
      a[k] = av.x, a[k + 1] = av.y, a[k + 2] = av.z, a[k + 3] = av.w;
      S[k] = sv.x, S[k + 1] = sv.y, S[k + 2] = sv.z, S[k + 3] = sv.w;
    }
  } else {
#pragma unroll
    for (int k = 0; k < NP; ++k) {
      a[k] = (live && k < N) ? A[(size_t)c * N + k] : 0.f;
      S[k] = (live && k < N && init) ? init[k] : 0.f;
    }
  }
  const float bias = live ? dt_bias[c] : 0.f, skip = live ? D[c] : 0.f;
  float sumdt = 0.f;
  for (int t0 = 0; t0 < n_new; t0 += kScanStage) {
    const int nt = min(kScanStage, n_new - t0);
    // the stage's own inputs of this channel: all loads in flight together, not one token's at a time inside the serial walk
    float dtv[kScanStage], xv[kScanStage], zv[kScanStage];
#pragma unroll
    for (int tt = 0; tt < kScanStage; ++tt) {
      dtv[tt] = xv[tt] = zv[tt] = 0.f;
      if (tt < nt && live) {
        const size_t t = (size_t)first + t0 + tt;
        dtv[tt] = ld(dt_in + t * ld_dt + c);
        xv[tt] = ld(x + t * ld_x + c);
        if (MODE != 1) zv[tt] = ld(z + t * ld_z + c);
      }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < nt * N; e += 256) {
      const int tt = e / N, k = e - tt * N;
      const T* row = bc + (size_t)(first + t0 + tt) * ld_bc;
      sB[tt][k] = ld(row + k);
      sC[tt][k] = ld(row + N + k);
    }
    __syncthreads();
    if (!live) continue;
#pragma unroll
    for (int tt = 0; tt < kScanStage; ++tt) {
      if (tt < nt) {
        const float dt = scan_softplus(dtv[tt] + bias, x);
        const float dx = dt * xv[tt];
        float y = 0.f;
#pragma unroll
        for (int k = 0; k < NP; ++k) {
          if (k < N) {
            S[k] = fmaf(decay_exp(dt * a[k], x), S[k], dx * sB[tt][k]);
            y = fmaf(S[k], sC[tt][k], y);
          }
        }
        if (MODE == 1) {
          sumdt += dt;
        } else {
          y = fmaf(skip, xv[tt], y);
          st(out + ((size_t)first + t0 + tt) * C + c, y * scan_silu(zv[tt], x));
        }
      }
    }
  }
  if (!live) return;
  float* dst = MODE == 1 ? lrow : (last_chunk ? srow : nullptr);
  if (MODE == 1) scratch[(size_t)n_items * C * N + (size_t)it * C + c] = sumdt;
  if (!dst) return;
  if (N == NP) {
#pragma unroll
    for (int k = 0; k < NP; k += 4) *reinterpret_cast<float4*>(dst + k) = float4{S[k], S[k + 1], S[k + 2], S[k + 3]};
  } else {
#pragma unroll
    for (int k = 0; k < NP; ++k)
      if (k < N) dst[k] = S[k];
  }
}

// Thread = (request, one state element e = c * N + k): start state of every chunk of the request, written over the chunk's L.
__global__ __launch_bounds__(256) void selective_join_kernel(const float* __restrict__ state, float* __restrict__ scratch,
                                                             const float* __restrict__ A, const int* __restrict__ cu_q,
                                                             const int* __restrict__ seq_lens, const int* __restrict__ slots,
                                                             const int* __restrict__ item_first, int C, int N, int n_items) {
  const int b = blockIdx.y;
  const size_t e = (size_t)blockIdx.x * 256 + threadIdx.x, CN = (size_t)C * N;
  if (e >= CN) return;
  const int i0 = item_first[b], i1 = item_first[b + 1];
  if (i1 <= i0) return;
  const bool from_zero = seq_lens[b] - (cu_q[b + 1] - cu_q[b]) == 0;
  const float a = A[e];
  float S = from_zero ? 0.f : state[(size_t)slots[b] * CN + e];
  const float* sd = scratch + (size_t)n_items * CN + e / N;
  float L = scratch[(size_t)i0 * CN + e], d = sd[(size_t)i0 * C];
  for (int it = i0; it < i1; ++it) {
    float Ln = 0.f, dn = 0.f;
    if (it + 1 < i1) {  // the next chunk's numbers are on their way while this one is joined
      Ln = scratch[(size_t)(it + 1) * CN + e];
      dn = sd[(size_t)(it + 1) * C];
    }
    scratch[(size_t)it * CN + e] = S;
    S = fmaf(expf(a * d), S, L);
    L = Ln;
    d = dn;
  }
}

// ------------------------------------------------------------------------------------------------ softmax attention with a window and a sink
// Query head h reads key/value head h / (H / G); token i sees the keys j with 0 <= i - j < window (window <= 0: every j <= i);
// weights = exp(score - max) / (sum over visible keys + exp(sink[h] - max)): the sink (may be null) has no key and no value.
// A workgroup = 16 query rows (QT tokens of one request x HB query heads of ONE key/value head) x 16 lanes, one range of the
// visible keys.  splits > 1: (max, sum, unnormalised output) per range, joined by sink_merge_kernel, where the sink enters.
constexpr int kSinkRows = 16;
constexpr int kSinkMaxC = 16;  // value columns per lane: dv <= 256

template <typename T>
__global__ __launch_bounds__(256) void sink_attn_kernel(T* __restrict__ out, int64_t ld_out, float* __restrict__ part_o,
                                                        float* __restrict__ part_ml, const float* __restrict__ q,
                                                        const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                                        const int* __restrict__ table, int64_t table_stride, const int* __restrict__ req_rows,
                                                        const int* __restrict__ seq_lens, const int* __restrict__ cu_q, int B, int total_q,
                                                        int H, int G, int d, int dv, float scale, int window, const float* __restrict__ sink,
                                                        int QT, int HB, int KT, int splits) {
  extern __shared__ float lds[];
  const int qs = d + 1, vs = dv + 1;
  float* sq = lds;                      // [16][d + 1]
  float* sk = sq + kSinkRows * qs;      // [KT][d + 1]
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
  const int limit = valid ? start + tl : -1;                          // last visible key
  const int lo_row = window > 0 ? max(0, limit - window + 1) : 0;     // first visible key
  const int last_tok = min(s_tok0 + QT, q_len) - 1;
  const int n_keys = start + last_tok + 1;
  const int lo_blk = window > 0 ? max(0, start + s_tok0 - window + 1) : 0;
  const int per = ((n_keys - lo_blk + splits - 1) / splits + KT - 1) / KT * KT;
  const int k_begin = lo_blk + blockIdx.z * per, k_end = min(n_keys, k_begin + per);
  for (int i = l; i < d; i += 16) sq[r * qs + i] = q[((size_t)tok * H + head) * d + i];
  const int* trow = table + (size_t)req_rows[b] * table_stride;
  float o[kSinkMaxC];
#pragma unroll
  for (int i = 0; i < kSinkMaxC; ++i) o[i] = 0.f;
  float m = -INFINITY, lsum = 0.f;
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
    float tmax = -INFINITY;
    for (int j = l; j < KT; j += 16) {
      float s = -INFINITY;
      if (j < nk && j0 + j <= limit && j0 + j >= lo_row) {
        float acc = 0.f;
        const float* qp = sq + r * qs;
        const float* kp = sk + j * qs;
        for (int i = 0; i < d; ++i) acc = fmaf(qp[i], kp[i], acc);
        s = acc * scale;
      }
      sp[r * KT + j] = s;
      tmax = fmaxf(tmax, s);
    }
#pragma unroll
    for (int x = 8; x >= 1; x >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, x, 64));
    const float m_new = fmaxf(m, tmax);
    const float alpha = m_new == -INFINITY ? 1.0f : expf(m - m_new);
    float psum = 0.f;
    for (int j = l; j < KT; j += 16) {
      const float s = sp[r * KT + j];
      const float p = s == -INFINITY ? 0.f : expf(s - m_new);
      sp[r * KT + j] = p;
      psum += p;
    }
#pragma unroll
    for (int x = 8; x >= 1; x >>= 1) psum += __shfl_xor(psum, x, 64);
    lsum = fmaf(lsum, alpha, psum);
    m = m_new;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kSinkMaxC; ++i) {
      const int c = l + 16 * i;
      if (c < dv) {
        float acc = o[i] * alpha;
        for (int j = 0; j < nk; ++j) acc = fmaf(sp[r * KT + j], sv[j * vs + c], acc);
        o[i] = acc;
      }
    }
  }
  if (!valid) return;
  if (splits == 1) {
    const float sk_h = sink ? sink[head] : -INFINITY;
    const float mf = fmaxf(m, sk_h);
    const float em = expf(m - mf);
    const float f = em / (lsum * em + (sink ? expf(sk_h - mf) : 0.f));
#pragma unroll
    for (int i = 0; i < kSinkMaxC; ++i) {
      const int c = l + 16 * i;
      if (c < dv) st(out + (size_t)tok * ld_out + (size_t)head * dv + c, o[i] * f);
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < kSinkMaxC; ++i) {
    const int c = l + 16 * i;
    if (c < dv) part_o[((size_t)blockIdx.z * total_q + tok) * H * dv + (size_t)head * dv + c] = o[i];
  }
  if (l == 0) {
    float* ml = part_ml + (((size_t)blockIdx.z * total_q + tok) * H + head) * 2;
    ml[0] = m;
    ml[1] = lsum;
  }
}

// The same on the matrix cores, for bf16 caches.  A workgroup = 64 query rows ((token, head) pairs of one request and ONE key/value
// head: QT tokens x HB heads) in 4 waves of 16 rows, one key range.  Keys and values come through LDS in tiles of 64 rows, row-major,
// 16-byte padded.  Per 64-key tile and wave:
//   S^T[16 keys x 16 rows] = K . Q^T     per 16-key subtile KC x v_mfma_f32_16x16x32_bf16 (Q fragments in registers, rounded to bf16 once)
//   ONE fp32 softmax step for the tile in the lane that holds the scores (a query row's 16 keys; the row's other keys sit in the
//   lanes 16, 32 and 48 further on): new maximum, rescale of the row's sum and output, weights as bf16 B operands;
//   O^T[16 v x 16 rows] += V^T . P^T     VC x v_mfma_f32_16x16x16_bf16, V^T fragments read TRANSPOSED out of the row-major value
//   tile (ds_read_b64_tr_b16).
constexpr int kNKT = 64;

template <int KC, int VC>
__global__ __launch_bounds__(256) void sink_attn_mfma_kernel(bf16_t* __restrict__ out, int64_t ld_out, float* __restrict__ part_o,
                                                             float* __restrict__ part_ml, const float* __restrict__ q,
                                                             const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                                                             const int* __restrict__ table, int64_t table_stride,
                                                             const int* __restrict__ req_rows, const int* __restrict__ seq_lens,
                                                             const int* __restrict__ cu_q, int B, int total_q, int H, int G, int d, int dv,
                                                             float scale, int window, const float* __restrict__ sink, int QT, int HB,
                                                             int splits, int kvec, int vvec) {
  constexpr int KS = KC * 32 + 8, VS = VC * 16 + 8;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* sk = smem;               // [kNKT][KS]
  uint16_t* sv = smem + kNKT * KS;   // [kNKT][VS]
  __shared__ int s_req, s_tok0, s_cnt[256];
  __shared__ int s_slot[2][kNKT];
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
  const int lo_row = window > 0 ? max(0, limit - window + 1) : 0;
  const int last_tok = min(s_tok0 + QT, q_len) - 1;
  const int n_keys = start + last_tok + 1;
  const int lo_blk = window > 0 ? max(0, start + s_tok0 - window + 1) : 0;
  const int per = ((n_keys - lo_blk + splits - 1) / splits + kNKT - 1) / kNKT * kNKT;
  const int k_begin = lo_blk + z * per, k_end = min(n_keys, k_begin + per);
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
  float m = -INFINITY, lsum = 0.f;  // the row's maximum (the same in its four lanes) and this lane's share of the row's sum
  const int* trow = table + (size_t)req_rows[b] * table_stride;
  const size_t nkd = (size_t)G * d, nvd = (size_t)G * dv, ko = (size_t)kvh * d, vo = (size_t)kvh * dv;
  // the next tile's rows are requested before the current tile's products: their latency hides under the MFMAs
  constexpr int NK = (kNKT * KC * 4 + 255) / 256, NV = (kNKT * VC * 2 + 255) / 256;
  Q4 pre_k[NK], pre_v[NV];
  auto request = [&](int j0, int buf) {
#pragma unroll
    for (int u = 0; u < NK; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (KC * 4), k = (e - key * (KC * 4)) * 8;
      pre_k[u] = Q4{0u, 0u, 0u, 0u};
      if (e < kNKT * KC * 4 && j0 + key < k_end && k < d) pre_k[u] = load8(k_cache + (size_t)s_slot[buf][key] * nkd + ko + k, d - k, kvec != 0);
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (VC * 2), c = (e - key * (VC * 2)) * 8;
      pre_v[u] = Q4{0u, 0u, 0u, 0u};
      if (e < kNKT * VC * 2 && j0 + key < k_end && c < dv) pre_v[u] = load8(v_cache + (size_t)s_slot[buf][key] * nvd + vo + c, dv - c, vvec != 0);
    }
  };
  if (threadIdx.x < kNKT && k_begin + (int)threadIdx.x < k_end) s_slot[0][threadIdx.x] = trow[k_begin + threadIdx.x];
  __syncthreads();
  if (k_begin < k_end) request(k_begin, 0);
  int buf = 0;
  for (int j0 = k_begin; j0 < k_end; j0 += kNKT, buf ^= 1) {
    __syncthreads();
    if (threadIdx.x < kNKT && j0 + kNKT + (int)threadIdx.x < k_end) s_slot[buf ^ 1][threadIdx.x] = trow[j0 + kNKT + threadIdx.x];
#pragma unroll
    for (int u = 0; u < NK; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (KC * 4), ch = e - key * (KC * 4);
      if (e < kNKT * KC * 4) *reinterpret_cast<Q4*>(&sk[key * KS + ch * 8]) = pre_k[u];
    }
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int e = u * 256 + threadIdx.x;
      const int key = e / (VC * 2), ch = e - key * (VC * 2);
      if (e < kNKT * VC * 2) *reinterpret_cast<Q4*>(&sv[key * VS + ch * 8]) = pre_v[u];
    }
    __syncthreads();
    if (j0 + kNKT < k_end) request(j0 + kNKT, buf ^ 1);
    if (!wave_live) continue;
    constexpr int NKS = kNKT / 16;
    f32x4_t sc[NKS];
    float tmax = -INFINITY;
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
        const float s = (j <= limit && j >= lo_row && j < k_end) ? sacc[c] * scale : -INFINITY;
        sacc[c] = s;
        tmax = fmaxf(tmax, s);
      }
      sc[ks] = sacc;
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m, tmax);
    const float alpha = m_new == -INFINITY ? 1.0f : __expf(m - m_new);
    s16x4_t pf[NKS];
    float psum = 0.f;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      float pe[4];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        pe[c] = sc[ks][c] == -INFINITY ? 0.f : __expf(sc[ks][c] - m_new);
        psum += pe[c];
      }
      const uint32_t p01 = bf16_bits(pe[0]) | (bf16_bits(pe[1]) << 16), p23 = bf16_bits(pe[2]) | (bf16_bits(pe[3]) << 16);
      pf[ks] = __builtin_bit_cast(s16x4_t, uint2{p01, p23});
    }
    lsum = fmaf(lsum, alpha, psum);
    m = m_new;
#pragma unroll
    for (int vt = 0; vt < VC; ++vt)
#pragma unroll
      for (int c = 0; c < 4; ++c) o[vt][c] *= alpha;
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
  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);
  if (!valid) return;
  if (splits == 1) {
    const float sk_h = sink ? sink[head] : -INFINITY;
    const float mf = fmaxf(m, sk_h);
    const float em = __expf(m - mf);
    const float f = em / (lsum * em + (sink ? __expf(sk_h - mf) : 0.f));
#pragma unroll
    for (int vt = 0; vt < VC; ++vt)
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int v = vt * 16 + 4 * lg + c;
        if (v < dv) st(out + (size_t)tok * ld_out + (size_t)head * dv + v, o[vt][c] * f);
      }
    return;
  }
#pragma unroll
  for (int vt = 0; vt < VC; ++vt)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int v = vt * 16 + 4 * lg + c;
      if (v < dv) part_o[((size_t)z * total_q + tok) * H * dv + (size_t)head * dv + v] = o[vt][c];
    }
  if (lg == 0) {
    float* ml = part_ml + (((size_t)z * total_q + tok) * H + head) * 2;
    ml[0] = m;
    ml[1] = lsum;
  }
}

// One wave per (token, head): the ranges' (max, sum, output) and the sink -> the normalised output row.
template <typename T>
__global__ __launch_bounds__(64) void sink_merge_kernel(T* __restrict__ out, int64_t ld_out, const float* __restrict__ part_o,
                                                        const float* __restrict__ part_ml, int total_q, int H, int dv, int splits,
                                                        const float* __restrict__ sink) {
  const size_t t = blockIdx.x / H;
  const int h = blockIdx.x % H;
  float M = sink ? sink[h] : -INFINITY;
  for (int s = 0; s < splits; ++s) M = fmaxf(M, part_ml[(((size_t)s * total_q + t) * H + h) * 2]);
  float den = sink ? expf(sink[h] - M) : 0.f;
  for (int s = 0; s < splits; ++s) {
    const float* ml = part_ml + (((size_t)s * total_q + t) * H + h) * 2;
    den += ml[1] * expf(ml[0] - M);
  }
  for (int c = threadIdx.x; c < dv; c += 64) {
    float v = 0.f;
    for (int s = 0; s < splits; ++s)
      v = fmaf(part_o[((size_t)s * total_q + t) * H * dv + (size_t)h * dv + c], expf(part_ml[(((size_t)s * total_q + t) * H + h) * 2] - M), v);
    st(out + t * ld_out + (size_t)h * dv + c, v / den);
  }
}

// ------------------------------------------------------------------------------------------------ router, expert inputs, gates, cap
// z: fp32 logits [tokens, E].  The `top` largest win (ties: lowest index); the weight of a choice is sigmoid(its logit).
__global__ __launch_bounds__(64) void route_sigmoid_kernel(int* __restrict__ ids, float* __restrict__ wts, const float* __restrict__ z,
                                                           int tokens, int E, int top, int TPB) {
  extern __shared__ float lds[];
  const int t = blockIdx.x * TPB + threadIdx.x;
  if (threadIdx.x >= TPB || t >= tokens) return;
  float* s = lds + threadIdx.x;
  for (int e = 0; e < E; ++e) s[e * TPB] = z[(size_t)t * E + e];
  for (int k = 0; k < top; ++k) {
    int best = 0;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      const float v = s[e * TPB];
      if (v > bv) {
        best = e;
        bv = v;
      }
    }
    ids[(size_t)t * top + k] = best;
    wts[(size_t)t * top + k] = sigmoidf_(bv);
    s[best * TPB] = -INFINITY;
  }
}

// out[t * top + k, :] = wts[t, k] * h[t, :]
template <typename T>
__global__ __launch_bounds__(256) void scale_rows_kernel(T* __restrict__ out, const T* __restrict__ h, const float* __restrict__ wts, int top,
                                                         int W) {
  const size_t r = blockIdx.x;
  const float f = wts[r];
  const T* src = h + (r / top) * W;
  for (int c = threadIdx.x; c < W; c += 256) st(out + r * W + c, f * ld(src + c));
}

// Router logits, choice and the scaled rows of ONE token per workgroup, for steps with few tokens (every token re-reads the router
// matrix, so long batches take the product kernel for the logits instead): z[e] = router[e] . h (fp32 accumulation over the row as
// stored), the `top` largest win, out[t * top + k] = sigmoid(z[best_k]) * h[t].
template <typename T>
__global__ __launch_bounds__(256) void route_scale_kernel(int* __restrict__ ids, float* __restrict__ wts, T* __restrict__ out,
                                                          const T* __restrict__ h, const T* __restrict__ router, int E, int top, int W) {
  extern __shared__ float lds[];
  float* row = lds;       // [W]
  float* z = lds + W;     // [E]
  float* sel = z + E;     // [top]
  const size_t t = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int c = tid; c < W; c += 256) row[c] = ld(h + t * W + c);
  __syncthreads();
  const bool vec = (W & 7) == 0 && ((uintptr_t)router & 15u) == 0;
  for (int e = wave; e < E; e += 4) {
    const T* r = router + (size_t)e * W;
    float acc = 0.f;
    if (vec) {  // 16-byte loads of the expert's row, several in flight
      for (int c0 = lane * 8; c0 < W; c0 += 512) {
        float wv[8];
        read8(r + c0, wv);
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = fmaf(row[c0 + i], wv[i], acc);
      }
    } else {
      for (int c = lane; c < W; c += 64) acc = fmaf(row[c], ld(r + c), acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) z[e] = acc;
  }
  __syncthreads();
  if (tid == 0) {
    for (int k = 0; k < top; ++k) {
      int best = 0;
      float bv = -INFINITY;
      for (int e = 0; e < E; ++e)
        if (z[e] > bv) {
          best = e;
          bv = z[e];
        }
      ids[t * top + k] = best;
      sel[k] = wts[t * top + k] = sigmoidf_(bv);
      z[best] = -INFINITY;
    }
  }
  __syncthreads();
  for (int k = 0; k < top; ++k) {
    const float f = sel[k];
    for (int c = tid; c < W; c += 256) st(out + (t * top + k) * W + c, f * row[c]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_kernel(T* __restrict__ out, const float* __restrict__ o, const T* __restrict__ g,
                                                           int64_t ld_g, int N) {
  const size_t t = blockIdx.x;
  for (int c = threadIdx.x; c < N; c += 256) st(out + t * N + c, o[t * N + c] * sigmoidf_(ld(g + t * ld_g + c)));
}

template <typename T>
__global__ __launch_bounds__(256) void softcap_kernel(T* __restrict__ x, int64_t stride, int N, float cap, float inv_cap) {
  T* row = x + (size_t)blockIdx.x * stride;
  for (int c = blockIdx.y * 1024 + threadIdx.x; c < min(N, (int)(blockIdx.y + 1) * 1024); c += 256) st(row + c, cap * tanhf(ld(row + c) * inv_cap));
}

}  // namespace

// ================================================================================================ C ABI
int msgl_mix_norm_conv(const float* x_in, float* x_out, const void* y0, int p0, const void* y1, int p1, float mult, const float* add,
                       const void* w, int groups, float eps, const void* taps, int n, const float* state, float* staging, void* h_out,
                       const int* cu_q, const int* seq_lens, const int* slots, int batch, int rows, int W, int dtype, void* stream) {
  MIX_REQUIRE(x_in && w && h_out && dtype_ok(dtype), "norm_conv: null pointer / dtype");
  MIX_REQUIRE(rows >= 0 && W >= 1 && groups >= 1 && W % groups == 0 && n >= 1 && n <= 64 && p0 >= 0 && p1 >= 0 && (p0 == 0 || y0) &&
                  (p1 == 0 || y1),
              "norm_conv: bad sizes W %d groups %d taps %d", W, groups, n);
  MIX_REQUIRE(x_out != x_in, "norm_conv: the sum needs a buffer of its own");
  MIX_REQUIRE(n == 1 || (taps && cu_q && seq_lens && slots && state && staging && batch >= 1),
              "norm_conv: a convolution over time needs taps, the requests and their state rows");
  if (rows == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto al16 = [](const void* p) { return ((uintptr_t)p & 15u) == 0; };
  const bool vec = W % 8 == 0 && (W / groups) % 8 == 0 && W <= 8192 && n <= 4 && al16(x_in) && al16(x_out) && al16(y0) && al16(y1) && al16(add) &&
                   al16(w) && al16(taps) && al16(state) && al16(staging) && al16(h_out);
  if (vec) {
    // enough workgroups to fill the chip before a workgroup walks more tokens: a walk of TB tokens re-reads n - 1 rows
    int TB = rows / 1024;
    TB = TB < 1 ? 1 : (TB > 8 ? 8 : TB);
    const int grid = cu_q ? (rows + TB - 1) / TB + batch : (rows + TB - 1) / TB;
    const size_t lds = ((size_t)(W / 8) + groups) * sizeof(float);
    const int nch = (W + 2047) / 2048;
#define NC_LAUNCH(NCH, NT)                                                                                                              \
  DISPATCH_T(dtype, hipLaunchKernelGGL((norm_conv_vec_kernel<T, NCH, NT>), dim3(grid), dim3(256), lds, s, x_in, x_out, cp<T>(y0), p0,   \
                                       cp<T>(y1), p1, mult, add, cp<T>(w), groups, eps, cp<T>(taps), state, staging, mp<T>(h_out), cu_q, \
                                       seq_lens, slots, batch, rows, W, TB);)
#define NC_TAPS(NCH)       \
  if (n == 1) {            \
    NC_LAUNCH(NCH, 1)      \
  } else if (n == 2) {     \
    NC_LAUNCH(NCH, 2)      \
  } else if (n == 3) {     \
    NC_LAUNCH(NCH, 3)      \
  } else {                 \
    NC_LAUNCH(NCH, 4)      \
  }
    if (nch == 1) {
      NC_TAPS(1)
    } else if (nch == 2) {
      NC_TAPS(2)
    } else {
      NC_TAPS(4)
    }
#undef NC_TAPS
#undef NC_LAUNCH
    MIX_LAUNCHED("norm_conv (16-byte accesses)");
    return MSGL_MIX_OK;
  }
  int TB = rows / 512;
  TB = TB < 1 ? 1 : (TB > 16 ? 16 : TB);
  const int grid = cu_q ? (rows + TB - 1) / TB + batch : (rows + TB - 1) / TB;
  const size_t lds = ((size_t)n * W + groups) * sizeof(float);
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)norm_conv_kernel<T>, lds) == 0, "norm_conv: %d rows of %d do not fit LDS", n, W);
             hipLaunchKernelGGL(norm_conv_kernel<T>, dim3(grid), dim3(256), lds, s, x_in, x_out, cp<T>(y0), p0, cp<T>(y1), p1, mult, add,
                                cp<T>(w), groups, eps, cp<T>(taps), n, state, staging, mp<T>(h_out), cu_q, seq_lens, slots, batch, rows, W,
                                TB);)
  MIX_LAUNCHED("norm_conv");
  return MSGL_MIX_OK;
}

int msgl_mix_selective_scan(void* out, const void* x, int64_t ld_x, const void* z, int64_t ld_z, const void* dt_in, int64_t ld_dt,
                            const void* bc, int64_t ld_bc, const float* A, const float* dt_bias, const float* D, float* state,
                            const int* cu_q, const int* seq_lens, const int* slots, int batch, int C, int N, int dtype, int n_items,
                            const int* items, const int* item_first, float* scratch, void* stream) {
  MIX_REQUIRE(out && x && z && dt_in && bc && A && dt_bias && D && state && cu_q && seq_lens && slots && dtype_ok(dtype),
              "selective_scan: null pointer / dtype");
  MIX_REQUIRE(batch >= 0 && C >= 1 && N >= 1 && N <= 256 && ld_x >= C && ld_z >= C && ld_dt >= C && ld_bc >= 2 * N,
              "selective_scan: bad sizes C %d N %d", C, N);
  MIX_REQUIRE(n_items == 0 || (items && item_first && scratch), "selective_scan: chunks need their lists and scratch");
  if (batch == 0) return MSGL_MIX_OK;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int cb = (C + 255) / 256;
#define SCAN_CASE(NP)                                                                                                                     \
  if (N <= NP) {                                                                                                                          \
    DISPATCH_T(dtype,                                                                                                                     \
               if (n_items == 0) {                                                                                                        \
                 hipLaunchKernelGGL((selective_scan_kernel<T, NP, 0>), dim3(cb, batch), dim3(256), 0, s, mp<T>(out), cp<T>(x), ld_x,      \
                                    cp<T>(z), ld_z, cp<T>(dt_in), ld_dt, cp<T>(bc), ld_bc, A, dt_bias, D, state, cu_q, seq_lens, slots,  \
                                    C, N, items, item_first, scratch, 0);                                                                 \
               } else {                                                                                                                   \
                 hipLaunchKernelGGL((selective_scan_kernel<T, NP, 1>), dim3(cb, n_items), dim3(256), 0, s, mp<T>(out), cp<T>(x), ld_x,    \
                                    cp<T>(z), ld_z, cp<T>(dt_in), ld_dt, cp<T>(bc), ld_bc, A, dt_bias, D, state, cu_q, seq_lens, slots,  \
                                    C, N, items, item_first, scratch, n_items);                                                           \
                 hipLaunchKernelGGL(selective_join_kernel, dim3((C * N + 255) / 256, batch), dim3(256), 0, s, state, scratch, A, cu_q, seq_lens,       \
                                    slots, item_first, C, N, n_items);                                                                    \
                 hipLaunchKernelGGL((selective_scan_kernel<T, NP, 2>), dim3(cb, n_items), dim3(256), 0, s, mp<T>(out), cp<T>(x), ld_x,    \
                                    cp<T>(z), ld_z, cp<T>(dt_in), ld_dt, cp<T>(bc), ld_bc, A, dt_bias, D, state, cu_q, seq_lens, slots,  \
                                    C, N, items, item_first, scratch, n_items);                                                           \
               })                                                                                                                         \
    MIX_LAUNCHED("selective_scan");                                                                                                       \
    return MSGL_MIX_OK;                                                                                                                   \
  }
  SCAN_CASE(16)
  SCAN_CASE(32)
  SCAN_CASE(64)
  SCAN_CASE(128)
  SCAN_CASE(256)
#undef SCAN_CASE
  return MSGL_MIX_EINVAL;
}

int msgl_mix_sink_attn_workspace_floats(int total_q, int H, int dv, int splits) { return splits > 1 ? total_q * H * (dv + 2) * splits : 0; }

int msgl_mix_sink_attn(void* out, int64_t ld_out, const float* q, const void* k_cache, const void* v_cache, const int* table,
                       int64_t table_stride, const int* req_rows, const int* seq_lens, const int* cu_q, int batch, int total_q, int H, int G,
                       int d, int dv, float scale, int window, const float* sink, int dtype, int splits, float* workspace, void* stream) {
  MIX_REQUIRE(out && q && k_cache && v_cache && table && req_rows && seq_lens && cu_q && dtype_ok(dtype), "sink_attn: null pointer / dtype");
  MIX_REQUIRE(batch >= 1 && total_q >= 0 && H >= 1 && G >= 1 && H % G == 0 && d >= 1 && dv >= 1 && dv <= 16 * kSinkMaxC &&
                  ld_out >= (int64_t)H * dv,
              "sink_attn: bad sizes H %d G %d d %d dv %d", H, G, d, dv);
  MIX_REQUIRE(splits >= 1 && splits <= 1024 && (splits == 1 || workspace), "sink_attn: %d splits need a workspace", splits);
  if (total_q == 0) return MSGL_MIX_OK;
  const int rep = H / G;
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* part_o = workspace;
  float* part_ml = workspace ? workspace + (size_t)splits * total_q * H * dv : nullptr;
  if (dtype == MSGL_MIX_BF16 && d <= 256 && dv <= 256) {
    // matrix-core kernel: the smallest (KC, VC) instance that holds d <= 32 KC and dv <= 16 VC
    int HBm = 1;
    while (HBm * 2 <= rep && HBm * 2 <= 64) HBm *= 2;
    const int QTm = 64 / HBm, hbl = (rep + HBm - 1) / HBm;
    const int groups_m = (total_q + QTm - 1) / QTm + batch;
    MIX_REQUIRE((int64_t)G * hbl <= 65535, "sink_attn: too many heads");
    const dim3 grid(groups_m, G * hbl, splits);
    const int kvec = (((uintptr_t)k_cache & 15u) == 0 && d % 8 == 0) ? 1 : 0, vvec = (((uintptr_t)v_cache & 15u) == 0 && dv % 8 == 0) ? 1 : 0;
#define SINK_CASE(KC, VC)                                                                                                                 \
  if (d <= KC * 32 && dv <= VC * 16) {                                                                                                    \
    const size_t lds_m = (size_t)kNKT * ((KC * 32 + 8) + (VC * 16 + 8)) * sizeof(uint16_t);                                               \
    MIX_REQUIRE(ensure_lds((const void*)sink_attn_mfma_kernel<KC, VC>, lds_m) == 0, "sink_attn: LDS request refused");                    \
    hipLaunchKernelGGL((sink_attn_mfma_kernel<KC, VC>), grid, dim3(256), lds_m, s, mp<bf16_t>(out), ld_out, part_o, part_ml, q,           \
                       cp<bf16_t>(k_cache), cp<bf16_t>(v_cache), table, table_stride, req_rows, seq_lens, cu_q, batch, total_q, H, G, d,  \
                       dv, scale, window, sink, QTm, HBm, splits, kvec, vvec);                                                            \
    MIX_LAUNCHED("sink_attn (matrix cores)");                                                                                             \
    if (splits > 1) {                                                                                                                     \
      hipLaunchKernelGGL(sink_merge_kernel<bf16_t>, dim3(total_q * H), dim3(64), 0, s, mp<bf16_t>(out), ld_out, part_o, part_ml, total_q, \
                         H, dv, splits, sink);                                                                                            \
      MIX_LAUNCHED("sink_attn merge");                                                                                                    \
    }                                                                                                                                     \
    return MSGL_MIX_OK;                                                                                                                   \
  }
    SINK_CASE(2, 4)
    SINK_CASE(3, 6)
    SINK_CASE(4, 8)
    SINK_CASE(6, 12)
    SINK_CASE(8, 16)
#undef SINK_CASE
  }
  int HB = 1;
  while (HB * 2 <= rep && HB * 2 <= kSinkRows) HB *= 2;
  const int QT = kSinkRows / HB, hblocks = (rep + HB - 1) / HB;
  int KT = 64;
  auto need = [&](int kt) { return (size_t)((kSinkRows + kt) * (d + 1) + kt * (dv + 1) + kSinkRows * kt) * sizeof(float); };
  while (KT > 8 && need(KT) > 160 * 1024) KT >>= 1;
  const size_t lds = need(KT);
  MIX_REQUIRE(lds <= 160 * 1024, "sink_attn: heads of %d / %d do not fit LDS", d, dv);
  const int groups = (total_q + QT - 1) / QT + batch;  // every request may end with one partial group
  MIX_REQUIRE((int64_t)G * hblocks <= 65535, "sink_attn: too many heads");
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)sink_attn_kernel<T>, lds) == 0, "sink_attn: LDS request refused");
             hipLaunchKernelGGL(sink_attn_kernel<T>, dim3(groups, G * hblocks, splits), dim3(256), lds, s, mp<T>(out), ld_out, part_o,
                                part_ml, q, cp<T>(k_cache), cp<T>(v_cache), table, table_stride, req_rows, seq_lens, cu_q, batch, total_q, H,
                                G, d, dv, scale, window, sink, QT, HB, KT, splits);
             if (splits > 1) hipLaunchKernelGGL(sink_merge_kernel<T>, dim3(total_q * H), dim3(64), 0, s, mp<T>(out), ld_out, part_o, part_ml,
                                                total_q, H, dv, splits, sink);)
  MIX_LAUNCHED("sink_attn");
  return MSGL_MIX_OK;
}

int msgl_mix_route_sigmoid(int* ids, float* wts, const float* z, int tokens, int E, int top, void* stream) {
  MIX_REQUIRE(ids && wts && z, "route_sigmoid: null pointer");
  MIX_REQUIRE(tokens >= 0 && E >= 1 && top >= 1 && top <= E, "route_sigmoid: bad sizes E %d top %d", E, top);
  if (tokens == 0) return MSGL_MIX_OK;
  int TPB = 64;
  while (TPB > 1 && (size_t)TPB * E * sizeof(float) > 64 * 1024) TPB >>= 1;
  MIX_REQUIRE((size_t)TPB * E * sizeof(float) <= 64 * 1024, "route_sigmoid: %d experts do not fit LDS", E);
  hipLaunchKernelGGL(route_sigmoid_kernel, dim3((tokens + TPB - 1) / TPB), dim3(64), (size_t)TPB * E * sizeof(float),
                     static_cast<hipStream_t>(stream), ids, wts, z, tokens, E, top, TPB);
  MIX_LAUNCHED("route_sigmoid");
  return MSGL_MIX_OK;
}

int msgl_mix_scale_rows(void* out, const void* h, const float* wts, int tokens, int top, int W, int dtype, void* stream) {
  MIX_REQUIRE(out && h && wts && dtype_ok(dtype) && tokens >= 0 && top >= 1 && W >= 1, "scale_rows: null pointer / sizes");
  if (tokens == 0) return MSGL_MIX_OK;
  DISPATCH_T(dtype, hipLaunchKernelGGL(scale_rows_kernel<T>, dim3(tokens * top), dim3(256), 0, static_cast<hipStream_t>(stream), mp<T>(out),
                                       cp<T>(h), wts, top, W);)
  MIX_LAUNCHED("scale_rows");
  return MSGL_MIX_OK;
}

int msgl_mix_route_scale(int* ids, float* wts, void* out, const void* h, const void* router, int tokens, int E, int top, int W, int dtype,
                         void* stream) {
  MIX_REQUIRE(ids && wts && out && h && router && dtype_ok(dtype), "route_scale: null pointer / dtype");
  MIX_REQUIRE(tokens >= 0 && E >= 1 && top >= 1 && top <= E && W >= 1, "route_scale: bad sizes E %d top %d", E, top);
  if (tokens == 0) return MSGL_MIX_OK;
  const size_t lds = ((size_t)W + E + top) * sizeof(float);
  DISPATCH_T(dtype, MIX_REQUIRE(ensure_lds((const void*)route_scale_kernel<T>, lds) == 0, "route_scale: a row of %d and %d experts do not fit LDS", W, E);
             hipLaunchKernelGGL(route_scale_kernel<T>, dim3(tokens), dim3(256), lds, static_cast<hipStream_t>(stream), ids, wts, mp<T>(out),
                                cp<T>(h), cp<T>(router), E, top, W);)
  MIX_LAUNCHED("route_scale");
  return MSGL_MIX_OK;
}

int msgl_mix_sigmoid_gate(void* out, const float* o, const void* g, int64_t ld_g, int rows, int N, int dtype, void* stream) {
  MIX_REQUIRE(out && o && g && dtype_ok(dtype) && rows >= 0 && N >= 1 && ld_g >= N, "sigmoid_gate: null pointer / sizes");
  if (rows == 0) return MSGL_MIX_OK;
  DISPATCH_T(dtype, hipLaunchKernelGGL(sigmoid_gate_kernel<T>, dim3(rows), dim3(256), 0, static_cast<hipStream_t>(stream), mp<T>(out), o,
                                       cp<T>(g), ld_g, N);)
  MIX_LAUNCHED("sigmoid_gate");
  return MSGL_MIX_OK;
}

int msgl_mix_softcap(void* x, int64_t ld, int rows, int N, float cap, int dtype, void* stream) {
  MIX_REQUIRE(x && dtype_ok(dtype) && rows >= 0 && N >= 1 && ld >= N && cap > 0.f, "softcap: null pointer / sizes / cap");
  if (rows == 0) return MSGL_MIX_OK;
  DISPATCH_T(dtype, hipLaunchKernelGGL(softcap_kernel<T>, dim3(rows, (N + 1023) / 1024), dim3(256), 0, static_cast<hipStream_t>(stream), mp<T>(x), ld, N, cap,
                                       1.0f / cap);)
  MIX_LAUNCHED("softcap");
  return MSGL_MIX_OK;
}
