// Shared device helpers and host-side argument checks of the sequence-mixing kernels (seqmix.hip, mix_delta.hip, mix_par.hip).
// Everything lives in an anonymous namespace: each translation unit of libmsgl_mix.so gets its own copy, and the one
// per-thread error text is reached through msgl_mix_set_error / msgl_mix_last_error.
#ifndef MSGL_MIX_COMMON_H_
#define MSGL_MIX_COMMON_H_

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/msgl_mix.h"

extern "C" void msgl_mix_set_error(const char* text);

namespace {

void set_err(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  msgl_mix_set_error(buf);
}
#define MIX_REQUIRE(cond, ...) \
  do {                         \
    if (!(cond)) {             \
      set_err(__VA_ARGS__);    \
      return MSGL_MIX_EINVAL;  \
    }                          \
  } while (0)
#define MIX_LAUNCHED(name)                                                \
  do {                                                                    \
    hipError_t e_ = hipGetLastError();                                    \
    if (e_ != hipSuccess) {                                               \
      set_err("%s: launch failed: %s", name, hipGetErrorString(e_));      \
      return MSGL_MIX_ELAUNCH;                                            \
    }                                                                     \
  } while (0)

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16_t* p) { return __uint_as_float((uint32_t)p->bits << 16); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) {  // round to nearest even, NaN kept quiet
  uint32_t u = __float_as_uint(v);
  if ((u & 0x7fffffffu) > 0x7f800000u) {
    p->bits = (uint16_t)((u >> 16) | 0x40u);
    return;
  }
  u += 0x7fffu + ((u >> 16) & 1u);
  p->bits = (uint16_t)(u >> 16);
}

// eight consecutive elements as fp32 (the caller guarantees 16-byte alignment)
__device__ __forceinline__ void read8(const float* p, float (&f)[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void read8(const bf16_t* p, float (&f)[8]) {
  const uint4 u = *reinterpret_cast<const uint4*>(p);
  f[0] = __uint_as_float(u.x << 16); f[1] = __uint_as_float(u.x & 0xffff0000u);
  f[2] = __uint_as_float(u.y << 16); f[3] = __uint_as_float(u.y & 0xffff0000u);
  f[4] = __uint_as_float(u.z << 16); f[5] = __uint_as_float(u.z & 0xffff0000u);
  f[6] = __uint_as_float(u.w << 16); f[7] = __uint_as_float(u.w & 0xffff0000u);
}

__device__ __forceinline__ void write8(float* p, const float (&f)[8]) {
  *reinterpret_cast<float4*>(p) = float4{f[0], f[1], f[2], f[3]};
  *reinterpret_cast<float4*>(p + 4) = float4{f[4], f[5], f[6], f[7]};
}
__device__ __forceinline__ void write8(bf16_t* p, const float (&f)[8]) {
  bf16_t t[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) st(&t[i], f[i]);
  *reinterpret_cast<uint4*>(p) = uint4{(uint32_t)t[0].bits | ((uint32_t)t[1].bits << 16), (uint32_t)t[2].bits | ((uint32_t)t[3].bits << 16),
                                       (uint32_t)t[4].bits | ((uint32_t)t[5].bits << 16), (uint32_t)t[6].bits | ((uint32_t)t[7].bits << 16)};
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// sum over a 256-thread workgroup, the same value (and the same order of additions) in every thread
__device__ __forceinline__ float block_sum256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

template <typename T>
const T* cp(const void* p) {
  return static_cast<const T*>(p);
}
template <typename T>
T* mp(void* p) {
  return static_cast<T*>(p);
}

// ---- matrix-core helpers: fragment types, packed bf16 loads
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
struct __attribute__((aligned(16))) Q4 {
  uint32_t x, y, z, w;
};
__device__ __forceinline__ uint32_t bf16_bits(float v) {
  bf16_t t;
  st(&t, v);
  return t.bits;
}

// eight consecutive k of one row as packed bf16; `n` of them exist (the rest read as zero); vec: 16-byte loads are legal
__device__ __forceinline__ Q4 load8(const bf16_t* p, int n, bool vec) {
  if (vec && n >= 8) return *reinterpret_cast<const Q4*>(p);
  uint32_t e[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) e[i] = i < n ? p[i].bits : 0u;
  return Q4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
}
__device__ __forceinline__ Q4 load8(const float* p, int n, bool vec) {
  float f[8];
  if (vec && n >= 8) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = i < n ? p[i] : 0.f;
  }
  return Q4{bf16_bits(f[0]) | (bf16_bits(f[1]) << 16), bf16_bits(f[2]) | (bf16_bits(f[3]) << 16),
            bf16_bits(f[4]) | (bf16_bits(f[5]) << 16), bf16_bits(f[6]) | (bf16_bits(f[7]) << 16)};
}

typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((address_space(3))) s16x4_t lds_s16x4_t;

// Which request and which of its QT-token groups workgroup `blockIdx.x` owns: group counts ceil(new tokens / QT) of up to 256
// requests at a time, scanned by the whole workgroup (one pass of independent loads instead of one thread walking the batch).
// Leaves request -1 for workgroups past the last group.  cnt: 256 ints of LDS; every thread of the (256-thread) workgroup calls.
__device__ __forceinline__ void find_group(const int* __restrict__ cu_q, int B, int QT, int* cnt, int* s_req, int* s_tok0) {
  const int tid = threadIdx.x;
  if (tid == 0) *s_req = -1;
  int base = 0;
  for (int c0 = 0; c0 < B; c0 += 256) {
    const int b = c0 + tid;
    const int g = b < B ? (cu_q[b + 1] - cu_q[b] + QT - 1) / QT : 0;
    cnt[tid] = g;
    __syncthreads();
    for (int off = 1; off < 256; off <<= 1) {
      const int v = tid >= off ? cnt[tid - off] : 0;
      __syncthreads();
      cnt[tid] += v;
      __syncthreads();
    }
    const int incl = cnt[tid], total = cnt[255];
    const int target = (int)blockIdx.x - base;
    if (b < B && target >= incl - g && target < incl) {
      *s_req = b;
      *s_tok0 = (target - (incl - g)) * QT;
    }
    __syncthreads();
    if (target < total) break;
    base += total;
  }
  __syncthreads();
}

bool dtype_ok(int dt) { return dt == MSGL_MIX_BF16 || dt == MSGL_MIX_F32; }

int ensure_lds(const void* fn, size_t bytes) {
  if (bytes <= 64 * 1024) return 0;
  if (bytes > 160 * 1024) return -1;
  return hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) == hipSuccess ? 0 : -1;
}

}  // namespace


#define DISPATCH_T(dt, ...)          \
  if ((dt) == MSGL_MIX_BF16) {       \
    using T = bf16_t;                \
    __VA_ARGS__                      \
  } else {                           \
    using T = float;                 \
    __VA_ARGS__                      \
  }

#endif
