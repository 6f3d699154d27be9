// Shared device/host helpers for libsiirl_hip.so (gfx950 only, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/siirl_hip.h"

namespace siirl {

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// The part has a 256 MB memory-side cache in front of the HBM.  A tensor that a later launch reads again is read
// and written with ordinary accesses while one pass over it moves no more than this many bytes (the cache and a
// little more: the measured break-even lies between 260 and 375 MiB), and with non-temporal ones beyond, where
// ordinary accesses would only evict each other.
constexpr double kCacheResidentBytes = 300.0 * 1048576.0;
inline bool streams_past_cache(double bytes_per_pass) { return bytes_per_pass > kCacheResidentBytes; }

// ---------------------------------------------------------------------------------- host side

// Records a message for siirl_hip_last_error() on this thread and returns `code`.
int fail(int code, const char* fmt, ...);

// Raises `kernel`'s dynamic LDS limit to `bytes` on the current device, once per (kernel, device); thread-safe.
int allow_dynamic_lds(const void* kernel, int bytes);

#define SIIRL_REQUIRE(cond, ...)                                              \
  do {                                                                        \
    if (!(cond)) return ::siirl::fail(SIIRL_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

#define SIIRL_HIP_CHECK(expr)                                                                   \
  do {                                                                                          \
    hipError_t e_ = (expr);                                                                     \
    if (e_ != hipSuccess)                                                                       \
      return ::siirl::fail(SIIRL_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));        \
  } while (0)

// Launch errors are read with hipGetLastError right after the launch; nothing synchronises.
#define SIIRL_LAUNCH_CHECK(what)                                                              \
  do {                                                                                        \
    hipError_t e_ = hipGetLastError();                                                        \
    if (e_ != hipSuccess)                                                                     \
      return ::siirl::fail(SIIRL_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e_)); \
  } while (0)

inline size_t dtype_size(int dt) {
  switch (dt) {
    case SIIRL_F32: case SIIRL_I32: return 4;
    case SIIRL_BF16: case SIIRL_F16: return 2;
    case SIIRL_F64: case SIIRL_I64: return 8;
    case SIIRL_U8: return 1;
    default: return 0;
  }
}

// -------------------------------------------------------------------------------- device side

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// v_exp_f32 (2^x) without the denormal-range fix-up of exp2f(): terms below 2^-126 become 0,
// which is what a softmax term that small is worth.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Two bf16 packed in a dword -> two floats (a shift and a mask, no conversion instruction).
__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xffff0000u); }

// 16-byte register vector; a native vector type so that the nontemporal load/store builtins accept it.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ u32x4 mk4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) { return u32x4{a, b, c, d}; }

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef _Float16 halfx2_t __attribute__((ext_vector_type(2)));

// Two floats -> packed bf16 pair, round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  floatx2_t v = {lo, hi};
  bf16x2_t b = __builtin_convertvector(v, bf16x2_t);
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  floatx2_t v = {lo, hi};
  halfx2_t b = __builtin_convertvector(v, halfx2_t);
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ float f16_lo(uint32_t w) {
  return (float)__builtin_bit_cast(halfx2_t, w).x;
}
__device__ __forceinline__ float f16_hi(uint32_t w) {
  return (float)__builtin_bit_cast(halfx2_t, w).y;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum over the workgroup; every thread gets the result.  `smem` holds >= blockDim.x / 64 + 1 items.
template <typename T>
__device__ __forceinline__ T block_sum(T v, T* smem) {
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  const int nw = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();  // protects smem against a previous call's readers
  if (lane == 0) smem[wid] = v;
  __syncthreads();
  T r = (lane < nw) ? smem[lane] : T(0);
  r = wave_sum(r);
  return r;
}

// Mask element of any supported dtype as a float (0 outside the mask).
__device__ __forceinline__ float load_mask(const void* p, int dt, int64_t i) {
  switch (dt) {
    case SIIRL_U8: return (float)((const uint8_t*)p)[i];
    case SIIRL_I64: return (float)((const int64_t*)p)[i];
    case SIIRL_I32: return (float)((const int32_t*)p)[i];
    case SIIRL_F32: return ((const float*)p)[i];
    case SIIRL_BF16: return u2f(((uint32_t)((const uint16_t*)p)[i]) << 16);
    case SIIRL_F16: return (float)((const _Float16*)p)[i];
    default: return 0.f;
  }
}

}  // namespace siirl
