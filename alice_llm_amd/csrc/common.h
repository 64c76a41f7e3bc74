// Shared device helpers and the host-side error channel of the HIP library.
// Everything here targets gfx950 (CDNA4): 64-lane wavefronts, 160 KB LDS per CU.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#define ALICE_WAVE 64

// Storage types.  DT_F32 / DT_BF16 are the dtype codes of the C interface.
enum { DT_F32 = 0, DT_BF16 = 1 };

struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v.bits) << 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) {
  return __uint_as_float(bits16 << 16);
}
// Round to nearest even; NaN stays NaN (the hardware conversion of gfx950).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  bf16_t r;
  r.bits = __builtin_bit_cast(uint16_t, (__bf16)f);
  return r;
}
// Two values rounded and packed, the first in the low half.
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  f32x2_t v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <typename T> __device__ __forceinline__ float load_f32(const T* p, size_t i);
template <> __device__ __forceinline__ float load_f32<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float load_f32<bf16_t>(const bf16_t* p, size_t i) { return bf16_to_f32(p[i]); }

template <typename T> __device__ __forceinline__ void store_f32(T* p, size_t i, float v);
template <> __device__ __forceinline__ void store_f32<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void store_f32<bf16_t>(bf16_t* p, size_t i, float v) { p[i] = f32_to_bf16(v); }

// Rounds through the storage type: what a value becomes when it is stored and read back.
template <typename T> __device__ __forceinline__ float round_to(float v);
template <> __device__ __forceinline__ float round_to<float>(float v) { return v; }
template <> __device__ __forceinline__ float round_to<bf16_t>(float v) { return bf16_to_f32(f32_to_bf16(v)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `red` holds 17 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();                       // `red` may still be read from an earlier call
  if (lane == 0) red[wid] = v;
  __syncthreads();
  if (wid == 0) {
    float t = lane < nw ? red[lane] : 0.f;
    t = wave_sum(t);
    if (lane == 0) red[16] = t;
  }
  __syncthreads();
  return red[16];
}
__device__ __forceinline__ float block_max(float v, float* red) {
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) red[wid] = v;
  __syncthreads();
  if (wid == 0) {
    float t = lane < nw ? red[lane] : -INFINITY;
    t = wave_max(t);
    if (lane == 0) red[16] = t;
  }
  __syncthreads();
  return red[16];
}

// tanh at full precision for the 32-bit path, a fast form for the bfloat16 path.
__device__ __forceinline__ float tanh_full(float x) { return tanhf(x); }
__device__ __forceinline__ float tanh_fast(float x) {
  // tanh(x) = 1 - 2 / (2^(2 log2e x) + 1) with the hardware's exp2 and reciprocal (about 1 ulp each):
  // absolute error about 2e-7; 2^x overflows to +inf and underflows to 0, which give exactly +-1.
  float e = __builtin_amdgcn_exp2f(x * 2.8853900817779268f);
  return fmaf(-2.f, __builtin_amdgcn_rcpf(e + 1.f), 1.f);
}
__device__ __forceinline__ float gelu_tanh_f(float z, bool full) {
  float u = 0.7978845608028654f * (z + 0.044715f * z * z * z);
  float t = full ? tanh_full(u) : tanh_fast(u);
  return 0.5f * z * (1.f + t);
}

// ---- host side -------------------------------------------------------------------------
void alice_set_error(const char* fmt, ...);

#define ALICE_CHECK(cond, ...)            \
  do {                                    \
    if (!(cond)) {                        \
      alice_set_error(__VA_ARGS__);       \
      return 1;                           \
    }                                     \
  } while (0)

#define ALICE_LAUNCH_CHECK()                                                   \
  do {                                                                         \
    hipError_t e_ = hipGetLastError();                                         \
    if (e_ != hipSuccess) {                                                    \
      alice_set_error("%s:%d: launch failed: %s", __FILE__, __LINE__,          \
                      hipGetErrorString(e_));                                  \
      return 2;                                                                \
    }                                                                          \
  } while (0)

static inline int ceil_div(long a, long b) { return (int)((a + b - 1) / b); }

// Calls `F<T>(...)`-style lambdas with the storage type that a dtype code names.
#define DISPATCH_DTYPE(code, T, ...)                         \
  do {                                                       \
    if ((code) == DT_F32) { using T = float; __VA_ARGS__; }  \
    else { using T = bf16_t; __VA_ARGS__; }                  \
  } while (0)

static inline bool dtype_ok(int code) { return code == DT_F32 || code == DT_BF16; }
