// Shared device helpers for the gfx950 kernels: element types, conversions,
// wave and block reductions. Every kernel file includes only this header.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

// Element type codes of the C interface.
#define TIE_F32 0
#define TIE_BF16 1
#define TIE_F16 2   // a cache of keys and values only (beside float32 arithmetic)

// Error codes of the C interface (besides hipError_t values, which are > 0).
#define TIE_OK 0
#define TIE_BAD_ARGUMENT (-1)

#define TIE_WAVE 64

typedef uint16_t bf16_t;  // raw bfloat16 bits
typedef _Float16 f16_t;   // IEEE half precision, converted by the hardware (round to nearest even)

__device__ __forceinline__ float bf16_to_float(bf16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// Round to nearest even; NaN stays NaN (quieted).
// Round to nearest even, NaN stays NaN: gfx950 converts in hardware (v_cvt_pk_bf16_f32).
typedef __bf16 tie_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float tie_floatx2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const tie_floatx2_t f = {lo, hi};
  const tie_bf16x2_t b = __builtin_convertvector(f, tie_bf16x2_t);
  return *reinterpret_cast<const uint32_t*>(&b);
}

__device__ __forceinline__ bf16_t float_to_bf16(float f) { return static_cast<bf16_t>(pack_bf16x2(f, 0.f) & 0xffffu); }

template <typename T>
__device__ __forceinline__ float load_as_float(const T* p);
template <>
__device__ __forceinline__ float load_as_float<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_as_float<bf16_t>(const bf16_t* p) { return bf16_to_float(*p); }

template <>
__device__ __forceinline__ float load_as_float<f16_t>(const f16_t* p) { return static_cast<float>(*p); }

template <typename T>
__device__ __forceinline__ void store_from_float(T* p, float v);
template <>
__device__ __forceinline__ void store_from_float<f16_t>(f16_t* p, float v) { *p = static_cast<f16_t>(v); }
template <>
__device__ __forceinline__ void store_from_float<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_from_float<bf16_t>(bf16_t* p, float v) { *p = float_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = TIE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TIE_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = TIE_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TIE_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds >= 16 floats of LDS.
// Every thread receives the total. The order of additions is fixed by the
// thread layout alone, so a row's sum does not depend on what else runs.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int wave = threadIdx.x / TIE_WAVE;
  const int waves = (blockDim.x + TIE_WAVE - 1) / TIE_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (TIE_WAVE - 1);
  const int wave = threadIdx.x / TIE_WAVE;
  const int waves = (blockDim.x + TIE_WAVE - 1) / TIE_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = scratch[0];
  for (int w = 1; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

static inline int tie_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? TIE_OK : static_cast<int>(e);
}

// Dispatch helpers: call `fn.template operator()<T>()` style lambdas are avoided;
// instead each launcher switches on the dtype codes explicitly.
