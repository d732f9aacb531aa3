// Shared helpers of the HIP kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

// dtype codes of the C interface
#define TNX_F32 0
#define TNX_BF16 1

// activation codes of the C interface
#define TNX_ACT_NONE 0
#define TNX_ACT_RELU 1
#define TNX_ACT_GELU 2      // 0.5 x (1 + erf(x / sqrt 2))
#define TNX_ACT_GELU_NEW 3  // 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))

#define TNX_WAVE 64

// Each library keeps the text of its last error; `tnx_last_error()` returns it.
#include <stdarg.h>
static thread_local char tnx_error_text[512];
static inline void tnx_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(tnx_error_text, sizeof(tnx_error_text), fmt, ap);
  va_end(ap);
}
#define TNX_DEFINE_ERROR_API \
  extern "C" const char* tnx_last_error() { return tnx_error_text; }

#define TNX_REQUIRE(cond, ...)            \
  do {                                    \
    if (!(cond)) {                        \
      tnx_set_error(__VA_ARGS__);         \
      return 1;                           \
    }                                     \
  } while (0)

#define TNX_CHECK_LAUNCH(name)                                              \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) {                                                 \
      tnx_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
      return 2;                                                             \
    }                                                                       \
  } while (0)

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return (float)x; }

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return (bf16_t)x; }

// Element `i` of an array whose dtype is known at run time only.
__device__ __forceinline__ float load_any(const void* p, int dtype, size_t i) {
  return dtype == TNX_F32 ? ((const float*)p)[i] : (float)((const bf16_t*)p)[i];
}
__device__ __forceinline__ void store_any(void* p, int dtype, size_t i, float v) {
  if (dtype == TNX_F32)
    ((float*)p)[i] = v;
  else
    ((bf16_t*)p)[i] = (bf16_t)v;
}

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

// Sum over a block of `NW` waves; every thread gets the result. `scratch` holds NW floats.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += scratch[i];
  return t;
}

__device__ __forceinline__ float apply_act(float x, int act) {
  switch (act) {
    case TNX_ACT_RELU:
      return fmaxf(x, 0.f);
    case TNX_ACT_GELU:
      return 0.5f * x * (1.f + erff(x * 0.70710678118654752440f));
    case TNX_ACT_GELU_NEW: {
      const float inner = 0.79788456080286535588f * (x + 0.044715f * x * x * x);
      return 0.5f * x * (1.f + tanhf(inner));
    }
    default:
      return x;
  }
}
