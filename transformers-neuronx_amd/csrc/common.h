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

// 16 bytes that are read once and by no one else (a weight in a decode step, a key or value of a request):
// the load is marked as streaming, so that the lines it brings in are the first to leave the caches again.
// A kernel that only reads memory reaches 6.8 TB/s on an MI355X with such loads and 5.8 to 6.1 with plain ones.
typedef __attribute__((ext_vector_type(4))) unsigned tnx_u32x4;
__device__ __forceinline__ bf16x8 load_once(const bf16_t* p) {
  return __builtin_bit_cast(bf16x8, __builtin_nontemporal_load((const tnx_u32x4*)p));
}

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

// Exchanges between the lanes of a wave without LDS. Within a row of 16 lanes the vector unit's data-parallel
// controls reach lane ^ 1 and lane ^ 2 (quad permutations), 7 - lane within 8 (the other quad) and 15 - lane
// (the other half of the row); between rows, gfx950's lane swaps exchange rows and halves of two registers.
// A shuffle would go through LDS and make the wave wait for it.
#define TNX_DPP_XOR1 0xB1         // quad_perm [1, 0, 3, 2]
#define TNX_DPP_XOR2 0x4E         // quad_perm [2, 3, 0, 1]
#define TNX_DPP_HALF_MIRROR 0x141 // lane -> 7 - lane within each 8
#define TNX_DPP_MIRROR 0x140      // lane -> 15 - lane within each 16
template <int CTRL>
__device__ __forceinline__ float lane_dpp(float v) {
  const int i = __builtin_bit_cast(int, v);
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(i, i, CTRL, 0xf, 0xf, false));
}
// The swaps give back both registers as a pair; its halves are taken into scalars before anything else is
// done with them (a bit cast applied to an element of the pair reads the first element, whichever is named).
__device__ __forceinline__ void swap_rows(unsigned u, unsigned& first, unsigned& second) {
  const auto p = __builtin_amdgcn_permlane16_swap(u, u, false, false);   // rows [r0 r0 r2 r2] and [r1 r1 r3 r3]
  first = p[0];
  second = p[1];
}
__device__ __forceinline__ void swap_halves(unsigned u, unsigned& first, unsigned& second) {
  const auto p = __builtin_amdgcn_permlane32_swap(u, u, false, false);   // halves [lo lo] and [hi hi]
  first = p[0];
  second = p[1];
}
// Maximum and sum over the four rows of 16 lanes of a wave (lanes l, l ^ 16, l ^ 32, l ^ 48), the same bits in
// all four.
__device__ __forceinline__ float rows_max(float x) {
  unsigned a, b;
  swap_halves(__float_as_uint(x), a, b);
  x = fmaxf(__uint_as_float(a), __uint_as_float(b));
  swap_rows(__float_as_uint(x), a, b);
  return fmaxf(__uint_as_float(a), __uint_as_float(b));
}
__device__ __forceinline__ float rows_sum(float x) {
  unsigned a, b;
  swap_halves(__float_as_uint(x), a, b);
  x = __uint_as_float(a) + __uint_as_float(b);
  swap_rows(__float_as_uint(x), a, b);
  return __uint_as_float(a) + __uint_as_float(b);
}
// Sum and maximum over the 64 lanes of a wave, the same bits in every lane.
__device__ __forceinline__ float wave_sum(float v) {
  v += lane_dpp<TNX_DPP_XOR1>(v);
  v += lane_dpp<TNX_DPP_XOR2>(v);
  v += lane_dpp<TNX_DPP_HALF_MIRROR>(v);
  v += lane_dpp<TNX_DPP_MIRROR>(v);
  return rows_sum(v);
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, lane_dpp<TNX_DPP_XOR1>(v));
  v = fmaxf(v, lane_dpp<TNX_DPP_XOR2>(v));
  v = fmaxf(v, lane_dpp<TNX_DPP_HALF_MIRROR>(v));
  v = fmaxf(v, lane_dpp<TNX_DPP_MIRROR>(v));
  return rows_max(v);
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

// the compute units of the current device (asked once a device)
inline int tnx_compute_units() {
  static int known[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (known[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    known[dev] = n;
  }
  return known[dev];
}

// ---- loads from global memory straight into LDS (`global_load_lds_dwordx4`)
// 16 bytes a lane from `base + offset` (offset in bytes, per lane) to LDS at `lds + 16 * lane` (the same for the
// whole wave). Written as assembly so that the compiler does not know of it: with such a load in flight it
// makes every wait for an LDS read a wait for all LDS reads, and the reads of the next fragments could not
// stay in flight during the products of these. The caller waits (`wait_for_loads`) before anyone reads.
// M0 is written here behind the compiler's back (it does not take M0 in a clobber list): a kernel that uses
// these loads must have no other instruction that reads M0, which holds for every kernel of ours.
__device__ __forceinline__ void load_to_lds(const void* base, unsigned offset, unsigned lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds), "v"(offset), "s"(base)
               : "memory");
}
// the same for bytes that are read once (see `load_once`)
__device__ __forceinline__ void load_to_lds_once(const void* base, unsigned offset, unsigned lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
               :
               : "s"(lds), "v"(offset), "s"(base)
               : "memory");
}
// the same from a pointer of the lane's own
__device__ __forceinline__ void load_to_lds(const void* address, unsigned lds) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds), "v"(address)
               : "memory");
}
__device__ __forceinline__ void wait_for_loads() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
// the address of a place in LDS as such a load wants it
__device__ __forceinline__ unsigned lds_offset(const void* p) {
  return (unsigned)(size_t)(const __attribute__((address_space(3))) char*)p;
}
