// Row gathers, the position add at the input, casts, LayerNorm.
#include "common.h"

TNX_DEFINE_ERROR_API

// out[m, :] = src[idx[m], :], rows of `row_bytes` bytes, moved in words of 4 bytes, or of 2 where a row is no
// whole number of those (bfloat16 rows of odd length). An index -1 - k stands for
// `indirect[k]`: a row number that an earlier kernel left in device memory (a token that was chosen on the
// device and has not been read by the host yet).
template <typename W>
__global__ void gather_rows_kernel(const W* __restrict__ src, const int* __restrict__ idx, W* __restrict__ out,
                                   int words, int src_rows, const int* __restrict__ indirect, int indirect_size) {
  const int m = blockIdx.x;
  int r = idx[m];
  if (r < 0 && indirect && -1 - r < indirect_size) r = indirect[-1 - r];
  if (r < 0 || r >= src_rows) return;  // the host checks ids; an id out of range writes nothing
  const W* s = src + (size_t)r * words;
  W* o = out + (size_t)m * words;
  for (int i = threadIdx.x; i < words; i += blockDim.x) o[i] = s[i];
}

extern "C" int tnx_gather_rows(const void* src, const int* idx, void* out, int m, int row_bytes, int src_rows,
                               const int* indirect, int indirect_size, hipStream_t stream) {
  TNX_REQUIRE(row_bytes > 0 && row_bytes % 2 == 0, "gather_rows: row of %d bytes is not a multiple of 2", row_bytes);
  TNX_REQUIRE(m >= 0 && src_rows > 0, "gather_rows: bad sizes m=%d rows=%d", m, src_rows);
  if (m == 0) return 0;
  if (row_bytes % 4 == 0)
    gather_rows_kernel<uint32_t><<<m, 256, 0, stream>>>((const uint32_t*)src, idx, (uint32_t*)out, row_bytes / 4,
                                                         src_rows, indirect, indirect ? indirect_size : 0);
  else
    gather_rows_kernel<uint16_t><<<m, 256, 0, stream>>>((const uint16_t*)src, idx, (uint16_t*)out, row_bytes / 2,
                                                         src_rows, indirect, indirect ? indirect_size : 0);
  TNX_CHECK_LAUNCH("gather_rows");
  return 0;
}

// Integers from pinned host memory into device memory by a kernel on the caller's stream: the step's
// integers arrive without a hand-over between the copy engine's queue and the compute queue.
__global__ void copy_ints_kernel(const int* __restrict__ src, int* __restrict__ dst, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

extern "C" int tnx_copy_ints(const int* src, int* dst, int n, hipStream_t stream) {
  TNX_REQUIRE(n >= 0 && src && dst, "copy_ints: bad arguments");
  if (n == 0) return 0;
  copy_ints_kernel<<<(n + 255) / 256, 256, 0, stream>>>(src, dst, n);
  TNX_CHECK_LAUNCH("copy_ints");
  return 0;
}

// The address under which kernels reach a block of pinned host memory.
extern "C" int tnx_device_pointer(void* host, void** device) {
  hipError_t e = hipHostGetDevicePointer(device, host, 0);
  if (e != hipSuccess) {
    tnx_set_error("device_pointer: %s", hipGetErrorString(e));
    return 1;
  }
  return 0;
}

// x[t, :] = src[t, :] + table[positions[t] + offset, :] in float32; a copy in `cd_dtype` beside it.
__global__ void add_positions_kernel(const void* __restrict__ src, int src_dtype, const int* __restrict__ positions,
                                     const void* __restrict__ table, int table_dtype, int table_rows, int offset,
                                     float* __restrict__ out_f32, void* __restrict__ out_cd, int cd_dtype, int width) {
  const int t = blockIdx.x;
  size_t base = (size_t)t * width;
  int row = table ? positions[t] + offset : 0;
  if (table && (row < 0 || row >= table_rows)) row = 0;  // the host checks positions
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    float v = load_any(src, src_dtype, base + i);
    if (table) v += load_any(table, table_dtype, (size_t)row * width + i);
    out_f32[base + i] = v;
    if (out_cd) store_any(out_cd, cd_dtype, base + i, v);
  }
}

extern "C" int tnx_add_positions(const void* src, int src_dtype, const int* positions, const void* table,
                                 int table_dtype, int table_rows, int offset, float* out_f32, void* out_cd,
                                 int cd_dtype, int tokens, int width, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0, "add_positions: bad sizes tokens=%d width=%d", tokens, width);
  if (tokens == 0) return 0;
  add_positions_kernel<<<tokens, 256, 0, stream>>>(src, src_dtype, positions, table, table_dtype, table_rows, offset,
                                                   out_f32, out_cd, cd_dtype, width);
  TNX_CHECK_LAUNCH("add_positions");
  return 0;
}

__global__ void cast_kernel(const void* __restrict__ src, int src_dtype, void* __restrict__ dst, int dst_dtype,
                            size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) store_any(dst, dst_dtype, i, load_any(src, src_dtype, i));
}

extern "C" int tnx_cast(const void* src, int src_dtype, void* dst, int dst_dtype, long long n, hipStream_t stream) {
  TNX_REQUIRE(n >= 0, "cast: negative size");
  if (n == 0) return 0;
  long long blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  cast_kernel<<<(int)blocks, 256, 0, stream>>>(src, src_dtype, dst, dst_dtype, (size_t)n);
  TNX_CHECK_LAUNCH("cast");
  return 0;
}

// LayerNorm of float32 rows: mean and biased variance in float32 (two passes over the row:
// the variance is taken around the mean, not as E[x^2] - mean^2), then weight and bias.
// One block of 256 threads per row; the row lives in registers as PER float4 per thread
// (width <= 1024 * PER, width % 4 == 0). Weight and bias are fetched before the reductions.
template <int PER, bool AFFINE, bool F32_OUT, bool BF16_OUT>
__global__ void __launch_bounds__(256)
layernorm_kernel(const float* __restrict__ x, const float* __restrict__ weight, const float* __restrict__ bias,
                 float eps, float* __restrict__ out_f32, bf16_t* __restrict__ out_bf16, int width, int center) {
  typedef __attribute__((ext_vector_type(4))) float f4;
  typedef __attribute__((ext_vector_type(4))) __bf16 b4;
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const int w4 = width >> 2;
  const f4* row = (const f4*)(x + (size_t)t * width);
  f4 v[PER], gw[PER], gb[PER];
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = threadIdx.x + j * 256;
    const bool ok = i < w4;
    v[j] = ok ? row[i] : (f4){0.f, 0.f, 0.f, 0.f};
    if (AFFINE) {
      gw[j] = ok ? ((const f4*)weight)[i] : (f4){0.f, 0.f, 0.f, 0.f};
      gb[j] = ok && bias ? ((const f4*)bias)[i] : (f4){0.f, 0.f, 0.f, 0.f};
    }
    s += (v[j].x + v[j].y) + (v[j].z + v[j].w);
  }
  // (`center` 0: a norm that only scales, by the root of the mean square: the mean stays where it is)
  const float mean = center ? block_sum<4>(s, scratch) / (float)width : 0.f;
  float q = 0.f;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    if (threadIdx.x + j * 256 < w4) {
      const f4 d = v[j] - mean;
      q += (d.x * d.x + d.y * d.y) + (d.z * d.z + d.w * d.w);
    }
  }
  const float var = block_sum<4>(q, scratch) / (float)width;
  const float rstd = rsqrtf(var + eps);
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < w4) {
      f4 y = (v[j] - mean) * rstd;
      if (AFFINE) y = y * gw[j] + gb[j];
      if (F32_OUT) ((f4*)(out_f32 + (size_t)t * width))[i] = y;
      if (BF16_OUT) {
        b4 o;
        o.x = (bf16_t)y.x; o.y = (bf16_t)y.y; o.z = (bf16_t)y.z; o.w = (bf16_t)y.w;
        ((b4*)(out_bf16 + (size_t)t * width))[i] = o;
      }
    }
  }
}

// Any width: three passes over the row in memory.
__global__ void __launch_bounds__(256)
layernorm_wide_kernel(const float* __restrict__ x, const float* __restrict__ weight, const float* __restrict__ bias,
                      float eps, float* __restrict__ out_f32, void* __restrict__ out_cd, int cd_dtype, int width,
                      int center) {
  __shared__ float scratch[4];
  const int t = blockIdx.x;
  const float* row = x + (size_t)t * width;
  float s = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) s += row[i];
  const float mean = center ? block_sum<4>(s, scratch) / (float)width : 0.f;
  float q = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float d = row[i] - mean;
    q += d * d;
  }
  const float var = block_sum<4>(q, scratch) / (float)width;
  const float rstd = rsqrtf(var + eps);
  for (int i = threadIdx.x; i < width; i += 256) {
    float y = (row[i] - mean) * rstd;
    if (weight) y *= weight[i];
    if (bias) y += bias[i];
    if (out_f32) out_f32[(size_t)t * width + i] = y;
    if (out_cd) store_any(out_cd, cd_dtype, (size_t)t * width + i, y);
  }
}

// `center` 1: y = (x - mean) / sqrt(var + eps) * weight + bias, the variance about the mean; 0: the same with the
// mean taken as 0, that is x / sqrt(mean(x^2) + eps) * weight + bias. Weight and bias are each optional.
extern "C" int tnx_layernorm(const float* x, const float* weight, const float* bias, float eps, float* out_f32,
                             void* out_cd, int cd_dtype, int tokens, int width, int center, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && width > 0, "layernorm: bad sizes tokens=%d width=%d", tokens, width);
  TNX_REQUIRE(eps > 0.f, "layernorm: eps must be positive");
  if (tokens == 0) return 0;
  TNX_REQUIRE(out_f32 != x, "layernorm: the float32 output may not alias the input");
  const bool affine = weight != nullptr;
  TNX_REQUIRE(weight != nullptr || bias == nullptr, "layernorm: a bias comes with a weight");
  const bool vec = width % 4 == 0 && width <= 1024 * 16 && (cd_dtype == TNX_BF16 || out_cd == nullptr);
  if (vec) {
    bf16_t* ob = (bf16_t*)out_cd;
#define LN_LAUNCH(PER, AFF, F, B) \
  layernorm_kernel<PER, AFF, F, B><<<tokens, 256, 0, stream>>>(x, weight, bias, eps, out_f32, ob, width, center)
#define LN_OUTS(PER, AFF)                                  \
  if (out_f32 && ob) LN_LAUNCH(PER, AFF, true, true);      \
  else if (ob) LN_LAUNCH(PER, AFF, false, true);           \
  else LN_LAUNCH(PER, AFF, true, false)
#define LN_AFF(PER)            \
  if (affine) { LN_OUTS(PER, true); } else { LN_OUTS(PER, false); }
    if (width <= 1024) { LN_AFF(1); }
    else if (width <= 1024 * 4) { LN_AFF(4); }
    else { LN_AFF(16); }
#undef LN_AFF
#undef LN_OUTS
#undef LN_LAUNCH
  } else {
    layernorm_wide_kernel<<<tokens, 256, 0, stream>>>(x, weight, bias, eps, out_f32, out_cd, cd_dtype, width, center);
  }
  TNX_CHECK_LAUNCH("layernorm");
  return 0;
}

// What follows a library matrix product: out = act(y + bias) + residual, eight elements a thread.
// y is bfloat16 [rows, width] (width a multiple of 8), bias and residual float32 and optional, out
// bfloat16 (may be y itself) or float32 (may be the residual itself).
__global__ void __launch_bounds__(256)
epilogue_kernel(const bf16_t* __restrict__ y, const float* __restrict__ bias, int act,
                const float* residual, void* out, int out_dtype, size_t chunks, int width8) {
  typedef __attribute__((ext_vector_type(8))) __bf16 b8;
  typedef __attribute__((ext_vector_type(4))) float f4;
  const size_t c = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (c >= chunks) return;
  const int col = (int)(c % width8) * 8;
  const b8 v = ((const b8*)y)[c];
  float f[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = (float)v[j];
  if (bias) {
    const f4 b0 = *(const f4*)(bias + col), b1 = *(const f4*)(bias + col + 4);
    f[0] += b0.x; f[1] += b0.y; f[2] += b0.z; f[3] += b0.w;
    f[4] += b1.x; f[5] += b1.y; f[6] += b1.z; f[7] += b1.w;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) f[j] = apply_act(f[j], act);
  if (residual) {
    const f4 r0 = ((const f4*)residual)[2 * c], r1 = ((const f4*)residual)[2 * c + 1];
    f[0] += r0.x; f[1] += r0.y; f[2] += r0.z; f[3] += r0.w;
    f[4] += r1.x; f[5] += r1.y; f[6] += r1.z; f[7] += r1.w;
  }
  if (out_dtype == TNX_F32) {
    ((f4*)out)[2 * c] = (f4){f[0], f[1], f[2], f[3]};
    ((f4*)out)[2 * c + 1] = (f4){f[4], f[5], f[6], f[7]};
  } else {
    b8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (bf16_t)f[j];
    ((b8*)out)[c] = o;
  }
}

extern "C" int tnx_epilogue(const void* y, const float* bias, int act, const float* residual, void* out,
                            int out_dtype, int rows, int width, hipStream_t stream) {
  TNX_REQUIRE(rows >= 0 && width > 0 && width % 8 == 0, "epilogue: width %d is not a multiple of 8", width);
  if (rows == 0) return 0;
  const size_t chunks = (size_t)rows * (width / 8);
  const size_t blocks = (chunks + 255) / 256;
  TNX_REQUIRE(blocks < (1ull << 31), "epilogue: too many elements");
  epilogue_kernel<<<(unsigned)blocks, 256, 0, stream>>>((const bf16_t*)y, bias, act, residual, out, out_dtype, chunks,
                                                        width / 8);
  TNX_CHECK_LAUNCH("epilogue");
  return 0;
}
