// A kernel that a part defined outside the package brings with it: a norm without mean or bias,
// y = x * w / sqrt(mean(x^2) + eps), statistics in float32. One block a row.
#include "common.h"

TNX_DEFINE_ERROR_API

__global__ void __launch_bounds__(256) toy_scale_norm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                             float eps, float* __restrict__ out_f32,
                                                             void* __restrict__ out_cd, int cd_dtype, int width) {
  __shared__ float partial[4];
  const float* row = x + (size_t)blockIdx.x * width;
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += 256) sum += row[i] * row[i];
  for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off, 64);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = sum;
  __syncthreads();
  const float inv = rsqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / width + eps);
  for (int i = threadIdx.x; i < width; i += 256) {
    const float y = row[i] * inv * w[i];
    if (out_f32) out_f32[(size_t)blockIdx.x * width + i] = y;
    if (out_cd) store_any(out_cd, cd_dtype, (size_t)blockIdx.x * width + i, y);
  }
}

extern "C" int tnx_toy_scale_norm(const float* x, const float* w, float eps, float* out_f32, void* out_cd,
                                  int cd_dtype, int rows, int width, hipStream_t stream) {
  TNX_REQUIRE(rows >= 0 && width > 0, "toy_scale_norm: bad sizes");
  TNX_REQUIRE(out_f32 || out_cd, "toy_scale_norm: no output asked for");
  if (rows == 0) return 0;
  toy_scale_norm_kernel<<<rows, 256, 0, stream>>>(x, w, eps, out_f32, out_cd, cd_dtype, width);
  TNX_CHECK_LAUNCH("toy_scale_norm");
  return 0;
}
