// What this device reaches at best, measured: the rate at which a kernel can read memory, and the rate of
// the matrix unit with operands in registers. A measurement sets a step's bytes and flops against these as
// well as against the published peaks. Nothing here is on the path of a model.
#include "common.h"

TNX_DEFINE_ERROR_API

// Every block reads its share of the buffer 16 bytes a lane, four loads in flight a lane, and leaves the
// exclusive-or of what it read, so that no load can be left out.
__global__ void __launch_bounds__(256)
stream_read_kernel(const uint4* __restrict__ data, size_t vectors, unsigned* __restrict__ out) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  uint4 a = {0, 0, 0, 0}, b = a, c = a, d = a;
  for (; i + 3 * stride < vectors; i += 4 * stride) {
    const uint4 v0 = data[i], v1 = data[i + stride], v2 = data[i + 2 * stride], v3 = data[i + 3 * stride];
    a.x ^= v0.x, a.y ^= v0.y, a.z ^= v0.z, a.w ^= v0.w;
    b.x ^= v1.x, b.y ^= v1.y, b.z ^= v1.z, b.w ^= v1.w;
    c.x ^= v2.x, c.y ^= v2.y, c.z ^= v2.z, c.w ^= v2.w;
    d.x ^= v3.x, d.y ^= v3.y, d.z ^= v3.z, d.w ^= v3.w;
  }
  for (; i < vectors; i += stride) {
    const uint4 v = data[i];
    a.x ^= v.x, a.y ^= v.y, a.z ^= v.z, a.w ^= v.w;
  }
  const unsigned x = a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  if (x == 0x9E3779B9u) out[blockIdx.x] = x;      // (all but never: the sums have to be made for it)
}

// `out` holds one word a block.
extern "C" int tnx_probe_stream_read(const void* data, size_t bytes, void* out, int blocks, hipStream_t stream) {
  TNX_REQUIRE(bytes % 16 == 0 && ((uintptr_t)data & 15) == 0, "stream_read: the buffer must be whole 16-byte vectors");
  TNX_REQUIRE(blocks > 0 && blocks <= 65536, "stream_read: %d blocks", blocks);
  stream_read_kernel<<<blocks, 256, 0, stream>>>((const uint4*)data, bytes / 16, (unsigned*)out);
  TNX_CHECK_LAUNCH("stream_read");
  return 0;
}

// Each wave keeps four chains of `v_mfma_f32_32x32x16_bf16` going on operands it never reloads: 32 * 32 * 16
// multiply-adds an instruction, no memory traffic.
__global__ void __launch_bounds__(256)
mfma_loop_kernel(int iterations, float* __restrict__ out) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (bf16_t)(float)((threadIdx.x + i) & 3);
    b[i] = (bf16_t)(float)((threadIdx.x * 3 + i) & 1);
  }
  f32x16 c0 = {0}, c1 = {0}, c2 = {0}, c3 = {0};
  for (int it = 0; it < iterations; ++it) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == -1.f) out[blockIdx.x * 256 + threadIdx.x] = s;     // never: the sums are not negative
}

// Launches `blocks` blocks of four waves; the flops of the launch are blocks * 4 * iterations * 4 * 32768.
extern "C" int tnx_probe_mfma_loop(int blocks, int iterations, void* out, hipStream_t stream) {
  TNX_REQUIRE(blocks > 0 && blocks <= 65536 && iterations > 0, "mfma_loop: %d blocks, %d iterations", blocks, iterations);
  mfma_loop_kernel<<<blocks, 256, 0, stream>>>(iterations, (float*)out);
  TNX_CHECK_LAUNCH("mfma_loop");
  return 0;
}
