// What this device reaches at best, measured: the rate at which a kernel can read memory, and the rate of
// the matrix unit with operands in registers. A measurement sets a step's bytes and flops against these as
// well as against the published peaks. Nothing here is on the path of a model.
#include "common.h"

TNX_DEFINE_ERROR_API

// Every block reads its share of the buffer 16 bytes a lane, eight loads in flight a lane, marked as streaming
// (of the forms tried, plain or streaming loads, four or eight in flight, 4 to 32 blocks a compute unit,
// strided or in runs, this one read fastest: 6.8 TB/s against 5.5 to 6.3), and leaves the exclusive-or of what
// it read, so that no load can be left out.
__global__ void __launch_bounds__(256)
stream_read_kernel(const tnx_u32x4* __restrict__ data, size_t vectors, unsigned* __restrict__ out) {
  const size_t stride = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  tnx_u32x4 acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = (tnx_u32x4){0, 0, 0, 0};
  for (; i + 7 * stride < vectors; i += 8 * stride) {
    tnx_u32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(data + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc[u] ^= v[u];
  }
  for (; i < vectors; i += stride) acc[0] ^= __builtin_nontemporal_load(data + i);
  tnx_u32x4 a = acc[0];
#pragma unroll
  for (int u = 1; u < 8; ++u) a ^= acc[u];
  const unsigned x = a[0] ^ a[1] ^ a[2] ^ a[3];
  if (x == 0x9E3779B9u) out[blockIdx.x] = x;      // (all but never: the sums have to be made for it)
}

// `out` holds one word a block.
extern "C" int tnx_probe_stream_read(const void* data, size_t bytes, void* out, int blocks, hipStream_t stream) {
  TNX_REQUIRE(bytes % 16 == 0 && ((uintptr_t)data & 15) == 0, "stream_read: the buffer must be whole 16-byte vectors");
  TNX_REQUIRE(blocks > 0 && blocks <= 65536, "stream_read: %d blocks", blocks);
  stream_read_kernel<<<blocks, 256, 0, stream>>>((const tnx_u32x4*)data, bytes / 16, (unsigned*)out);
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
