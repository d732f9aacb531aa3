// Attention over the paged cache.
//   qkv_write        bias, query scale, and the step's keys and values into their pages
//   attention_any    one wave per (token, head), any dtype, any head size in steps of 16: the float32 path
//                    and the fallback of the bfloat16 path
// Cache layout: keys [pages, kv_heads, page_size, head_size], values [pages, kv_heads, head_size, page_size].
// A token at position p of run r lies in page table[r][p / page_size] at place p % page_size.
// Reads are bounded by the reader's own position, so what an earlier holder left in a page is never seen.
#include "common.h"

TNX_DEFINE_ERROR_API

template <typename T>
__global__ void __launch_bounds__(256)
qkv_write_kernel(const T* __restrict__ qkv, const float* __restrict__ bias, float scale,
                 const int* __restrict__ positions, const int* __restrict__ token_request,
                 const int* __restrict__ table, int table_width, int page_size, int num_pages, T* __restrict__ q_out,
                 T* __restrict__ k_pages, T* __restrict__ v_pages, int num_heads, int num_kv, int head_size) {
  const int t = blockIdx.x;
  const int nq = num_heads * head_size, nk = num_kv * head_size;
  const int total = nq + 2 * nk;
  int page = -1, off = 0;
  if (num_kv > 0) {
    const int pos = positions[t];
    const int blk = pos / page_size;
    if (blk < table_width) page = table[token_request[t] * table_width + blk];
    if (page >= num_pages) page = -1;
    off = pos % page_size;
  }
  const T* row = qkv + (size_t)t * total;
  for (int i = threadIdx.x; i < total; i += 256) {
    float v = to_f32(row[i]);
    if (bias) v += bias[i];
    if (i < nq) {
      q_out[(size_t)t * nq + i] = from_f32<T>(v * scale);
    } else if (page >= 0) {
      if (i < nq + nk) {
        const int j = i - nq, h = j / head_size, d = j % head_size;
        k_pages[(((size_t)page * num_kv + h) * page_size + off) * head_size + d] = from_f32<T>(v);
      } else {
        const int j = i - nq - nk, h = j / head_size, d = j % head_size;
        v_pages[(((size_t)page * num_kv + h) * head_size + d) * page_size + off] = from_f32<T>(v);
      }
    }
  }
}

extern "C" int tnx_qkv_write(const void* qkv, int dtype, const float* bias, float scale, const int* positions,
                             const int* token_request, const int* table, int table_width, int page_size,
                             int num_pages, void* q_out, void* k_pages, void* v_pages, int tokens, int num_heads,
                             int num_kv, int head_size, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && num_heads > 0 && num_kv >= 0 && head_size > 0, "qkv_write: bad sizes");
  TNX_REQUIRE(page_size > 0 && table_width > 0, "qkv_write: bad page table");
  if (tokens == 0) return 0;
  if (dtype == TNX_F32)
    qkv_write_kernel<float><<<tokens, 256, 0, stream>>>((const float*)qkv, bias, scale, positions, token_request,
                                                        table, table_width, page_size, num_pages, (float*)q_out,
                                                        (float*)k_pages, (float*)v_pages, num_heads, num_kv, head_size);
  else
    qkv_write_kernel<bf16_t><<<tokens, 256, 0, stream>>>((const bf16_t*)qkv, bias, scale, positions, token_request,
                                                         table, table_width, page_size, num_pages, (bf16_t*)q_out,
                                                         (bf16_t*)k_pages, (bf16_t*)v_pages, num_heads, num_kv,
                                                         head_size);
  TNX_CHECK_LAUNCH("qkv_write");
  return 0;
}

// ------------------------------------------------------------------------------------------ any dtype

__device__ __forceinline__ float exp_for(float x, float) { return expf(x); }      // float32 path: full precision
__device__ __forceinline__ float exp_for(float x, bf16_t) { return __expf(x); }

// One wave per (token, head). Keys are taken 64 at a time, one per lane; the softmax is the running kind
// (maximum and sum carried in float32, earlier sums rescaled); the value sum is kept per lane for the
// head-size elements lane, lane + 64, ... Keys before `position - window + 1` are not read.
template <typename T>
__global__ void __launch_bounds__(256)
attention_any_kernel(const T* __restrict__ q, const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                     const int* __restrict__ positions, const int* __restrict__ token_request,
                     const int* __restrict__ table, int table_width, int page_size, int num_pages,
                     T* __restrict__ out, int tokens, int num_heads, int num_kv, int head_size, int window) {
  __shared__ float qs[4][256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long idx = (long long)blockIdx.x * 4 + wave;
  const bool active = idx < (long long)tokens * num_heads;
  const int t = active ? (int)(idx / num_heads) : 0;
  const int h = active ? (int)(idx % num_heads) : 0;
  const int kvh = h / (num_heads / num_kv);
  const int nq = num_heads * head_size;
  for (int d = lane; d < head_size; d += 64) qs[wave][d] = to_f32(q[(size_t)t * nq + h * head_size + d]);
  __syncthreads();
  if (!active) return;

  const int pos = positions[t];
  const int* tab = table + (size_t)token_request[t] * table_width;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};

  for (int c = (lo / 64) * 64; c <= pos; c += 64) {
    const int key = c + lane;
    const bool valid = key >= lo && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = tab[key / page_size];
      if (page >= 0 && page < num_pages) {
        const T* kp = k_pages + (((size_t)page * num_kv + kvh) * page_size + key % page_size) * head_size;
        float a = 0.f;
        for (int d = 0; d < head_size; d += 4) {
          a = fmaf(qs[wave][d], to_f32(kp[d]), a);
          a = fmaf(qs[wave][d + 1], to_f32(kp[d + 1]), a);
          a = fmaf(qs[wave][d + 2], to_f32(kp[d + 2]), a);
          a = fmaf(qs[wave][d + 3], to_f32(kp[d + 3]), a);
        }
        s = a;
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? exp_for(s - m_new, T()) : 0.f;
    const float alpha = exp_for(m - m_new, T());
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int a = 0; a < 4; ++a) acc[a] *= alpha;
    // values: 16 keys at a time lie in one page (page sizes are multiples of 16)
#pragma unroll
    for (int grp = 0; grp < 4; ++grp) {
      const int key0 = c + 16 * grp;
      if (key0 > pos || key0 + 15 < lo) continue;
      const int page = tab[key0 / page_size];
      if (page < 0 || page >= num_pages) continue;
      const int off0 = key0 % page_size;
      const T* vbase = v_pages + ((size_t)page * num_kv + kvh) * head_size * page_size + off0;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const float pj = __shfl(p, 16 * grp + j, 64);
        const int kj = key0 + j;
        if (kj < lo || kj > pos) continue;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          const int d = lane + 64 * a;
          if (d < head_size) acc[a] = fmaf(pj, to_f32(vbase[(size_t)d * page_size + j]), acc[a]);
        }
      }
    }
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int d = lane + 64 * a;
    if (d < head_size) out[(size_t)t * nq + h * head_size + d] = from_f32<T>(acc[a] * inv);
  }
}

extern "C" int tnx_attention_any(const void* q, int dtype, const void* k_pages, const void* v_pages,
                                 const int* positions, const int* token_request, const int* table, int table_width,
                                 int page_size, int num_pages, void* out, int tokens, int num_heads, int num_kv,
                                 int head_size, int window, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && num_heads > 0 && num_kv > 0 && num_heads % num_kv == 0, "attention: bad head counts");
  TNX_REQUIRE(head_size % 16 == 0 && head_size >= 16 && head_size <= 256,
              "attention: head size %d is not a multiple of 16 in [16, 256]", head_size);
  TNX_REQUIRE(page_size % 16 == 0 && page_size > 0, "attention: page size %d is not a multiple of 16", page_size);
  if (tokens == 0) return 0;
  const long long waves = (long long)tokens * num_heads;
  const long long blocks = (waves + 3) / 4;
  TNX_REQUIRE(blocks < (1ll << 31), "attention: too many (token, head) pairs");
  if (dtype == TNX_F32)
    attention_any_kernel<float><<<(unsigned)blocks, 256, 0, stream>>>(
        (const float*)q, (const float*)k_pages, (const float*)v_pages, positions, token_request, table, table_width,
        page_size, num_pages, (float*)out, tokens, num_heads, num_kv, head_size, window);
  else
    attention_any_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, positions, token_request, table,
        table_width, page_size, num_pages, (bf16_t*)out, tokens, num_heads, num_kv, head_size, window);
  TNX_CHECK_LAUNCH("attention_any");
  return 0;
}
