// Attention over the paged cache.
//   qkv_write        bias, query scale, and the step's keys and values into their pages
//   attention_any    one wave per (token, head), any dtype, any head size in steps of 16: the float32 path
//                    and the fallback of the bfloat16 path
// Cache layout: keys [pages, kv_heads, page_size, head_size], values [pages, kv_heads, head_size, page_size].
// A token at position p of run r lies in page table[r][p / page_size] at place p % page_size.
// Reads are bounded by the reader's own position, so what an earlier holder left in a page is never seen.
#include "common.h"
#include "tnx_attention.h"
#include <mutex>

TNX_DEFINE_ERROR_API

// One thread takes 8 consecutive elements of a token's [q | k | v] row: a query chunk goes to the dense
// query matrix scaled, a key chunk to its page as it is (head-size elements are contiguous there), a value
// chunk element by element (values lie transposed inside a page). Chunks are read and written 16 bytes at a
// time in bfloat16 (rows and pages are 16-byte aligned there: the launcher sees to it).
template <typename T>
__device__ __forceinline__ void load8(const T* p, float* v) {
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = to_f32(p[j]);
}
template <>
__device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float* v) {
  const bf16x8 x = *(const bf16x8*)p;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = (float)x[j];
}
template <typename T>
__device__ __forceinline__ void store8(T* p, const float* v) {
#pragma unroll
  for (int j = 0; j < 8; ++j) p[j] = from_f32<T>(v[j]);
}
template <>
__device__ __forceinline__ void store8<bf16_t>(bf16_t* p, const float* v) {
  bf16x8 x;
#pragma unroll
  for (int j = 0; j < 8; ++j) x[j] = (bf16_t)v[j];
  *(bf16x8*)p = x;
}

template <typename T>
__global__ void __launch_bounds__(256)
qkv_write_kernel(const T* __restrict__ qkv, const float* __restrict__ bias, float scale,
                 const int* __restrict__ positions, const int* __restrict__ token_request,
                 const int* __restrict__ table, int table_width, int page_size, int num_pages, T* __restrict__ q_out,
                 T* __restrict__ k_pages, T* __restrict__ v_pages, int num_heads, int num_kv, int head_size,
                 const int* __restrict__ run_start, int values_of_single_tokens_only,
                 const float* __restrict__ turn_a, const float* __restrict__ turn_b, int turn_rows, int page_pad) {
  const size_t page_stride = (size_t)num_kv * page_size * head_size + page_pad;     // elements from page to page
  const int t = blockIdx.x;
  const int nq = num_heads * head_size, nk = num_kv * head_size;
  const int total = nq + 2 * nk;
  const int i0 = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (i0 >= total) return;
  if (values_of_single_tokens_only && i0 >= nq + nk) {   // the values of longer runs are written by tiles
    const int r = token_request[t];
    if (run_start[r + 1] - run_start[r] > 1) return;
  }
  float v[8];
  load8<T>(qkv + (size_t)t * total + i0, v);
  if (bias) {
    const f32x4 b0 = *(const f32x4*)(bias + i0), b1 = *(const f32x4*)(bias + i0 + 4);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[j] += b0[j];
      v[4 + j] += b1[j];
    }
  }
  if (turn_a && i0 < nq + nk) {
    // a position encoding that turns queries and keys pair by pair: x[d] becomes a[p][d] x[d] + b[p][d] x[d ^ 1]
    // (the eight elements of a thread lie in one head: head sizes are multiples of 8)
    const size_t at = (size_t)min(max(positions[t], 0), turn_rows - 1) * head_size + i0 % head_size;
    float w[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) w[j] = turn_a[at + j] * v[j] + turn_b[at + j] * v[j ^ 1];
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = w[j];
  }
  if (i0 < nq) {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] *= scale;
    store8<T>(q_out + (size_t)t * nq + i0, v);
    return;
  }
  const int pos = positions[t];
  const int blk = pos / page_size, off = pos % page_size;
  int page = -1;
  if (blk < table_width) page = table[token_request[t] * table_width + blk];
  if (page < 0 || page >= num_pages) return;
  if (i0 < nq + nk) {
    const int j0 = i0 - nq, h = j0 / head_size, d = j0 % head_size;
    store8<T>(k_pages + (size_t)page * page_stride + ((size_t)h * page_size + off) * head_size + d, v);
  } else {
    const int j0 = i0 - nq - nk, h = j0 / head_size, d = j0 % head_size;
    T* dst = v_pages + (size_t)page * page_stride + ((size_t)h * head_size + d) * page_size + off;
#pragma unroll
    for (int j = 0; j < 8; ++j) dst[(size_t)j * page_size] = from_f32<T>(v[j]);
  }
}

// The values of a tile of up to 128 consecutive tokens of one run, one kv head a block. Values lie transposed
// in a page (consecutive positions are neighbours): a thread takes 8 consecutive positions and 8 consecutive
// elements of the head, reads them as 8 rows of the product, 16 bytes each, and writes them as 8 rows of the
// page, 16 bytes each; the lanes of a wave are 8 groups of positions (a row of a 64-token page: 128 bytes a
// store) by 8 chunks of elements (128 bytes of a token's row a load). Groups of 8 are aligned to positions, not
// to the tile; a group that the tile covers in part is written element by element.
constexpr int VT_TOKENS = 128;

__global__ void __launch_bounds__(256)
value_tiles_kernel(const bf16_t* __restrict__ qkv, const float* __restrict__ bias, const int* __restrict__ run_start,
                   const int* __restrict__ cached_lens, const int* __restrict__ table, int table_width,
                   int page_size, int num_pages, const int* __restrict__ tile_run,
                   const int* __restrict__ tile_q0, bf16_t* __restrict__ v_pages, int num_heads, int num_kv,
                   int head_size, int page_pad) {
  const size_t page_stride = (size_t)num_kv * page_size * head_size + page_pad;
  const int run = tile_run[blockIdx.x], q0 = tile_q0[blockIdx.x], kvh = blockIdx.y;
  const int t0 = run_start[run] + q0;
  const int n = min(VT_TOKENS, run_start[run + 1] - t0);
  const int p0 = cached_lens[run] + q0;   // position of the tile's first token
  const int total = (num_heads + 2 * num_kv) * head_size;
  const int col0 = (num_heads + num_kv) * head_size + kvh * head_size;
  const int* tab = table + (size_t)run * table_width;
  const int groups = (p0 + n - 1) / 8 - p0 / 8 + 1;
  const int chunks = head_size / 8;
  // item = (chunk / 8, group / 8, chunk % 8, group % 8): the groups run fastest within a wave's 64 lanes
  const int group_blocks = (groups + 7) / 8;
  for (int item = threadIdx.x; item < group_blocks * 8 * ((chunks + 7) / 8) * 8; item += 256) {
    const int g = (item >> 6) % group_blocks * 8 + (item & 7);
    const int c = (item >> 6) / group_blocks * 8 + ((item >> 3) & 7);
    if (g >= groups || c >= chunks) continue;
    const int pos = (p0 / 8 + g) * 8;                 // first position of the group
    const int blk = pos / page_size;
    const int page = blk < table_width ? tab[blk] : -1;
    if (page < 0 || page >= num_pages) continue;
    const int i0 = pos - p0;                           // the group's first token within the tile; may be < 0
    bf16x8 rows[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = min(max(i0 + j, 0), n - 1);        // (tokens outside the tile are read somewhere and not written)
      rows[j] = *(const bf16x8*)(qkv + (size_t)(t0 + i) * total + col0 + c * 8);
    }
    if (bias) {
      const f32x4 b0 = *(const f32x4*)(bias + col0 + c * 8), b1 = *(const f32x4*)(bias + col0 + c * 8 + 4);
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) rows[j][e] = (bf16_t)((float)rows[j][e] + (e < 4 ? b0[e] : b1[e - 4]));
    }
    bf16_t* dst = v_pages + (size_t)page * page_stride + ((size_t)kvh * head_size + c * 8) * page_size + pos % page_size;
    const bool whole = i0 >= 0 && i0 + 8 <= n;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (whole) {
        bf16x8 v;
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = rows[j][e];
        *(bf16x8*)(dst + (size_t)e * page_size) = v;
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (i0 + j >= 0 && i0 + j < n) dst[(size_t)e * page_size + j] = rows[j][e];
      }
    }
  }
}

// With `num_tiles > 0` (bfloat16 only) the values of the runs that `tile_run` / `tile_q0` cut into tiles of
// `tile_tokens` tokens are written by tiles, and the token-wise kernel leaves them out.
extern "C" int tnx_qkv_write(const void* qkv, int dtype, const float* bias, float scale, const int* positions,
                             const int* token_request, const int* table, int table_width, int page_size,
                             int num_pages, void* q_out, void* k_pages, void* v_pages, int tokens, int num_heads,
                             int num_kv, int head_size, const int* run_start, const int* cached_lens,
                             const int* tile_run, const int* tile_q0, int num_tiles, int tile_tokens,
                             const float* turn_a, const float* turn_b, int turn_rows, int page_pad,
                             hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && num_heads > 0 && num_kv >= 0 && head_size > 0, "qkv_write: bad sizes");
  TNX_REQUIRE(page_pad >= 0 && page_pad % 8 == 0, "qkv_write: pages are %d elements apart beyond their size, not a "
              "multiple of 8 from 0 up", page_pad);
  TNX_REQUIRE((turn_a == nullptr) == (turn_b == nullptr) && (!turn_a || turn_rows > 0),
              "qkv_write: the pair-turning tables come both or not at all, with their number of rows");
  TNX_REQUIRE(page_size > 0 && table_width > 0, "qkv_write: bad page table");
  if (tokens == 0) return 0;
  TNX_REQUIRE(head_size % 8 == 0, "qkv_write: head size %d is not a multiple of 8", head_size);
  TNX_REQUIRE(((uintptr_t)qkv | (uintptr_t)bias | (uintptr_t)q_out | (uintptr_t)k_pages | (uintptr_t)v_pages) % 16 == 0,
              "qkv_write: the projections, the bias, the queries and the pages must be 16-byte aligned");
  const bool by_tiles = num_tiles > 0 && num_kv > 0;
  if (by_tiles) {
    TNX_REQUIRE(dtype == TNX_BF16, "qkv_write: values are written by tiles in bfloat16 only");
    TNX_REQUIRE(tile_tokens > 0 && tile_tokens <= VT_TOKENS, "qkv_write: tiles of %d tokens, at most %d fit",
                tile_tokens, VT_TOKENS);
    TNX_REQUIRE(page_size % 8 == 0, "qkv_write: page size %d is not a multiple of 8", page_size);
    TNX_REQUIRE(run_start && cached_lens && tile_run && tile_q0, "qkv_write: tiles without their tables");
    TNX_REQUIRE(num_kv <= 65535, "qkv_write: too many heads");
  }
  const dim3 grid(tokens, ((num_heads + 2 * num_kv) * head_size / 8 + 255) / 256);
  if (dtype == TNX_F32)
    qkv_write_kernel<float><<<grid, 256, 0, stream>>>((const float*)qkv, bias, scale, positions, token_request,
                                                        table, table_width, page_size, num_pages, (float*)q_out,
                                                        (float*)k_pages, (float*)v_pages, num_heads, num_kv, head_size,
                                                        run_start, 0, turn_a, turn_b, turn_rows, page_pad);
  else
    qkv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)qkv, bias, scale, positions, token_request,
                                                         table, table_width, page_size, num_pages, (bf16_t*)q_out,
                                                         (bf16_t*)k_pages, (bf16_t*)v_pages, num_heads, num_kv,
                                                         head_size, run_start, by_tiles ? 1 : 0, turn_a, turn_b,
                                                         turn_rows, page_pad);
  TNX_CHECK_LAUNCH("qkv_write");
  if (by_tiles) {
    value_tiles_kernel<<<dim3(num_tiles, num_kv), 256, 0, stream>>>(
        (const bf16_t*)qkv, bias, run_start, cached_lens, table, table_width, page_size, num_pages, tile_run, tile_q0,
        (bf16_t*)v_pages, num_heads, num_kv, head_size, page_pad);
    TNX_CHECK_LAUNCH("value_tiles");
  }
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
                     T* __restrict__ out, int tokens, int num_heads, int num_kv, int head_size, int window,
                     int page_pad) {
  __shared__ float qs[4][256];
  const size_t page_stride = (size_t)num_kv * page_size * head_size + page_pad;
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
        const T* kp = k_pages + (size_t)page * page_stride + ((size_t)kvh * page_size + key % page_size) * head_size;
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
      const T* vbase = v_pages + (size_t)page * page_stride + (size_t)kvh * head_size * page_size + off0;
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
                                 int head_size, int window, int page_pad, hipStream_t stream) {
  TNX_REQUIRE(tokens >= 0 && num_heads > 0 && num_kv > 0 && num_heads % num_kv == 0, "attention: bad head counts");
  TNX_REQUIRE(page_pad >= 0 && page_pad % 8 == 0, "attention: bad distance between pages");
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
        page_size, num_pages, (float*)out, tokens, num_heads, num_kv, head_size, window, page_pad);
  else
    attention_any_kernel<bf16_t><<<(unsigned)blocks, 256, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, positions, token_request, table,
        table_width, page_size, num_pages, (bf16_t*)out, tokens, num_heads, num_kv, head_size, window, page_pad);
  TNX_CHECK_LAUNCH("attention_any");
  return 0;
}

// ------------------------------------------------------------------------------------------ bfloat16, prompts


#define PREFILL_Q_TILE 128  // queries per block: four waves of 32
#define LOG2E 1.4426950408889634f


// Flash-style attention of a run of queries over its request's pages, on MFMA 16x16x32.
// A wave owns 32 queries (two column blocks of 16) and walks the keys 64 at a time. It computes the
// transposed scores S^T = K Q^T, so that the accumulator layout (lane = query, four consecutive keys per
// register group) is at once the layout of the B operand of O^T += V^T P^T: the probabilities never leave
// their registers. The keys of a 32-key MFMA step are taken in the order (16b + 4g + i), b the half, g the
// lane group, which is the order the accumulators hold them in; the values are read in the same order.
// NDB bounds the head size (16 * NDB); smaller head sizes run with the blocks beyond them switched off.
template <int NDB>
__global__ void __launch_bounds__(256)
attention_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                         const bf16_t* __restrict__ v_pages, const int* __restrict__ run_start,
                         const int* __restrict__ cached_lens, const int* __restrict__ table, int table_width,
                         int page_size, int num_pages, const int* __restrict__ tile_run,
                         const int* __restrict__ tile_q0, bf16_t* __restrict__ out, int num_heads, int num_kv,
                         int head_size, int window, int page_pad) {
  constexpr int NKS = (NDB + 1) / 2;  // MFMA steps of 32 over the head size
  const size_t page_stride = (size_t)num_kv * page_size * head_size + page_pad;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x / num_heads, h = blockIdx.x % num_heads;
  const int run = tile_run[tile];
  const int kvh = h / (num_heads / num_kv);
  const int t0 = run_start[run], qlen = run_start[run + 1] - t0, cached = cached_lens[run];
  const int qw0 = tile_q0[tile] + 32 * wave;
  if (qw0 >= qlen) return;
  const int nq = num_heads * head_size;
  const int* tab = table + (size_t)run * table_width;
  const int total = cached + qlen;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const int ndb = head_size / 16;

  bf16x8 qf[2][NKS];
  int qpos[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    qpos[qb] = cached + qi;
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      const int d0 = 32 * s + 8 * g;
      qf[qb][s] = (qi < qlen && d0 < head_size) ? *(const bf16x8*)(q + (size_t)(t0 + qi) * nq + h * head_size + d0)
                                                : zero8;
    }
  }
  const int last_q = cached + min(qw0 + 31, qlen - 1);          // the wave's last query position
  const int first_q = cached + qw0;
  const int lo = window > 0 ? max(0, first_q - window + 1) : 0;  // no query of the wave reads before this

  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  f32x4 o[NDB][2];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) o[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  for (int tile0 = (lo / 64) * 64; tile0 <= last_q; tile0 += 64) {
    f32x4 s[4][2];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const int key0 = tile0 + 16 * kb;
      f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
      int page = -1;
      if (key0 <= last_q) page = tab[key0 / page_size];
      if (page >= 0 && page < num_pages) {
        const bf16_t* kbase =
            k_pages + (size_t)page * page_stride + ((size_t)kvh * page_size + key0 % page_size + r) * head_size;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const int d0 = 32 * ks + 8 * g;
          const bf16x8 kf = d0 < head_size ? *(const bf16x8*)(kbase + d0) : zero8;
          a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[0][ks], a0, 0, 0, 0);
          a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[1][ks], a1, 0, 0, 0);
        }
      }
      s[kb][0] = a0;
      s[kb][1] = a1;
    }
    // what a query may not see becomes -inf: later keys, keys before its window, keys without a page
    const bool full_tile = tile0 + 63 <= first_q && (window <= 0 || tile0 > last_q - window);
    if (!full_tile) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = tile0 + 16 * kb + 4 * g + i;
            const bool ok = key <= qpos[qb] && (window <= 0 || key > qpos[qb] - window);
            if (!ok) s[kb][qb][i] = -INFINITY;
          }
    }
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[kb][qb][i]);
      mx = rows_max(mx);
      const float m_new = fmaxf(m[qb], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __expf(m[qb] - m_safe);
      float sum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __expf(s[kb][qb][i] - m_safe);
          s[kb][qb][i] = p;
          sum += p;
        }
      sum = rows_sum(sum);
      l[qb] = l[qb] * alpha + sum;
      m[qb] = m_new;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[db][qb][i] *= alpha;
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (tile0 + 32 * t > last_q) continue;
      bf16x8 pb[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int j = 0; j < 8; ++j) pb[qb][j] = (bf16_t)s[2 * t + (j >> 2)][qb][j & 3];
      const bf16_t* vbase[2];
      bool vok[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int key0 = tile0 + 32 * t + 16 * b;
        int page = -1;
        if (key0 <= last_q) page = tab[key0 / page_size];
        vok[b] = page >= 0 && page < num_pages;
        vbase[b] = v_pages + (size_t)(vok[b] ? page : 0) * page_stride + (size_t)kvh * head_size * page_size +
                   key0 % page_size + 4 * g;
      }
      const bool tail = tile0 + 32 * t + 32 > total;   // some keys of this step lie beyond the request
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        if (db >= ndb) continue;
        const int d = 16 * db + r;
        bf16x8 vf;
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          bf16x4 v4 = {0, 0, 0, 0};
          if (vok[b]) v4 = *(const bf16x4*)(vbase[b] + (size_t)d * page_size);
          if (tail) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (tile0 + 32 * t + 16 * b + 4 * g + i >= total) v4[i] = 0;
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) vf[4 * b + i] = v4[i];
        }
        o[db][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[0], o[db][0], 0, 0, 0);
        o[db][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pb[1], o[db][1], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    if (qi >= qlen) continue;
    const float inv = 1.f / l[qb];
    bf16_t* orow = out + (size_t)(t0 + qi) * nq + h * head_size;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      if (db >= ndb) continue;
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[db][qb][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v4;
    }
  }
}

// The same computation with the keys and values of a tile staged through LDS, once for the four waves of a
// block, and the next tile's global loads in flight while the current one is computed (two LDS buffers, one
// barrier a tile). Page sizes that are powers of two. K is staged as [key][head_size + pad] and V^T as
// [head_size][64 + pad].
// FAST is the case of a head size of exactly 16 * NDB and pages of 64 keys or more: a tile then lies within
// one page, whose number is one scalar lookup, every thread's place within the tile is fixed, and no part of
// the inner loops depends on a size known only at run time.
// Where the rows lie in LDS is chosen by measurement of the fragment reads (16 rows by 4 chunks of 16 bytes
// a wave): rows of 16 (2 n + 1) bytes, the usual padding, take twice the time of rows of 32 (2 n + 1) bytes,
// which are read at the full rate, as are unpadded 256-byte rows whose chunk c lies at c ^ (row's index among
// the 16 that are read together). The 8-byte reads of the general case's values want 16 (2 n + 1).
// With GROUPS = 2 a block has two such sets of four waves for the same 128 queries: the first takes the
// first half of the key tiles and the second the rest, each through LDS buffers of its own, and their
// partial results (maximum, sum, weighted values, float32) meet in LDS at the end. The tile of the last
// queries of a long prompt, which sees the most keys, then takes half as long, and it is that tile which the
// launch waits for.
template <int NDB, bool FAST>
struct PrefillTileLayout {
  static constexpr int DMAX = 16 * NDB;
  static constexpr bool SWIZZLED = FAST && NDB == 8;            // 256-byte key rows, chunks exchanged
  static constexpr int KSTR = SWIZZLED ? DMAX : DMAX + 16;      // elements per staged key row
  static constexpr int VSTR = FAST ? 64 + 16 : 64 + 8;          // per staged value row (one element, 64 keys)
  static constexpr int KBUF = 64 * KSTR, VBUF = DMAX * VSTR;
};
template <int NDB, bool FAST, int GROUPS>
__global__ void __launch_bounds__(256 * GROUPS, (NDB <= 8 && GROUPS == 1 ? 2 : 1))
attention_prefill_lds_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                             const bf16_t* __restrict__ v_pages, const int* __restrict__ run_start,
                             const int* __restrict__ cached_lens, const int* __restrict__ table, int table_width,
                             int page_shift, int num_pages, const int* __restrict__ tile_run,
                             const int* __restrict__ tile_q0, bf16_t* __restrict__ out, int num_heads, int num_kv,
                             int head_size, int window, int page_pad) {
  constexpr int NKS = (NDB + 1) / 2;
  constexpr int DMAX = 16 * NDB;
  using Layout = PrefillTileLayout<NDB, FAST>;
  constexpr bool SWZ = Layout::SWIZZLED;
  constexpr int KSTR = Layout::KSTR, VSTR = Layout::VSTR, KBUF = Layout::KBUF, VBUF = Layout::VBUF;
  constexpr int KCH = (64 * DMAX / 8 + 255) / 256;   // 16-byte chunks a thread stages per tile, keys
  constexpr int VCH = (DMAX * 8 + 255) / 256;        // and values
  extern __shared__ __attribute__((aligned(16))) bf16_t smem[];
  const int grp = GROUPS == 1 ? 0 : threadIdx.x >> 8;      // which set of four waves
  bf16_t* ks_buf = smem + grp * 2 * (KBUF + VBUF);          // [2][KBUF]
  bf16_t* vs_buf = ks_buf + 2 * KBUF;                       // [2][VBUF]

  const int tid = threadIdx.x & 255, lane = tid & 63, wave = tid >> 6;   // within the set
  const int r = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x / num_heads, h = blockIdx.x % num_heads;
  const int run = tile_run[tile];
  const int kvh = h / (num_heads / num_kv);
  const int t0 = run_start[run], qlen = run_start[run + 1] - t0, cached = cached_lens[run];
  const int q0 = tile_q0[tile];
  const int qw0 = q0 + 32 * wave;
  const bool wave_on = qw0 < qlen;
  const int nq = num_heads * head_size;
  const int* tab = table + (size_t)run * table_width;
  const int total = cached + qlen;
  const int page_size = 1 << page_shift, pmask = page_size - 1;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  if (FAST) head_size = DMAX;
  const int ndb = head_size / 16;
  const int cpr = head_size / 8;            // chunks per key row
  const size_t head_stride = (size_t)page_size * head_size;
  const size_t page_stride = (size_t)num_kv * head_stride + page_pad;

  bf16x8 qf[2][NKS];
  int qpos[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    qpos[qb] = cached + qi;
#pragma unroll
    for (int s = 0; s < NKS; ++s) {
      const int d0 = 32 * s + 8 * g;
      qf[qb][s] = (qi < qlen && d0 < head_size) ? *(const bf16x8*)(q + (size_t)(t0 + qi) * nq + h * head_size + d0)
                                                : zero8;
    }
  }
  // block-wide range of key tiles; each wave computes only the tiles its own queries can see
  const int blk_last = cached + min(q0 + PREFILL_Q_TILE - 1, qlen - 1);
  const int blk_lo = window > 0 ? max(0, cached + q0 - window + 1) : 0;
  const int last_q = cached + min(qw0 + 31, qlen - 1);
  const int first_q = cached + qw0;
  const int lo = window > 0 ? max(0, first_q - window + 1) : 0;

  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  f32x4 o[NDB][2];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) o[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  bf16x8 kreg[KCH], vreg[VCH];
  // Global loads of one tile into registers. Keys beyond the request read the request's last key (a valid
  // place); they are masked by position below, and their values are zeroed when the tile is staged.
  // No load here depends on a branch (a thread with no chunk of its own reads the last chunk again), and
  // the page numbers are fetched for all chunks before the first chunk is.
  const int k_chunks = 64 * cpr, v_chunks = head_size * 8;
  int kc_key[KCH], kc_dc[KCH], vc_d[VCH], vc_kc[VCH];
#pragma unroll
  for (int j = 0; j < KCH; ++j) {
    const int c = min(tid + 256 * j, k_chunks - 1);
    kc_key[j] = c / cpr;
    kc_dc[j] = c - kc_key[j] * cpr;
  }
#pragma unroll
  for (int j = 0; j < VCH; ++j) {
    const int c = min(tid + 256 * j, v_chunks - 1);
    vc_d[j] = c >> 3;
    vc_kc[j] = c & 7;
  }
  // Page numbers are looked up one tile earlier than the data they lead to, so that the data loads of the
  // next tile can be issued without waiting for a lookup.
  int kpage[KCH], vpage[VCH];
  int tile_page = 0;                        // FAST: the one page of the tile looked up last
  int koff[KCH], voff[VCH];                 // FAST: a thread's chunks within the tile's part of the page
#pragma unroll
  for (int j = 0; j < KCH; ++j) koff[j] = kc_key[j] * head_size + kc_dc[j] * 8;
#pragma unroll
  for (int j = 0; j < VCH; ++j) voff[j] = vc_d[j] * page_size + 8 * vc_kc[j];
  auto lookup = [&](int tile0) {
    if (FAST) {
      tile_page = tab[min(tile0, total - 1) >> page_shift];
      return;
    }
#pragma unroll
    for (int j = 0; j < KCH; ++j) kpage[j] = tab[min(tile0 + kc_key[j], total - 1) >> page_shift];
#pragma unroll
    for (int j = 0; j < VCH; ++j) vpage[j] = tab[min(tile0 + 8 * vc_kc[j], (total - 1) & ~7) >> page_shift];
  };
  auto fetch = [&](int tile0) {
    if (FAST) {
      // keys of the page beyond the request are read as they lie: their scores are masked by position and
      // their values are zeroed when the tile is staged
      const int page = min(max(tile_page, 0), num_pages - 1);
      const size_t base = (size_t)page * page_stride + (size_t)kvh * head_stride;
      const bf16_t* kb = k_pages + base + (size_t)(tile0 & pmask) * head_size;
      const bf16_t* vb = v_pages + base + (tile0 & pmask);
#pragma unroll
      for (int j = 0; j < KCH; ++j) kreg[j] = *(const bf16x8*)(kb + koff[j]);
#pragma unroll
      for (int j = 0; j < VCH; ++j) vreg[j] = *(const bf16x8*)(vb + voff[j]);
      return;
    }
#pragma unroll
    for (int j = 0; j < KCH; ++j) {
      const int key = min(tile0 + kc_key[j], total - 1);
      const int page = min(max(kpage[j], 0), num_pages - 1);
      kreg[j] = *(const bf16x8*)(k_pages + (size_t)page * page_stride + (size_t)kvh * head_stride +
                                 (size_t)(key & pmask) * head_size + kc_dc[j] * 8);
    }
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      const int key = min(tile0 + 8 * vc_kc[j], (total - 1) & ~7);
      const int page = min(max(vpage[j], 0), num_pages - 1);
      vreg[j] = *(const bf16x8*)(v_pages + (size_t)page * page_stride + (size_t)kvh * head_stride +
                                 (size_t)vc_d[j] * page_size + (key & pmask));
    }
  };
  auto stage = [&](int buf, int tile0) {
    bf16_t* kd = ks_buf + buf * KBUF;
    bf16_t* vd = vs_buf + buf * VBUF;
#pragma unroll
    for (int j = 0; j < KCH; ++j)
      if (tid + 256 * j < k_chunks) {
        // swizzled: chunk c of key row k lies at c ^ (4 ((k / 8) % 4) + k % 4), the row's index among the 16
        // that a fragment read takes together (see `read_keys`)
        const int dc = SWZ ? (kc_dc[j] ^ ((((kc_key[j] >> 3) & 3) << 2) | (kc_key[j] & 3))) : kc_dc[j];
        *(bf16x8*)(kd + kc_key[j] * KSTR + dc * 8) = kreg[j];
      }
#pragma unroll
    for (int j = 0; j < VCH; ++j) {
      if (tid + 256 * j < v_chunks) {
        bf16x8 v = vreg[j];
        const int k0 = tile0 + 8 * vc_kc[j];
        // Keys beyond the request, and keys that no query of the block sees any more (their pages may have
        // been given back: the lookup then leads to some other page): their probabilities are zero, and
        // their values must not be NaN.
        if (k0 + 8 > total || k0 < blk_lo) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (k0 + e >= total || k0 + e < blk_lo) v[e] = 0;
        }
        *(bf16x8*)(vd + vc_d[j] * VSTR + vc_kc[j] * 8) = v;
      }
    }
  };

  int buf = 0;
  // the block's key tiles, in equal shares for its sets of waves; every set passes the same number of
  // barriers, a set whose share is shorter (or empty) idles at the end
  const int blk_begin = (blk_lo / 64) * 64;
  const int share = ((blk_last - blk_begin) / 64 + GROUPS) / GROUPS;      // tiles a set, rounded up
  const int tile_begin = blk_begin + grp * share * 64;
  const int tile_last = min(blk_last, tile_begin + share * 64 - 1);         // the last key of this set
  lookup(tile_begin);               // past the request the lookups repeat its last page: harmless
  fetch(tile_begin);
  lookup(tile_begin + 64);
  for (int it = 0, tile0 = tile_begin; it < share; ++it, tile0 += 64, buf ^= 1) {
    const bool live = tile0 <= tile_last;
    if (live) stage(buf, tile0);
    __syncthreads();
    if (tile0 + 64 <= tile_last) {
      fetch(tile0 + 64);
      lookup(tile0 + 128);
    }
    if (!live || !wave_on || tile0 > last_q || tile0 + 63 < lo) continue;
    const bf16_t* kd = ks_buf + buf * KBUF;
    const bf16_t* vd = vs_buf + buf * VBUF;

    // the keys of 16 rows are read from LDS while the products of the 16 rows before them run (where the
    // registers allow a second set of them: head sizes up to 128)
    constexpr int KA = NDB <= 8 ? 2 : 1;
    f32x4 s[4][2];
    bf16x8 kf[KA][NKS];
    // FAST: row r of key block kb is key 32 (kb / 2) + 8 (r / 4) + 4 (kb % 2) + r % 4 of the tile, so that the
    // probabilities a lane holds are those of 8 consecutive keys and the values are read 16 bytes a lane;
    // otherwise key 16 kb + r, the values being read in two halves in the accumulators' order
    auto read_keys = [&](int kb, bf16x8* dst) {
      const int row = FAST ? 32 * (kb >> 1) + 8 * (r >> 2) + 4 * (kb & 1) + (r & 3) : 16 * kb + r;
      const bf16_t* krow = kd + row * KSTR;
      const int flip = SWZ ? r : 0;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
        dst[ks] = (32 * ks + 8 * g < head_size) ? *(const bf16x8*)(krow + ((4 * ks + g) ^ flip) * 8) : zero8;
    };
    if (KA == 2) read_keys(0, kf[0]);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      if (KA == 2) {
        if (kb < 3) read_keys(kb + 1, kf[(kb + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);    // the reads stay ahead of the products, as written
      } else {
        read_keys(kb, kf[0]);
      }
      const bf16x8* kc = kf[KA == 2 ? kb & 1 : 0];
      f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kc[ks], qf[0][ks], a0, 0, 0, 0);
        a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kc[ks], qf[1][ks], a1, 0, 0, 0);
      }
      s[kb][0] = a0;
      s[kb][1] = a1;
      if (KA == 2) __builtin_amdgcn_sched_barrier(0);
    }
    const bool full_tile = tile0 + 63 <= first_q && (window <= 0 || tile0 > last_q - window);
    if (!full_tile) {
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int qb = 0; qb < 2; ++qb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = FAST ? tile0 + 32 * (kb >> 1) + 8 * g + 4 * (kb & 1) + i : tile0 + 16 * kb + 4 * g + i;
            const bool ok = key <= qpos[qb] && (window <= 0 || key > qpos[qb] - window);
            if (!ok) s[kb][qb][i] = -INFINITY;
          }
    }
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) mx = fmaxf(mx, s[kb][qb][i]);
      mx = rows_max(mx);
      const float m_new = fmaxf(m[qb], mx);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      // e^(x - m) as 2^(x log2 e - m log2 e): one multiply-add and the hardware's 2^x
      const float m_log2 = m_safe * LOG2E;
      const float alpha = __builtin_amdgcn_exp2f((m[qb] - m_safe) * LOG2E);
      float sum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][qb][i], LOG2E, -m_log2));
          s[kb][qb][i] = p;
          sum += p;
        }
      sum = rows_sum(sum);
      l[qb] = l[qb] * alpha + sum;
      // the sums so far are rescaled only if the maximum of some query of the wave moved
      if (__builtin_amdgcn_ballot_w64(m_new != m[qb]) != 0) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[db][qb][i] *= alpha;
      }
      m[qb] = m_new;
    }
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      bf16x8 pb[2];
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int j = 0; j < 8; ++j) pb[qb][j] = (bf16_t)s[2 * t + (j >> 2)][qb][j & 3];
      // the values of 16 head-size elements are read while the products of the 16 before them run
      auto read_values = [&](int db) {
        if (FAST) return *(const bf16x8*)(vd + (16 * db + r) * VSTR + 32 * t + 8 * g);
        const bf16_t* vrow = vd + (16 * db + r) * VSTR + 32 * t + 4 * g;
        const bf16x4 lo4 = *(const bf16x4*)(vrow);
        const bf16x4 hi4 = *(const bf16x4*)(vrow + 16);
        bf16x8 vf;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          vf[i] = lo4[i];
          vf[4 + i] = hi4[i];
        }
        return vf;
      };
      bf16x8 vf[3];
      vf[0] = read_values(0);
      vf[1] = read_values(min(1, NDB - 1));
#pragma unroll
      for (int db = 0; db < NDB; ++db) {
        if (db + 2 < NDB) vf[(db + 2) % 3] = read_values(db + 2);
        __builtin_amdgcn_sched_barrier(0);    // the reads stay ahead of the products, as written
        if (db < ndb) {
          o[db][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db % 3], pb[0], o[db][0], 0, 0, 0);
          o[db][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db % 3], pb[1], o[db][1], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  if (GROUPS == 2) {
    // the second set leaves what it has in LDS (every lane its own words, lanes side by side), the first adds it
    float* po = (float*)smem;                                   // [4 waves][NDB][2][4][64]
    float* pml = po + 4 * NDB * 2 * 4 * 64;                     // [4 waves][2][2][64]
    __syncthreads();                                            // the staged tiles are done with
    if (grp == 1 && wave_on) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) po[(((wave * NDB + db) * 2 + qb) * 4 + i) * 64 + lane] = o[db][qb][i];
        pml[((wave * 2 + qb) * 2 + 0) * 64 + lane] = m[qb];
        pml[((wave * 2 + qb) * 2 + 1) * 64 + lane] = l[qb];
      }
    }
    __syncthreads();
    if (grp == 1) return;
    if (wave_on) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const float m1 = pml[((wave * 2 + qb) * 2 + 0) * 64 + lane];
        const float l1 = pml[((wave * 2 + qb) * 2 + 1) * 64 + lane];
        const float m_all = fmaxf(m[qb], m1);
        const float m_safe = m_all == -INFINITY ? 0.f : m_all;
        const float a0 = __builtin_amdgcn_exp2f((m[qb] - m_safe) * LOG2E);
        const float a1 = __builtin_amdgcn_exp2f((m1 - m_safe) * LOG2E);
        l[qb] = l[qb] * a0 + l1 * a1;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            o[db][qb][i] = o[db][qb][i] * a0 + po[(((wave * NDB + db) * 2 + qb) * 4 + i) * 64 + lane] * a1;
      }
    }
  }
  if (!wave_on) return;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    if (qi >= qlen) continue;
    const float inv = 1.f / l[qb];
    bf16_t* orow = out + (size_t)(t0 + qi) * nq + h * head_size;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      if (db >= ndb) continue;
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[db][qb][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v4;
    }
  }
}

template <int NDB, bool FAST, int GROUPS>
static int launch_prefill_lds(dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* k_pages,
                              const bf16_t* v_pages, const int* run_start, const int* cached_lens, const int* table,
                              int table_width, int page_shift, int num_pages, const int* tile_run,
                              const int* tile_q0, bf16_t* out, int num_heads, int num_kv, int head_size,
                              int window, int page_pad) {
  constexpr int DMAX = 16 * NDB;
  using Layout = PrefillTileLayout<NDB, FAST>;
  constexpr size_t bytes = GROUPS * 2 * (size_t)(Layout::KBUF + Layout::VBUF) * sizeof(bf16_t);
  static_assert(bytes <= 160 * 1024, "the staging buffers must fit the 160 KB of LDS");
  static_assert(GROUPS == 1 || bytes >= (4 * NDB * 2 * 4 * 64 + 4 * 2 * 2 * 64) * sizeof(float),
                "the partial results of the second set of waves must fit the staging buffers");
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)attention_prefill_lds_kernel<NDB, FAST, GROUPS>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) {
      tnx_set_error("attention_prefill: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  attention_prefill_lds_kernel<NDB, FAST, GROUPS><<<grid, 256 * GROUPS, bytes, stream>>>(q, k_pages, v_pages, run_start, cached_lens, table,
                                                                 table_width, page_shift, num_pages, tile_run,
                                                                 tile_q0, out, num_heads, num_kv, head_size, window,
                                                                 page_pad);
  return 0;
}


// The staged computation once more for the FAST case (see above) without a window, arranged so that the
// matrix unit and the vector unit work at the same time within a wave: the scores of tile i + 1 are multiplied
// while the softmax of tile i is computed (the two are independent, and a wave issues vector instructions
// while its matrix instruction runs; measured, a matrix instruction costs a wave the time of two vector
// instructions to issue and the unit that of four to run, so two vector instructions to a product keep both
// busy). The keys therefore run one tile ahead of the values in LDS. What keeps the vector unit's share small:
//  - the sums so far are rescaled only when some query's maximum has moved far (see `softmax_maximum`);
//  - the sum of a query's probabilities comes from the matrix unit (a block of ones beside the values);
//  - tiles go from the pages to LDS without passing through registers (`load_to_lds`: a wave instruction
//    fills 1 KB of LDS in lane order, so the layout's exchange of chunks is applied to the global addresses),
//    one load at a time between the products: issued together they held every wave of the block at the
//    memory pipeline's queue.
// Rows lie unpadded in LDS, chunk c of key row k at c ^ (k's index among the 16 rows read together) and chunk
// c of value row d at c ^ (d % 8), which the fragment reads take without bank conflicts. What a load brings
// of keys beyond the request is zeroed in LDS by the lane that asked for it (values only: their probabilities
// are zero, and zero times a stale NaN is not). Measured at 32 heads of size 128 and a prompt of 2,048: 54.6 us
// against 64.3 for the kernel above (per 64-key step of a block: 0.97 us is what the 136 matrix instructions of
// its two waves a SIMD take, 1.8 us is what the step takes; LDS reads and the tile loads account for most of
// the rest).
template <int NDB, int GROUPS>
__global__ void __launch_bounds__(256 * GROUPS, GROUPS == 1 ? 2 : 1)
attention_prefill_pipelined_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                                   const bf16_t* __restrict__ v_pages, const int* __restrict__ run_start,
                                   const int* __restrict__ cached_lens, const int* __restrict__ table,
                                   int table_width, int page_shift, int num_pages,
                                   const int* __restrict__ tile_run, const int* __restrict__ tile_q0,
                                   bf16_t* __restrict__ out, int num_heads, int num_kv, int page_pad) {
  static_assert(NDB == 4 || NDB == 8, "head sizes 64 and 128");
  constexpr int NKS = NDB / 2, DH = 16 * NDB, CPR = 2 * NDB;   // CPR: 16-byte chunks of a key row
  constexpr int TILE_BYTES = 64 * DH * 2;                       // 64 keys, and as many values
  constexpr int NLD = TILE_BYTES / 4096;                        // 1 KB loads of a wave for a tile
  extern __shared__ __attribute__((aligned(16))) char pipelined_smem[];
  const int grp = GROUPS == 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 8);
  char* kbuf = pipelined_smem + grp * 4 * TILE_BYTES;           // [2][TILE_BYTES]
  char* vbuf = kbuf + 2 * TILE_BYTES;                           // [2][TILE_BYTES]
  const unsigned kbuf_lds = (unsigned)(size_t)(__attribute__((address_space(3))) char*)kbuf;
  const unsigned vbuf_lds = kbuf_lds + 2 * TILE_BYTES;
  const int tid = threadIdx.x & 255, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int tile = blockIdx.x / num_heads, h = blockIdx.x % num_heads;
  const int run = tile_run[tile];
  const int kvh = h / (num_heads / num_kv);
  const int t0 = run_start[run], qlen = run_start[run + 1] - t0, cached = cached_lens[run];
  const int q0 = tile_q0[tile];
  const int qw0 = q0 + 32 * wave;
  const bool wave_on = qw0 < qlen;
  const int nq = num_heads * DH;
  const int* tab = table + (size_t)run * table_width;
  const int total = cached + qlen;
  const int page_size = 1 << page_shift, pmask = page_size - 1;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
  const size_t head_stride = (size_t)page_size * DH;
  const size_t page_stride = (size_t)num_kv * head_stride + page_pad;

  bf16x8 qf[2][NKS];
  int qpos[2];
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    qpos[qb] = cached + qi;
#pragma unroll
    for (int s = 0; s < NKS; ++s)
      qf[qb][s] = qi < qlen ? *(const bf16x8*)(q + (size_t)(t0 + qi) * nq + h * DH + 32 * s + 8 * g) : zero8;
  }
  const int blk_last = cached + min(q0 + PREFILL_Q_TILE - 1, qlen - 1);
  const int last_q = cached + min(qw0 + 31, qlen - 1);
  const int first_q = cached + qw0;

  // What each lane asks for: place p = (4 j + wave) * 64 + lane of a tile, in chunks. The offsets of the NLD
  // loads differ by a constant and, for the keys, by which two bits the chunk is exchanged with; they are made
  // from one register each when they are needed (and hidden from the compiler, which would keep them all).
  //   keys: row (4 j + wave) (64 / CPR) + lane / CPR, stored chunk lane % CPR -> chunk (lane % CPR) ^ swizzle(row)
  //   values: row 32 j + 8 wave + lane / 8, stored chunk lane % 8 -> chunk (lane % 8) ^ (row % 8)
  unsigned kbase, vbase;      // bytes from the tile's first key within its page, for j = 0 (keys: bits 2-3 of the
                              // exchange left out)
  {
    const int krow = wave * (64 / CPR) + lane / CPR;
    kbase = (krow * DH + ((lane % CPR) ^ (krow & 3)) * 8) * 2;
    const int d = 8 * wave + (lane >> 3);
    vbase = (d * page_size + ((lane & 7) ^ (d & 7)) * 8) * 2;
  }
  const int vkey = ((lane & 7) ^ ((lane >> 3) & 7)) * 8;     // the first key of the lane's value chunks
  auto key_offset = [&](int j) -> unsigned {
    // bits 3-4 of the row (head size 128: rows 16 j + 4 wave + ..) or bit 3 (head size 64: rows 32 j + 8 wave
    // + ..) go to bits 2-3 of the chunk number, bits 6-7 of the byte offset
    const int high = NDB == 8 ? ((2 * j + (wave >> 1)) & 3) : (wave & 1);
    unsigned base = kbase;
    asm volatile("" : "+v"(base));
    return (base ^ (high << 6)) + j * 4096;
  };
  auto value_offset = [&](int j) -> unsigned {
    unsigned base = vbase;
    asm volatile("" : "+v"(base));
    return base + j * 32 * page_size * 2;
  };
  auto lookup = [&](int tile0) { return tab[min(tile0, total - 1) >> page_shift]; };
  auto key_source = [&](int tile0, int page) -> const bf16_t* {
    const int pg = min(max(page, 0), num_pages - 1);
    return k_pages + (size_t)pg * page_stride + (size_t)kvh * head_stride + (size_t)(tile0 & pmask) * DH;
  };
  auto value_source = [&](int tile0, int page) -> const bf16_t* {
    const int pg = min(max(page, 0), num_pages - 1);
    return v_pages + (size_t)pg * page_stride + (size_t)kvh * head_stride + (tile0 & pmask);
  };
  auto issue_key_load = [&](int j, int buf, const bf16_t* src) {
    load_to_lds(src, key_offset(j), kbuf_lds + buf * TILE_BYTES + wave * 1024 + j * 4096);
  };
  auto issue_value_load = [&](int j, int buf, const bf16_t* src) {
    load_to_lds(src, value_offset(j), vbuf_lds + buf * TILE_BYTES + wave * 1024 + j * 4096);
  };
  auto issue_keys = [&](int buf, int tile0, int page) {
    const bf16_t* src = key_source(tile0, page);
#pragma unroll
    for (int j = 0; j < NLD; ++j) issue_key_load(j, buf, src);
  };
  auto issue_values = [&](int buf, int tile0, int page) {
    const bf16_t* src = value_source(tile0, page);
#pragma unroll
    for (int j = 0; j < NLD; ++j) issue_value_load(j, buf, src);
  };
  // after the lane's own loads have landed: zero what must not be seen
  auto clear_values = [&](int buf, int tile0) {
    if (tile0 + 64 <= total) return;
#pragma unroll
    for (int j = 0; j < NLD; ++j) {
      const int k0 = tile0 + vkey;
      if (k0 + 8 > total) {
        bf16x8* at = (bf16x8*)(vbuf + buf * TILE_BYTES + ((4 * j + wave) * 64 + lane) * 16);
        bf16x8 v = *at;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (k0 + e >= total) v[e] = 0;
        *at = v;
      }
    }
  };

  // the block's key tiles in equal shares for its sets of waves, as in the kernel above
  const int share = (blk_last / 64 + GROUPS) / GROUPS;
  const int tile_begin = grp * share * 64;
  const int tile_last = min(blk_last, tile_begin + share * 64 - 1);
  const int n_live = tile_last >= tile_begin ? (tile_last - tile_begin) / 64 + 1 : 0;     // tiles of this set
  // the tiles of this wave: those that some query of it sees
  int it_b = last_q >= tile_begin ? min(n_live - 1, (last_q - tile_begin) >> 6) : -1;
  if (!wave_on) it_b = -1;
  it_b = __builtin_amdgcn_readfirstlane(it_b);

  float m[2] = {-INFINITY, -INFINITY}, l[2] = {0.f, 0.f};
  f32x4 o[NDB][2];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) o[db][qb] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // fragment reads: byte offsets of this lane, to which the block of rows adds a constant
  const int swr = NDB == 8 ? r : (r & 7);
  const int krow_off = (8 * (r >> 2) + (r & 3)) * CPR * 16;
  int kchunk[NKS], vchunk[2];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) kchunk[ks] = krow_off + (((4 * ks + g) ^ swr) & (CPR - 1)) * 16;
#pragma unroll
  for (int t = 0; t < 2; ++t) vchunk[t] = r * 128 + ((4 * t + g) ^ (r & 7)) * 16;

  // S^T = K Q^T of one tile: row r of key block kb is key 32 (kb / 2) + 8 (r / 4) + 4 (kb % 2) + r % 4
  auto read_keys = [&](const char* kd, int kb, bf16x8* dst) {
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks)
      dst[ks] = *(const bf16x8*)(kd + (32 * (kb >> 1) + 4 * (kb & 1)) * CPR * 16 + kchunk[ks]);
  };
  auto multiply_keys = [&](const bf16x8* kf, f32x4 (&s)[2]) {
    f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf[0][ks], a0, 0, 0, 0);
      a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[ks], qf[1][ks], a1, 0, 0, 0);
    }
    s[0] = a0;
    s[1] = a1;
  };
  auto scores = [&](int buf, f32x4 (&s)[4][2]) {
    const char* kd = kbuf + buf * TILE_BYTES;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      bf16x8 kf[NKS];
      read_keys(kd, kb, kf);
      multiply_keys(kf, s[kb]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto mask = [&](int tile0, f32x4 (&s)[4][2]) {
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = tile0 + 32 * (kb >> 1) + 8 * g + 4 * (kb & 1) + i;
          if (key > qpos[qb]) s[kb][qb][i] = -INFINITY;
        }
  };
  // The softmax of a tile in parts, so that each can be set beside a quarter of the next tile's score
  // products. The scores become probabilities in place.
  // The reference maximum m of a query (probabilities are e^(score - m)) follows the true maximum lazily: it
  // moves, for all queries of the wave at once, when some query meets a score more than RESCALE_AT powers of
  // two above its own m. Between such moves no sum needs rescaling and a probability is at most 2^RESCALE_AT,
  // which changes nothing in the quotient of the sums. `moved` tells the caller to multiply the sums so far
  // by `alpha`.
  constexpr float RESCALE_AT = 8.f;
  float m_log2[2] = {0.f, 0.f};
  auto softmax_maximum = [&](const f32x4 (&s)[4][2], float (&alpha)[2]) -> bool {
    float mx[2];
    bool jump = false;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      float x = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 4; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i) x = fmaxf(x, s[kb][qb][i]);
      mx[qb] = rows_max(x);
      jump = jump || (mx[qb] - m[qb]) * LOG2E > RESCALE_AT;     // false where both are -inf
    }
    const bool moved = __builtin_amdgcn_ballot_w64(jump) != 0;
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float m_new = moved ? fmaxf(m[qb], mx[qb]) : m[qb];
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;
      // e^(x - m) as 2^(x log2 e - m log2 e): one multiply-add and the hardware's 2^x
      m_log2[qb] = m_safe * LOG2E;
      alpha[qb] = __builtin_amdgcn_exp2f((m[qb] - m_safe) * LOG2E);
      m[qb] = m_new;
    }
    return moved;
  };
  // the probabilities of four keys (one block of four registers)
  auto exponentials = [&](f32x4 (&s)[4][2], int kb, int qb) {
#pragma unroll
    for (int i = 0; i < 4; ++i) s[kb][qb][i] = __builtin_amdgcn_exp2f(fmaf(s[kb][qb][i], LOG2E, -m_log2[qb]));
  };
  // the probabilities of keys 32 t .. 32 t + 31 of the tile as the B operands of the value products
  auto rounded = [&](const f32x4 (&s)[4][2], int t, bf16x8 (&pb)[2]) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb)
#pragma unroll
      for (int j = 0; j < 8; ++j) pb[qb][j] = (bf16_t)s[2 * t + (j >> 2)][qb][j & 3];
  };
  // The sums of the probabilities come from the matrix unit as well: a block of ones in the place of the
  // values gives every lane the sum over the keys for its query, of the probabilities as they are multiplied
  // (rounded), with no addition or exchange between lanes on the vector unit.
  f32x4 lsum[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
  bf16x8 ones;
#pragma unroll
  for (int j = 0; j < 8; ++j) ones[j] = (bf16_t)1.f;
  auto rescale = [&](const float (&alpha)[2]) {
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[db][qb][i] *= alpha[qb];
#pragma unroll
      for (int i = 0; i < 4; ++i) lsum[qb][i] *= alpha[qb];
    }
  };
  // O^T += V^T P^T, and the second half of the softmax. The probabilities of the tile's first 32 keys are
  // there; those of the other 32 are made between the products of the first, and `next`, if asked, takes the
  // place of the probabilities between the products of the second half: some two vector instructions to a
  // matrix instruction everywhere, as beside the score products, so that neither unit waits for the other
  // for long. The values of 16 head-size elements are read two steps before their products.
  auto weighted_values = [&](int buf, f32x4 (&s)[4][2], const f32x4 (&next)[4][2], bool take_next) {
    const char* vd = vbuf + buf * TILE_BYTES;
    auto read_values = [&](int j) { return *(const bf16x8*)(vd + 16 * (j % NDB) * 128 + vchunk[j / NDB]); };
    constexpr int AHEAD = 2;
    bf16x8 vf[AHEAD + 1], pb[2];
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) vf[j] = read_values(j);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 2 * NDB; ++j) {
      const int db = j % NDB;
      if (j + AHEAD < 2 * NDB) vf[(j + AHEAD) % (AHEAD + 1)] = read_values(j + AHEAD);
      if (db == 0) {
        rounded(s, j / NDB, pb);
        lsum[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[0], lsum[0], 0, 0, 0);
        lsum[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[1], lsum[1], 0, 0, 0);
      }
      o[db][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j % (AHEAD + 1)], pb[0], o[db][0], 0, 0, 0);
      o[db][1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[j % (AHEAD + 1)], pb[1], o[db][1], 0, 0, 0);
      // the vector work of this step: 4 * NDB / ... pieces of four registers over the NDB steps of a half
      constexpr int PER = 4 / (NDB / 2 > 4 ? 4 : NDB / 2);     // blocks of four registers a step: 1 (NDB 8), 2 (NDB 4)
#pragma unroll
      for (int c = PER * db; c < PER * db + PER; ++c) {
        if (c >= 4) break;
        if (j < NDB) {
          exponentials(s, 2 + (c >> 1), c & 1);
        } else if (take_next) {
          s[c >> 1][c & 1] = next[c >> 1][c & 1];
          s[2 + (c >> 1)][c & 1] = next[2 + (c >> 1)][c & 1];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto softmax_and_values = [&](int buf, f32x4 (&s)[4][2], const f32x4 (&next)[4][2], bool take_next) {
    float alpha[2];
    const bool moved = softmax_maximum(s, alpha);
#pragma unroll
    for (int c = 0; c < 4; ++c) exponentials(s, c >> 1, c & 1);
    __builtin_amdgcn_sched_barrier(0);
    if (moved) rescale(alpha);
    weighted_values(buf, s, next, take_next);
  };
  // The scores of the next tile beside the softmax of the current one: after each product a few vector
  // instructions of the softmax part that stands beside this quarter of the products.
  // The loads of the step (the values of the next tile, the keys of the one after it) are issued one at a
  // time between the quarters, not together at the step's start, where every wave of the block would wait
  // for room in the queue of the memory pipeline with the matrix unit idle.
  auto scores_beside_softmax = [&](int buf, f32x4 (&next)[4][2], f32x4 (&cur)[4][2], float (&alpha)[2],
                                   int load_buf_v, const bf16_t* vsrc, int load_buf_k, const bf16_t* ksrc) -> bool {
    const char* kd = kbuf + buf * TILE_BYTES;
    // The fragments of half a block of keys (NKS / 2 steps of 32 over the head size) at a time, three such sets
    // in turn: a set is asked for two half-blocks (eight products) before it is used; the registers do not
    // hold more.
    constexpr int HK = NKS / 2;
    bf16x8 kf[3][HK];
    bool moved = false;
    auto read_half = [&](int slot, bf16x8* dst) {      // half-block `slot` of the tile: key block slot / 2
      const int kb = slot >> 1, half = slot & 1;
#pragma unroll
      for (int i = 0; i < HK; ++i)
        dst[i] = *(const bf16x8*)(kd + (32 * (kb >> 1) + 4 * (kb & 1)) * CPR * 16 + kchunk[half * HK + i]);
    };
    read_half(0, kf[0]);
    read_half(1, kf[1]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      f32x4 a0 = {0.f, 0.f, 0.f, 0.f}, a1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        const int slot = 2 * kb + half;
        if (slot + 2 < 8) read_half(slot + 2, kf[(slot + 2) % 3]);
#pragma unroll
        for (int i = 0; i < HK; ++i) {
          const int ks = half * HK + i;
          a0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[slot % 3][i], qf[0][ks], a0, 0, 0, 0);
          a1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[slot % 3][i], qf[1][ks], a1, 0, 0, 0);
        }
        // the maximum beside the first two blocks of products, the first half's probabilities beside the rest
        if (kb == 0 && half == 0) moved = softmax_maximum(cur, alpha);
        if (kb >= 2) exponentials(cur, kb - 2, half);
        if (slot + 2 < 8) __builtin_amdgcn_sched_group_barrier(0x100, HK, 0);
#pragma unroll
        for (int i = 0; i < NKS; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          if (kb < 2) __builtin_amdgcn_sched_group_barrier(0x002, 12 / NKS, 0);
          else __builtin_amdgcn_sched_group_barrier(0x002, 8 / NKS, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        {
          constexpr int PER = NLD / 4 > 0 ? NLD / 4 : 1;       // loads a half-quarter: 2 NLD loads over 8 of them
          if (NLD == 4 || slot % 2 == 0) {
            const int j = NLD == 4 ? slot : slot / 2;          // 0 .. 2 NLD - 1
            if (j < NLD) issue_value_load(j, load_buf_v, vsrc);
            else issue_key_load(j - NLD, load_buf_k, ksrc);
          }
          (void)PER;
        }
      }
      next[kb][0] = a0;
      next[kb][1] = a1;
    }
    return moved;
  };

  f32x4 s_even[4][2], s_odd[4][2];
  int page1, page2;       // pages of the tiles one and two after the current one
  {
    const int page0 = lookup(tile_begin);
    page1 = lookup(tile_begin + 64);
    page2 = lookup(tile_begin + 128);
    if (n_live > 0) {
      issue_keys(0, tile_begin, page0);
      issue_values(0, tile_begin, page0);
    }
    if (n_live > 1) issue_keys(1, tile_begin + 64, page1);
    wait_for_loads();                                 // this lane's loads are in LDS
    if (n_live > 0) clear_values(0, tile_begin);
    __syncthreads();
    if (it_b >= 0) scores(0, s_even);
  }
  // Step `it`: LDS holds the keys of tile it + 1 and the values of tile it; `cur` holds the scores of tile it.
  // Every step passes one barrier, whichever loop below it belongs to: the waves of a block take different
  // numbers of steps in the first loop and the same number in both together.
  auto begin_step = [&](int it, bool with_loads) {
    __syncthreads();      // every wave is done with tile it - 1; tile it's values and tile it + 1's keys are there
    const int tile0 = tile_begin + 64 * it;
    if (with_loads) {
      if (it + 1 < n_live) issue_values((it + 1) & 1, tile0 + 64, page1);
      if (it + 2 < n_live) issue_keys(it & 1, tile0 + 128, page2);
    }
  };
  auto end_step = [&](int it) {
    // the page of the tile after the next two is looked up here, where the wave waits anyway
    page1 = page2;
    page2 = lookup(tile_begin + 64 * it + 192);
    wait_for_loads();
    if (it + 1 < n_live) clear_values((it + 1) & 1, tile_begin + 64 * it + 64);
  };
  // the tiles that every query of the wave sees whole and that another tile of the wave follows
  const int n_full = first_q + 1 > tile_begin ? (first_q + 1 - tile_begin) >> 6 : 0;
  const int n_hot = __builtin_amdgcn_readfirstlane(max(0, min(it_b, n_full)));
  f32x4 (&cur)[4][2] = s_even, (&next)[4][2] = s_odd;
  int it = 0;
  for (; it < n_hot; ++it) {
    begin_step(it, false);
    float alpha[2];
    // a tile beyond the set's last is not read by anyone: its loads bring the last tile once more
    const int tile_v = tile_begin + 64 * min(it + 1, n_live - 1), tile_k = tile_begin + 64 * min(it + 2, n_live - 1);
    const bool moved = scores_beside_softmax((it + 1) & 1, next, cur, alpha, (it + 1) & 1, value_source(tile_v, page1),
                                             it & 1, key_source(tile_k, it + 2 < n_live ? page2 : page1));
    if (moved) rescale(alpha);
    weighted_values(it & 1, cur, next, true);
    end_step(it);
  }
  // the wave's last tiles, which the positions mask, and the steps in which it only loads and waits
  for (; it < share; ++it) {
    begin_step(it, true);
    const int tile0 = tile_begin + 64 * it;
    const bool has_cur = it <= it_b, has_next = it + 1 <= it_b;
    if (has_next) scores((it + 1) & 1, next);
    if (has_cur) {
      if (tile0 + 63 > first_q) mask(tile0, cur);
      softmax_and_values(it & 1, cur, next, has_next);
    }
    end_step(it);
  }

  l[0] = lsum[0][0];
  l[1] = lsum[1][0];
  if (GROUPS == 2) {
    // the second set leaves what it has in LDS (every lane its own words, lanes side by side), the first adds it
    float* po = (float*)pipelined_smem;                         // [4 waves][NDB][2][4][64]
    float* pml = po + 4 * NDB * 2 * 4 * 64;                     // [4 waves][2][2][64]
    __syncthreads();                                            // the staged tiles are done with
    if (grp == 1 && wave_on) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i) po[(((wave * NDB + db) * 2 + qb) * 4 + i) * 64 + lane] = o[db][qb][i];
        pml[((wave * 2 + qb) * 2 + 0) * 64 + lane] = m[qb];
        pml[((wave * 2 + qb) * 2 + 1) * 64 + lane] = l[qb];
      }
    }
    __syncthreads();
    if (grp == 1) return;
    if (wave_on) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        const float m1 = pml[((wave * 2 + qb) * 2 + 0) * 64 + lane];
        const float l1 = pml[((wave * 2 + qb) * 2 + 1) * 64 + lane];
        const float m_all = fmaxf(m[qb], m1);
        const float m_safe = m_all == -INFINITY ? 0.f : m_all;
        const float a0 = __builtin_amdgcn_exp2f((m[qb] - m_safe) * LOG2E);
        const float a1 = __builtin_amdgcn_exp2f((m1 - m_safe) * LOG2E);
        l[qb] = l[qb] * a0 + l1 * a1;
#pragma unroll
        for (int db = 0; db < NDB; ++db)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            o[db][qb][i] = o[db][qb][i] * a0 + po[(((wave * NDB + db) * 2 + qb) * 4 + i) * 64 + lane] * a1;
      }
    }
  }
  if (!wave_on) return;
#pragma unroll
  for (int qb = 0; qb < 2; ++qb) {
    const int qi = qw0 + 16 * qb + r;
    if (qi >= qlen) continue;
    const float inv = 1.f / l[qb];
    bf16_t* orow = out + (size_t)(t0 + qi) * nq + h * DH;
#pragma unroll
    for (int db = 0; db < NDB; ++db) {
      bf16x4 v4;
#pragma unroll
      for (int i = 0; i < 4; ++i) v4[i] = (bf16_t)(o[db][qb][i] * inv);
      *(bf16x4*)(orow + 16 * db + 4 * g) = v4;
    }
  }
}

template <int NDB, int GROUPS>
static int launch_prefill_pipelined(dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* k_pages,
                                    const bf16_t* v_pages, const int* run_start, const int* cached_lens,
                                    const int* table, int table_width, int page_shift, int num_pages,
                                    const int* tile_run, const int* tile_q0, bf16_t* out, int num_heads, int num_kv,
                                    int head_size, int window, int page_pad) {
  constexpr size_t bytes = GROUPS * 4 * (size_t)(64 * 16 * NDB * 2);
  static_assert(bytes <= 160 * 1024, "the staging buffers must fit the 160 KB of LDS");
  static_assert(GROUPS == 1 || bytes >= (4 * NDB * 2 * 4 * 64 + 4 * 2 * 2 * 64) * sizeof(float),
                "the partial results of the second set of waves must fit the staging buffers");
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)attention_prefill_pipelined_kernel<NDB, GROUPS>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) {
      tnx_set_error("attention_prefill: cannot reserve %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  (void)head_size;
  (void)window;
  attention_prefill_pipelined_kernel<NDB, GROUPS><<<grid, 256 * GROUPS, bytes, stream>>>(
      q, k_pages, v_pages, run_start, cached_lens, table, table_width, page_shift, num_pages, tile_run, tile_q0, out,
      num_heads, num_kv, page_pad);
  return 0;
}

extern "C" int tnx_attention_prefill(const void* q, const void* k_pages, const void* v_pages, const int* run_start,
                                     const int* cached_lens, const int* table, int table_width, int page_size,
                                     int num_pages, const int* tile_run, const int* tile_q0, int num_tiles, void* out,
                                     int num_heads, int num_kv, int head_size, int window, int direct,
                                     int query_tile, int page_pad, hipStream_t stream) {
  TNX_REQUIRE(page_pad >= 0 && page_pad % 8 == 0, "attention_prefill: bad distance between pages");
  TNX_REQUIRE(query_tile == PREFILL_Q_TILE,
              "attention_prefill: the tiles hold %d queries each, the kernels take %d: a tile's later queries would "
              "be skipped", query_tile, PREFILL_Q_TILE);
  TNX_REQUIRE(num_heads > 0 && num_kv > 0 && num_heads % num_kv == 0, "attention_prefill: bad head counts");
  TNX_REQUIRE(head_size % 16 == 0 && head_size >= 16 && head_size <= 256,
              "attention_prefill: head size %d is not a multiple of 16 in [16, 256]", head_size);
  TNX_REQUIRE(page_size % 16 == 0 && page_size > 0, "attention_prefill: page size %d is not a multiple of 16",
              page_size);
  if (num_tiles <= 0) return 0;
  TNX_REQUIRE((long long)num_tiles * num_heads < (1ll << 31), "attention_prefill: too many tiles");
  // Blocks are numbered with the head running fastest: the tiles come ordered by falling work, so the blocks
  // that run longest start first and the short ones fill in behind them.
  dim3 grid((unsigned)num_tiles * num_heads);
  if ((page_size & (page_size - 1)) == 0 && direct != 1) {
    // `direct` 0 or 3: two sets of waves a block; 2: one set; 6 and 7: the same with the staged kernel where the
    // pipelined one would run (head sizes 64 and 128, pages of 64 keys or more, no window)
    const int sets = (direct == 2 || direct == 7) ? 1 : 2;
    const bool pipelined = direct != 6 && direct != 7 && window <= 0 && page_size >= 64 &&
                           (head_size == 64 || head_size == 128);
    int page_shift = 0;
    while ((1 << page_shift) < page_size) ++page_shift;
    int rc = -1;
#define LDS_ARGS                                                                                                 \
  grid, stream, (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, run_start, cached_lens, table, \
      table_width, page_shift, num_pages, tile_run, tile_q0, (bf16_t*)out, num_heads, num_kv, head_size, window, \
      page_pad
#define LAUNCH_LDS(NDB)                                                                                          \
  {                                                                                                              \
    constexpr int G = NDB <= 8 ? 2 : 1;     /* two sets of waves where LDS holds the buffers of both */          \
    const bool fast = NDB <= 8 && page_size >= 64 && head_size == 16 * NDB;                                      \
    if (sets == 1)                                                                                               \
      rc = fast ? launch_prefill_lds<NDB, true, 1>(LDS_ARGS) : launch_prefill_lds<NDB, false, 1>(LDS_ARGS);      \
    else                                                                                                         \
      rc = fast ? launch_prefill_lds<NDB, true, G>(LDS_ARGS) : launch_prefill_lds<NDB, false, G>(LDS_ARGS);      \
  }
    if (pipelined) {
      if (head_size == 64)
        rc = sets == 2 ? launch_prefill_pipelined<4, 2>(LDS_ARGS) : launch_prefill_pipelined<4, 1>(LDS_ARGS);
      else
        rc = sets == 2 ? launch_prefill_pipelined<8, 2>(LDS_ARGS) : launch_prefill_pipelined<8, 1>(LDS_ARGS);
    } else if (head_size <= 64) {
      LAUNCH_LDS(4);
    } else if (head_size <= 128) {
      LAUNCH_LDS(8);
    } else {
      LAUNCH_LDS(16);
    }
#undef LAUNCH_LDS
#undef LDS_ARGS
    if (rc) return rc;
    TNX_CHECK_LAUNCH("attention_prefill_lds");
    return 0;
  }
#define LAUNCH_PREFILL(NDB)                                                                                        \
  attention_prefill_kernel<NDB><<<grid, 256, 0, stream>>>(                                                         \
      (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, run_start, cached_lens, table, table_width, \
      page_size, num_pages, tile_run, tile_q0, (bf16_t*)out, num_heads, num_kv, head_size, window, page_pad)
  if (head_size <= 64)
    LAUNCH_PREFILL(4);
  else if (head_size <= 128)
    LAUNCH_PREFILL(8);
  else
    LAUNCH_PREFILL(16);
#undef LAUNCH_PREFILL
  TNX_CHECK_LAUNCH("attention_prefill");
  return 0;
}

// ------------------------------------------------------------------------------------------ bfloat16, decoding

// One query per request over its pages, on the matrix unit. The keys of a request are split over `num_splits`
// blocks; a block's NW waves (four or eight) take 64-key tiles in turn. Partial results (maximum, sum, weighted
// values, all float32) of waves meet in LDS and those of splits in a workspace that a second kernel merges. The
// page size is a power of two here.
// The one query of a (request, head) is the B operand of S^T = K q in all 16 of
// its columns (the products cost nothing more, and with them the scores come out in the accumulator layout
// that is at once the B operand of O^T += V^T P^T, as in the prompt kernel); row r of key block kb of a 64-key
// tile is key 32 (kb / 2) + 8 (r / 4) + 4 (kb % 2) + r % 4, so that the probabilities a lane holds are those of
// 8 consecutive keys and the values are read 16 bytes a lane as they lie. A tile costs 32 matrix
// instructions and some 150 others, where dot products on the vector unit took a thousand: the step of a few
// requests is the time its instructions take to arrive from memory, and the step of many requests was close
// to the vector unit's limit (measured at head size 128, context 2,048: 18.1 -> 15.6 us for one request,
// 52.4 -> 49.7 for 8, 381 -> 369 for 64).
// The pages of a tile are looked up with scalar loads (a tile's keys lie in at most four pages, the same for
// every lane), which do not queue behind the tile data; the next tile's keys are asked for as soon as this
// tile's scores are made, its values as soon as this tile's are used (NDB <= 8; beyond that the registers
// hold one of the two at a time).
// PACK: for query heads that share their keys and values (fewer kv heads than heads). A block then takes one
// kv head of one request, and the 16 columns hold up to 16 (8 at the largest head size) different query heads
// of its group, so the keys and values are read once for all of them and not once a head; the maxima, sums and
// results are a column's own throughout (a column is the lanes with the same lane % 16).
template <int NDB, int NW, bool PACK>
__global__ void __launch_bounds__(64 * NW, (NDB <= 8 ? 8 / NW : 1))
attention_decode_mfma_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                             const bf16_t* __restrict__ v_pages, const int* __restrict__ run_start,
                             const int* __restrict__ cached_lens, const int* __restrict__ table, int table_width,
                             int page_shift, int num_pages, const int* __restrict__ decode_runs,
                             bf16_t* __restrict__ out, float* __restrict__ part_o, float* __restrict__ part_ml,
                             int num_heads, int num_kv, int window, int num_splits,
                             const int* __restrict__ longest_ptr, int head_size, int page_pad) {
  constexpr int NKS = (NDB + 1) / 2;  // steps of 32 over the head size
  constexpr int DH = 16 * NDB;        // the registers are laid out for this head size; `head_size` <= DH
  constexpr bool PIPE = NDB <= 8;     // keys and values of different tiles are in registers together
  constexpr int COLS = !PACK ? 1 : NDB <= 8 ? 16 : 8;     // query heads a block takes (what LDS holds of results)
  __shared__ float sm_o[NW][COLS][DH];
  __shared__ float sm_m[NW][COLS], sm_l[NW][COLS];
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15, g = lane >> 4;
  const int split = blockIdx.x, dz = blockIdx.z;
  const int group = num_heads / num_kv;
  // h: the query head of this lane's column; kvh: the kv head of the block
  const int chunks = PACK ? (group + COLS - 1) / COLS : 1;
  const int kvh = PACK ? blockIdx.y / chunks : blockIdx.y / group;
  const int col0 = PACK ? (blockIdx.y % chunks) * COLS : 0;          // the group's first head in this block
  const bool col_on = !PACK || (r < COLS && col0 + r < group);
  const int h = PACK ? kvh * group + min(col0 + r, group - 1) : blockIdx.y;
  const int run = decode_runs[dz];
  const int longest_given = longest_ptr[0];
  const int t = run_start[run];
  const int pos = cached_lens[run];   // the query's own position; its key is stored already
  const int* tab = table + (size_t)run * table_width;
  const int nq = num_heads * head_size;
  const int page_size = 1 << page_shift, pmask = page_size - 1;
  const int last_key = table_width * page_size - 1;      // the last key the table has a place for
  const int longest = window > 0 ? min(longest_given, window + 64) : longest_given;
  const int keys_per_split = (((longest + num_splits - 1) / num_splits) + 63) & ~63;
  const size_t head_stride = (size_t)page_size * head_size;   // elements of one head of one page
  const size_t page_stride = (size_t)num_kv * head_stride + page_pad;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // the pages of a tile's four blocks of 16 keys (a block of 16 lies in one page; pages of 64 keys and more
  // hold a whole tile): the same for every lane
  auto lookup = [&](int (&pg)[4], int tile0) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int key = __builtin_amdgcn_readfirstlane(min(tile0 + 16 * c, last_key));
      pg[c] = min(max(tab[key >> page_shift], 0), num_pages - 1);
    }
  };
  bf16x8 kf[4][NKS], vf[NDB][2];
  // a lane's chunk of 8 elements at head-size offset 32 ks + 8 g; where the head ends inside a step the lanes
  // beyond it read the last chunk again and drop it
  const int dlast = head_size - 8;
  auto load_keys = [&](const int (&pg)[4], int tile0) {
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const int off = 32 * (kb >> 1) + 8 * (r >> 2) + 4 * (kb & 1) + (r & 3);
      const int page = (r >> 3) ? pg[2 * (kb >> 1) + 1] : pg[2 * (kb >> 1)];
      const bf16_t* kp = k_pages + (size_t)page * page_stride + (size_t)kvh * head_stride +
                         (size_t)((tile0 + off) & pmask) * head_size;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) kf[kb][ks] = *(const bf16x8*)(kp + min(32 * ks + 8 * g, dlast));
    }
  };
  auto load_values = [&](const int (&pg)[4], int tile0) {
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      const int page = (g >> 1) ? pg[2 * st + 1] : pg[2 * st];
      const bf16_t* vp = v_pages + (size_t)page * page_stride + (size_t)kvh * head_stride + ((tile0 + 32 * st + 8 * g) & pmask);
#pragma unroll
      for (int db = 0; db < NDB; ++db)
        vf[db][st] = *(const bf16x8*)(vp + (size_t)min(16 * db + r, head_size - 1) * page_size);
    }
  };

  int pg[4], pgn[4];
  int tile0 = 0;
  bool fetched = false;
  if (window <= 0) {
    // the first tile of this wave's share, asked for before the request's length is known: from places that
    // are valid whatever it turns out to be, and masked afterwards
    tile0 = split * keys_per_split + 64 * wave;
    if (64 * wave < keys_per_split) {
      lookup(pg, tile0);
      load_keys(pg, tile0);
      if (PIPE) load_values(pg, tile0);
      fetched = true;
    }
  }
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int k_begin = (lo / 64) * 64 + split * keys_per_split;
  const int k_end = min(pos + 1, k_begin + keys_per_split);
  tile0 = k_begin + 64 * wave;

  bf16x8 qf[NKS];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    const bf16x8 qv = *(const bf16x8*)(q + (size_t)t * nq + h * head_size + min(32 * ks + 8 * g, dlast));
    qf[ks] = (32 * ks + 8 * g < head_size && col_on) ? qv : zero8;
  }
  float m = -INFINITY, l = 0.f;       // `l`: this lane's share of the sum (its own 16 keys a tile)
  f32x4 o[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db) o[db] = (f32x4){0.f, 0.f, 0.f, 0.f};

  if (tile0 < k_end && !fetched) {
    lookup(pg, tile0);
    load_keys(pg, tile0);
    if (PIPE) load_values(pg, tile0);
  }
  while (tile0 < k_end) {
    const int next = tile0 + 64 * NW;
    const bool more = next < k_end;
    f32x4 sc[4];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)   // a lane's chunk beyond the head's end holds the last chunk again: its query chunk is zero
        a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kb][ks], qf[ks], a, 0, 0, 0);
      sc[kb] = a;
    }
    if (PIPE && more) {
      lookup(pgn, next);
      load_keys(pgn, next);
    }
    // sc[kb][i] of a lane is the score of key tile0 + 32 (kb / 2) + 8 g + 4 (kb % 2) + i, the same in the 16
    // lanes of a row group
    const bool edge = tile0 + 64 > k_end || tile0 < lo;
    float mx = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        if (edge) {
          const int key = tile0 + 32 * (kb >> 1) + 8 * g + 4 * (kb & 1) + i;
          if (key < lo || key >= k_end) sc[kb][i] = -INFINITY;
        }
        mx = fmaxf(mx, sc[kb][i]);
      }
    mx = rows_max(mx);
    const float m_new = fmaxf(m, mx);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __expf(m - m_safe);
    float sum = 0.f;
    bf16x8 pf[2];
#pragma unroll
    for (int kb = 0; kb < 4; ++kb)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float pr = __expf(sc[kb][i] - m_safe);
        sum += pr;
        pf[kb >> 1][4 * (kb & 1) + i] = (bf16_t)pr;
      }
    l = l * alpha + sum;
    m = m_new;
    if (!PIPE) load_values(pg, tile0);
    if (edge) {
      // values of keys that are not the request's (beyond its end, before its window, in a page that was given
      // back) may be anything: their probabilities are zero, and they must not be NaN
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int key = tile0 + 32 * st + 8 * g + j;
          if (key < lo || key >= k_end) {
#pragma unroll
            for (int db = 0; db < NDB; ++db) vf[db][st][j] = 0;
          }
        }
    }
#pragma unroll
    for (int db = 0; db < NDB; ++db) {   // blocks beyond the head's end repeat its last row; they are never stored
      f32x4 a = o[db] * alpha;
      a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db][0], pf[0], a, 0, 0, 0);
      a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[db][1], pf[1], a, 0, 0, 0);
      o[db] = a;
    }
    if (more) {
      if (PIPE) {
        load_values(pgn, next);
      } else {
        lookup(pg, next);
        load_keys(pg, next);
      }
    }
    tile0 = next;
  }
  // o[db][i] of a lane is element 16 db + 4 g + i of the weighted values of its column (without PACK the same in
  // the 16 lanes of a row group)
  l = rows_sum(l);
  if (PACK ? r < COLS : r == 0) {
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) sm_o[wave][PACK ? r : 0][16 * db + 4 * g + i] = o[db][i];
  }
  if (PACK ? (g == 0 && r < COLS) : lane == 0) {
    sm_m[wave][PACK ? r : 0] = m;
    sm_l[wave][PACK ? r : 0] = l;
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < COLS * head_size; idx += 64 * NW) {
    const int col = idx / head_size, d = idx - col * head_size;
    if (PACK && col0 + col >= group) break;          // (columns beyond the group: none follows that is within it)
    const int hh = PACK ? kvh * group + col0 + col : h;
    float mm = sm_m[0][col];
#pragma unroll
    for (int w = 1; w < NW; ++w) mm = fmaxf(mm, sm_m[w][col]);
    const float ms = mm == -INFINITY ? 0.f : mm;
    float ll = 0.f, oo = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = __expf(sm_m[w][col] - ms);
      ll += sm_l[w][col] * f;
      oo += sm_o[w][col][d] * f;
    }
    if (num_splits == 1) {
      out[(size_t)t * nq + hh * head_size + d] = (bf16_t)(oo / ll);
    } else {
      const size_t pi = ((size_t)dz * num_heads + hh) * num_splits + split;
      part_o[pi * head_size + d] = oo;
      if (d == 0) {
        part_ml[pi * 2] = mm;
        part_ml[pi * 2 + 1] = ll;
      }
    }
  }
}

__global__ void attention_decode_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                              const int* __restrict__ run_start, const int* __restrict__ decode_runs,
                                              bf16_t* __restrict__ out, int num_heads, int head_size,
                                              int num_splits) {
  const int h = blockIdx.x, dz = blockIdx.y;
  const int run = decode_runs[dz];            // where the result goes is asked for beside the partial results
  const size_t base = ((size_t)dz * num_heads + h) * num_splits;
  if (num_splits <= 8) {
    // The usual case. Everything is asked for before anything is computed, so that the kernel waits for
    // memory once (shares beyond the last read the last one again and are left out of the sums); the sums
    // are made in the order of the loop below, to the same bits.
    float ms[8], ls[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      const size_t i = base + min(s, num_splits - 1);
      ms[s] = part_ml[i * 2];
      ls[s] = part_ml[i * 2 + 1];
    }
    const int t = run_start[run];
    for (int d = threadIdx.x; d < head_size; d += blockDim.x) {
      float os[8];
#pragma unroll
      for (int s = 0; s < 8; ++s) os[s] = part_o[(base + min(s, num_splits - 1)) * head_size + d];
      float mm = -INFINITY;
#pragma unroll
      for (int s = 0; s < 8; ++s)
        if (s < num_splits) mm = fmaxf(mm, ms[s]);
      float ll = 0.f, oo = 0.f;
#pragma unroll
      for (int s = 0; s < 8; ++s)
        if (s < num_splits) {
          const float f = ms[s] == -INFINITY ? 0.f : __expf(ms[s] - mm);
          ll += ls[s] * f;
          oo += os[s] * f;
        }
      out[((size_t)t * num_heads + h) * head_size + d] = (bf16_t)(oo / ll);
    }
    return;
  }
  float mm = -INFINITY;
  for (int s = 0; s < num_splits; ++s) mm = fmaxf(mm, part_ml[(base + s) * 2]);
  const int t = run_start[run];
  for (int d = threadIdx.x; d < head_size; d += blockDim.x) {
    float ll = 0.f, oo = 0.f;
    for (int s = 0; s < num_splits; ++s) {
      const float ms = part_ml[(base + s) * 2];
      const float f = ms == -INFINITY ? 0.f : __expf(ms - mm);
      ll += part_ml[(base + s) * 2 + 1] * f;
      oo += part_o[(base + s) * head_size + d] * f;
    }
    out[((size_t)t * num_heads + h) * head_size + d] = (bf16_t)(oo / ll);
  }
}

static int attention_decode_run(const void* q, const void* k_pages, const void* v_pages, const int* run_start,
                                const int* cached_lens, const int* table, int table_width, int page_size,
                                int num_pages, const int* decode_runs, int num_decode, void* out, float* part_o,
                                float* part_ml, int num_heads, int num_kv, int head_size, int window,
                                int num_splits, int waves, const int* longest, int page_pad, hipStream_t stream) {
  TNX_REQUIRE(num_heads > 0 && num_kv > 0 && num_heads % num_kv == 0, "attention_decode: bad head counts");
  TNX_REQUIRE(page_pad >= 0 && page_pad % 8 == 0, "attention_decode: bad distance between pages");
  TNX_REQUIRE(head_size % 16 == 0 && head_size >= 16 && head_size <= 256,
              "attention_decode: head size %d is not a multiple of 16 in [16, 256]", head_size);
  TNX_REQUIRE(page_size >= 16 && (page_size & (page_size - 1)) == 0,
              "attention_decode: page size %d is not a power of two from 16 up", page_size);
  int page_shift = 0;
  while ((1 << page_shift) < page_size) ++page_shift;
  TNX_REQUIRE(num_splits >= 1 && longest != nullptr, "attention_decode: bad split count or no length given");
  TNX_REQUIRE(num_splits == 1 || (part_o && part_ml), "attention_decode: splits need a workspace");
  TNX_REQUIRE(num_heads <= 65535 && num_decode <= 65535, "attention_decode: too many heads or requests");
  TNX_REQUIRE(waves == 4 || (waves == 8 && head_size <= 128),
              "attention_decode: blocks have 4 waves, or 8 up to head size 128; not %d at head size %d", waves, head_size);
  if (num_decode <= 0) return 0;
  // query heads that share keys and values are taken together, up to 16 a block (8 at head sizes beyond 128)
  const int group = num_heads / num_kv;
  const bool pack = group > 1;
  const int cols = head_size <= 128 ? 16 : 8;
  dim3 grid(num_splits, pack ? num_kv * ((group + cols - 1) / cols) : num_heads, num_decode);
#define MFMA_ARGS                                                                                                 \
  (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, run_start, cached_lens, table, table_width,    \
      page_shift, num_pages, decode_runs, (bf16_t*)out, part_o, part_ml, num_heads, num_kv, window, num_splits,    \
      longest, head_size, page_pad
#define LAUNCH_MFMA(NDB)                                                                         \
  if (waves == 8 && pack)                                                                        \
    attention_decode_mfma_kernel<NDB, 8, true><<<grid, 512, 0, stream>>>(MFMA_ARGS);             \
  else if (waves == 8)                                                                           \
    attention_decode_mfma_kernel<NDB, 8, false><<<grid, 512, 0, stream>>>(MFMA_ARGS);            \
  else if (pack)                                                                                 \
    attention_decode_mfma_kernel<NDB, 4, true><<<grid, 256, 0, stream>>>(MFMA_ARGS);             \
  else                                                                                           \
    attention_decode_mfma_kernel<NDB, 4, false><<<grid, 256, 0, stream>>>(MFMA_ARGS)
    // the registers are laid out for the next of these sizes; a smaller head repeats its last chunk there
    if (head_size <= 32) {
      LAUNCH_MFMA(2);
    } else if (head_size <= 64) {
      LAUNCH_MFMA(4);
    } else if (head_size <= 96) {
      LAUNCH_MFMA(6);
    } else if (head_size <= 128) {
      LAUNCH_MFMA(8);
    } else if (pack) {
      attention_decode_mfma_kernel<16, 4, true><<<grid, 256, 0, stream>>>(MFMA_ARGS);
    } else {
      attention_decode_mfma_kernel<16, 4, false><<<grid, 256, 0, stream>>>(MFMA_ARGS);
    }
#undef MFMA_ARGS
#undef LAUNCH_MFMA
  TNX_CHECK_LAUNCH("attention_decode");
  if (num_splits > 1) {
    attention_decode_merge_kernel<<<dim3(num_heads, num_decode), head_size < 64 ? 64 : head_size, 0, stream>>>(
        part_o, part_ml, run_start, decode_runs, (bf16_t*)out, num_heads, head_size, num_splits);
    TNX_CHECK_LAUNCH("attention_decode_merge");
  }
  return 0;
}

extern "C" int tnx_attention_decode(const void* q, const void* k_pages, const void* v_pages, const int* run_start,
                                    const int* cached_lens, const int* table, int table_width, int page_size,
                                    int num_pages, const int* decode_runs, int num_decode, void* out, float* part_o,
                                    float* part_ml, int num_heads, int num_kv, int head_size, int window,
                                    int num_splits, int waves, const int* longest, int page_pad,
                                    hipStream_t stream) {
  return attention_decode_run(q, k_pages, v_pages, run_start, cached_lens, table, table_width, page_size, num_pages,
                              decode_runs, num_decode, out, part_o, part_ml, num_heads, num_kv, head_size, window,
                              num_splits, waves, longest, page_pad, stream);
}

// The partial results of split keys for callers that cannot allocate: one array per GPU, held until the
// process ends. In host code this name is a stand-in, not a device address: the address on the current
// device comes from hipGetSymbolAddress, once per device, and only that address is handed to kernels.
static __device__ __align__(256) float tnx_decode_scratch[TNX_DECODE_SCRATCH_FLOATS];

#define TNX_MAX_DEVICES 64
static float* decode_scratch_of_device[TNX_MAX_DEVICES];
static std::mutex decode_scratch_lock;

extern "C" int tnx_attention_decode_static(const void* q, const void* k_pages, const void* v_pages,
                                           const int* run_start, const int* cached_lens, const int* table,
                                           int table_width, int page_size, int num_pages, const int* decode_runs,
                                           int num_decode, void* out, int num_heads, int num_kv, int head_size,
                                           int window, int num_splits, int waves, const int* longest,
                                           hipStream_t stream) {
  TNX_REQUIRE(num_decode >= 0 && num_heads > 0 && head_size > 0 && num_splits >= 1,
              "attention_decode_static: bad sizes");
  const long long partials = (long long)num_decode * num_heads * num_splits;
  const long long floats = num_splits > 1 ? partials * (head_size + 2) : 0;
  TNX_REQUIRE(floats <= TNX_DECODE_SCRATCH_FLOATS,
              "attention_decode_static: %d requests x %d heads x %d splits at head size %d need %lld floats of "
              "partial results; the static array holds %d. Use fewer splits, or tnx_attention_decode with a "
              "workspace of the caller's",
              num_decode, num_heads, num_splits, head_size, floats, (int)TNX_DECODE_SCRATCH_FLOATS);
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  TNX_REQUIRE(e == hipSuccess && device >= 0 && device < TNX_MAX_DEVICES,
              "attention_decode_static: no current device (%s)", hipGetErrorString(e));
  float* scratch;
  {
    std::lock_guard<std::mutex> hold(decode_scratch_lock);
    if (decode_scratch_of_device[device] == nullptr) {
      float* address = nullptr;
      e = hipGetSymbolAddress((void**)&address, HIP_SYMBOL(tnx_decode_scratch));
      TNX_REQUIRE(e == hipSuccess && address != nullptr,
                  "attention_decode_static: the static array has no address on device %d (%s)", device,
                  hipGetErrorString(e));
      decode_scratch_of_device[device] = address;
    }
    scratch = decode_scratch_of_device[device];
  }
  // weighted values first, then (maximum, sum) pairs; every partial that the merge reads is written by this
  // call's first kernel, so nothing of an earlier call's contents has to be cleared
  float* part_o = scratch;
  float* part_ml = scratch + partials * head_size;
  return attention_decode_run(q, k_pages, v_pages, run_start, cached_lens, table, table_width, page_size, num_pages,
                              decode_runs, num_decode, out, part_o, part_ml, num_heads, num_kv, head_size, window,
                              num_splits, waves, longest, 0, stream);       // (pages that lie one behind the other)
}
