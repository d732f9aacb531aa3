// Token selection from float32 logits: argmax, and temperature / top-k / top-p sampling with a draw by
// inverse CDF from a counter-based random number (Philox-4x32-10, keyed by the request's seed, counter =
// the request's step), so that a request's draws do not depend on what else is in the batch.
//
// Order among tokens is total: by logit, ties to the lower token id (a 64-bit key: ordered logit bits above
// the inverted token id). Top-k keeps the k largest keys. Top-p keeps, of those, every token whose
// predecessors in descending order hold less than top_p of the softmax mass (the first token always).
// Both thresholds are found without sorting, by narrowing level by level with 256 bins a level (the bytes of
// the key; for top-p first the distance below the row's maximum), until few enough keys are left to rank in
// LDS. The draw runs over the kept tokens in ascending order of token id.
#include "common.h"

TNX_DEFINE_ERROR_API

#define SAMPLE_THREADS 1024
// The most keys that are gathered in LDS and ranked against one another there (each against all: what a wave
// reads from LDS is the limit, 256 keys take a few microseconds, 1,024 would take a hundred).
#define SAMPLE_GATHER 256

__device__ __forceinline__ uint64_t order_key(float x, int idx) {
  if (x != x) x = -INFINITY;  // NaN orders last
  if (x == 0.f) x = 0.f;      // -0 and +0 are one value: the lower token id decides between them
  uint32_t u = __float_as_uint(x);
  u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
  return ((uint64_t)u << 32) | (uint32_t)(~(uint32_t)idx);
}

__device__ __forceinline__ float philox_uniform(uint64_t seed, uint64_t counter) {
  const uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
  uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = 0, c3 = 0;
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(M0, c0), lo0 = M0 * c0;
    const uint32_t hi1 = __umulhi(M1, c2), lo1 = M1 * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += W0; k1 += W1;
  }
  return (float)(c0 >> 8) * (1.0f / 16777216.0f);
}

// One block of 1,024 threads a row; four logits a load where the rows allow it.
__global__ void __launch_bounds__(1024)
argmax_kernel(const float* __restrict__ logits, int* __restrict__ out, int vocab) {
  __shared__ unsigned long long best[16];
  const float* row = logits + (size_t)blockIdx.x * vocab;
  uint64_t b = 0;
  if ((vocab & 3) == 0) {
    const f32x4* row4 = (const f32x4*)row;
    for (int i = threadIdx.x; i < vocab / 4; i += 1024) {
      const f32x4 v = row4[i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint64_t k = order_key(v[j], 4 * i + j);
        b = k > b ? k : b;
      }
    }
  } else {
    for (int i = threadIdx.x; i < vocab; i += 1024) {
      const uint64_t k = order_key(row[i], i);
      b = k > b ? k : b;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const uint64_t other = __shfl_xor((unsigned long long)b, o, 64);
    b = other > b ? other : b;
  }
  if ((threadIdx.x & 63) == 0) best[threadIdx.x >> 6] = b;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 16; ++w) b = best[w] > b ? best[w] : b;
    out[blockIdx.x] = (int)(~(uint32_t)b);
  }
}

extern "C" int tnx_argmax(const float* logits, int* out, int rows, int vocab, hipStream_t stream) {
  TNX_REQUIRE(rows >= 0 && vocab > 0, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  if (rows == 0) return 0;
  argmax_kernel<<<rows, 1024, 0, stream>>>(logits, out, vocab);
  TNX_CHECK_LAUNCH("argmax");
  return 0;
}

// kept[slot of the request of row rows[i]] = tokens[i]: the chosen tokens, left where the next step's
// embedding finds them by the request's slot; and landing[i] = tokens[i] in pinned host memory, where the
// host reads them once the kernel has ended.
__global__ void store_tokens_kernel(const int* __restrict__ tokens, const int* __restrict__ rows,
                                    const int* __restrict__ token_request, const int* __restrict__ slots, int n,
                                    int* __restrict__ kept, int kept_size, int* __restrict__ landing) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int slot = slots[token_request[rows[i]]];
  if (slot >= 0 && slot < kept_size) kept[slot] = tokens[i];
  if (landing) landing[i] = tokens[i];
}

extern "C" int tnx_store_tokens(const int* tokens, const int* rows, const int* token_request, const int* slots,
                                int n, int* kept, int kept_size, int* landing, hipStream_t stream) {
  TNX_REQUIRE(n >= 0 && kept_size > 0, "store_tokens: bad sizes n=%d size=%d", n, kept_size);
  if (n == 0) return 0;
  store_tokens_kernel<<<(n + 255) / 256, 256, 0, stream>>>(tokens, rows, token_request, slots, n, kept, kept_size,
                                                           landing);
  TNX_CHECK_LAUNCH("store_tokens");
  return 0;
}

// logits[row, token[row]] = -inf where token[row] >= 0: a token that must not be chosen.
__global__ void ban_tokens_kernel(float* __restrict__ logits, const int* __restrict__ token, int rows, int vocab) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r < rows && token[r] >= 0 && token[r] < vocab) logits[(size_t)r * vocab + token[r]] = -INFINITY;
}

// logits[rows[i], tokens[i]] = -inf for a list of (row, token) pairs: tokens that must not follow what a
// request has generated (the n-grams it may not repeat).
__global__ void ban_pairs_kernel(float* __restrict__ logits, const int* __restrict__ rows,
                                 const int* __restrict__ tokens, int n, int num_rows, int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int r = rows[i], t = tokens[i];
  if (r >= 0 && r < num_rows && t >= 0 && t < vocab) logits[(size_t)r * vocab + t] = -INFINITY;
}

extern "C" int tnx_ban_pairs(float* logits, const int* rows, const int* tokens, int n, int num_rows, int vocab,
                             hipStream_t stream) {
  TNX_REQUIRE(n >= 0 && num_rows >= 0 && vocab > 0, "ban_pairs: bad sizes n=%d rows=%d vocab=%d", n, num_rows, vocab);
  if (n == 0) return 0;
  ban_pairs_kernel<<<(n + 255) / 256, 256, 0, stream>>>(logits, rows, tokens, n, num_rows, vocab);
  TNX_CHECK_LAUNCH("ban_pairs");
  return 0;
}

extern "C" int tnx_ban_tokens(float* logits, const int* token, int rows, int vocab, hipStream_t stream) {
  TNX_REQUIRE(rows >= 0 && vocab > 0, "ban_tokens: bad sizes rows=%d vocab=%d", rows, vocab);
  if (rows == 0) return 0;
  ban_tokens_kernel<<<(rows + 63) / 64, 64, 0, stream>>>(logits, token, rows, vocab);
  TNX_CHECK_LAUNCH("ban_tokens");
  return 0;
}

// Inclusive sums from the top: out[d] = x[d] + x[d + 1] + ... + x[255], by the first 256 threads of the block
// (four waves); `carry` holds four values. Every thread of the block calls it.
template <typename T>
__device__ __forceinline__ void sums_from_the_top(const T* x, T* out, T* carry) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  T v = 0;
  if (tid < 256) {
    v = x[255 - tid];                    // thread t takes digit 255 - t: a scan upwards over t runs down the digits
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const T w = __shfl_up(v, o, 64);
      if (lane >= o) v += w;
    }
    if (lane == 63) carry[wave] = v;
  }
  __syncthreads();
  if (tid < 256) {
    for (int w = 0; w < wave; ++w) v += carry[w];
    out[255 - tid] = v;
  }
  __syncthreads();
}

// A weight of at most 1 as a whole number of 2^-40: 24 bits before and 16 behind the point of w * 2^24. Sums of
// such numbers do not depend on the order they are added in, and differ from the exact sum by less than
// 2^-40 a term.
__device__ __forceinline__ unsigned long long fixed40(float w) {
  const float w24 = w * 16777216.f;
  const uint32_t whole = (uint32_t)w24;
  const uint32_t rest = (uint32_t)((w24 - (float)whole) * 65536.f);
  return ((unsigned long long)whole << 16) + rest;
}

// exp(a - m) for a <= m, to the last place or two of a float: the rounding of a - m is found (two-sum) and put
// back after the exponential, which is the library's full-precision one. What is below 2^-40 counts as nothing
// (fixed40 would cut it off anyway); that takes in a = -inf, and m = +inf beside a finite a.
__device__ __forceinline__ float exp_below(float a, float m) {
  if (a == m) return 1.f;
  const float d = a - m;
  if (!(d > -30.f)) return 0.f;
  const float b = -m, bb = d - a;
  const float err = (a - (d - bb)) + (b - bb);
  const float e = expf(d);
  return fmaf(e, err, e);
}

// One block per row; a row with temperature 0 takes its argmax.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperature, const int* __restrict__ top_k,
              const float* __restrict__ top_p, const long long* __restrict__ seeds,
              const long long* __restrict__ counters, const int* __restrict__ min_keep, int* __restrict__ out,
              int vocab) {
  __shared__ unsigned int cnt[256];
  __shared__ unsigned long long mass[256];           // in units of 2^-40, like every sum of weights here
  // Eight copies of both, a lane adding to copy lane % 8: in the first pass nearly all keys of a row fall into
  // two or three bins, and 64 lanes adding to one word take their turns one after the other.
  __shared__ unsigned int cnt8[256 * 8];
  __shared__ unsigned long long mass8[256 * 8];     // in units of 2^-40: whole numbers add up in any order alike
  const int copy = threadIdx.x & 7;
  __shared__ unsigned long long best[16];
  __shared__ int sh_digit;
  __shared__ unsigned int sh_remaining, sh_bin;
  __shared__ unsigned long long sh_above;
  __shared__ int sh_result, sh_last, sh_n, sh_owner, sh_owner_last;
  __shared__ unsigned long long sh_key, sh_itotal;
  __shared__ unsigned long long ipart[SAMPLE_THREADS];
  __shared__ unsigned long long tkey[SAMPLE_GATHER], ckey[SAMPLE_GATHER], tmass[SAMPLE_GATHER];
  __shared__ float tval[SAMPLE_GATHER];
  __shared__ unsigned int cnt_above[256], carry_u[4];
  __shared__ unsigned long long mass_above[256], carry_m[4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rowi = blockIdx.x;
  const float* row = logits + (size_t)rowi * vocab;
  const float temp = temperature[rowi];
  const bool greedy = !(temp > 0.f);
  const int keep = min_keep ? max(min_keep[rowi], 1) : 1;
  int k = top_k[rowi];
  if (k > 0) k = max(k, keep);
  // after a top-k of no more than SAMPLE_GATHER the kept tokens are gathered and the rest is done over these
  const bool few = !greedy && k > 0 && k < vocab && k <= SAMPLE_GATHER;
  const float inv_temp = greedy ? 0.f : 1.f / temp;     // for the bins of the search only; weights divide by temp

  // the largest key: argmax, and the maximum for the softmax (the gathered tokens bring their own)
  float xmax = 0.f;
  int arg = 0;
  if (!few) {
    uint64_t b = 0;
    for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
      const uint64_t key = order_key(row[i], i);
      b = key > b ? key : b;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const uint64_t other = __shfl_xor((unsigned long long)b, o, 64);
      b = other > b ? other : b;
    }
    if (lane == 0) best[wave] = b;
    __syncthreads();
    b = best[0];
    for (int w = 1; w < 16; ++w) b = best[w] > b ? best[w] : b;
    arg = (int)(~(uint32_t)b);
    if (greedy) {
      if (tid == 0) out[rowi] = arg;
      return;
    }
    xmax = row[arg] / temp;
  }

  // A token's share of the softmax before it is divided by the sum, as sampling.py:337-345 computes it: the
  // logit divided by the temperature (a true division), less the largest such, exponentiated in full precision;
  // as a whole number of 2^-40. A NaN has none, as it orders last.
  auto weight = [&](float x) -> unsigned long long { return x != x ? 0ull : fixed40(exp_below(x / temp, xmax)); };
  // p of a sum of weights, rounded down
  auto share = [](float p, unsigned long long total) -> unsigned long long {
    return (unsigned long long)((double)p * (double)total);
  };

  // the k-th largest key of the row, by radix selection; every thread of the block calls it together
  auto kth_largest = [&](unsigned int k) -> uint64_t {
    uint64_t prefix = 0, mask = 0;
    unsigned int remaining = k;
    for (int pass = 0; pass < 8; ++pass) {
      const int shift = 56 - 8 * pass;
      for (int j = tid; j < 256 * 8; j += SAMPLE_THREADS) cnt8[j] = 0;
      __syncthreads();
      for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
        const uint64_t key = order_key(row[i], i);
        if ((key & mask) == prefix) atomicAdd(&cnt8[((unsigned int)(key >> shift) & 255u) * 8 + copy], 1u);
      }
      __syncthreads();
      if (tid < 256) {
        unsigned int c = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) c += cnt8[tid * 8 + j];
        cnt[tid] = c;
      }
      __syncthreads();
      // the digit of the `remaining`-th largest: the highest one with that many keys at or above it
      sums_from_the_top(cnt, cnt_above, carry_u);
      if (tid < 256) {
        const unsigned int here = cnt_above[tid], over = tid < 255 ? cnt_above[tid + 1] : 0u;
        if ((here >= remaining && over < remaining) || (tid == 0 && here < remaining)) {
          sh_digit = tid;
          sh_remaining = remaining - min(over, remaining);
          sh_bin = cnt[tid];
        }
      }
      __syncthreads();
      prefix |= (uint64_t)sh_digit << shift;
      mask |= 0xFFull << shift;
      remaining = sh_remaining;
      const unsigned int bin = sh_bin;
      __syncthreads();
      if (bin == remaining) break;  // everything under this prefix is kept: the threshold is the prefix itself
      if (pass < 7 && bin <= SAMPLE_GATHER) {
        // few keys are left under the prefix: they are gathered, and the one with remaining - 1 larger
        // ones beside it is the threshold (keys differ, so there is exactly one)
        if (tid == 0) sh_n = 0;
        __syncthreads();
        for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
          const uint64_t key = order_key(row[i], i);
          if ((key & mask) == prefix) tkey[atomicAdd(&sh_n, 1)] = key;
        }
        __syncthreads();
        if (tid < (int)bin) {
          const uint64_t mine = tkey[tid];
          unsigned int larger = 0;
          for (unsigned int j = 0; j < bin; ++j) larger += tkey[j] > mine ? 1u : 0u;
          if (larger == remaining - 1) sh_key = mine;
        }
        __syncthreads();
        prefix = sh_key;
        __syncthreads();
        break;
      }
    }
    return prefix;
  };

  // top-k: tokens with key >= floor_key are kept; never fewer than `min_keep` (sampling.py:204-205)
  uint64_t floor_key = 0;
  if (k > 0 && k < vocab) floor_key = kth_largest((unsigned int)k);

  const float p = top_p[rowi];
  // a counter below zero asks for the constant 0.5 the reference calls deterministic (hlo.py:2455-2456)
  const float u = counters[rowi] < 0 ? 0.5f : philox_uniform((uint64_t)seeds[rowi], (uint64_t)counters[rowi]);
  if (few) {
    // Few tokens are left, the k largest exactly (keys differ in their token ids): they are gathered, one a
    // thread, put in the order of their token ids, and top-p and the draw are made over these alone.
    if (tid == 0) {
      sh_n = 0;
      sh_result = -1;
      sh_last = -1;
    }
    __syncthreads();
    for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
      const uint64_t key = order_key(row[i], i);
      if (key >= floor_key) {
        const int at = atomicAdd(&sh_n, 1);
        if (at < SAMPLE_GATHER) {
          tkey[at] = key;
          tval[at] = row[i] != row[i] ? -INFINITY : row[i] / temp;
        }
      }
    }
    __syncthreads();
    const int n = min(sh_n, SAMPLE_GATHER);
    const bool mine_too = wave * 64 < n;         // a wave with none of them has nothing to find out
    float largest = -INFINITY;
    for (int j = 0; mine_too && j < n; ++j) largest = fmaxf(largest, tval[j]);
    __syncthreads();
    if (tid < n) tmass[tid] = fixed40(exp_below(tval[tid], largest));     // (all -inf: alike, 1 each)
    __syncthreads();
    // of each of them: its place in the order of token ids, and the mass and the number of those with a larger key
    const bool have = tid < n;
    const uint64_t my_key = have ? tkey[tid] : 0;
    const unsigned long long my_val = have ? tmass[tid] : 0;
    const uint32_t my_low = (uint32_t)my_key;          // the complement of the token id: larger is earlier
    unsigned long long above = 0, z = 0;
    int rank = 0, place = 0;
    for (int j = 0; mine_too && j < n; ++j) {
      const uint64_t kj = tkey[j];
      const unsigned long long e = tmass[j];
      z += e;
      if (kj > my_key) {
        above += e;
        ++rank;
      }
      place += (uint32_t)kj > my_low ? 1 : 0;
    }
    // top-p keeps a token while those above it hold less than p of the mass, the largest always, and never
    // fewer than `keep` (sampling.py:213-249, :232)
    const bool kept = have && (p >= 1.f || above < share(p, z) || rank == 0 || rank < keep);
    if (tid < SAMPLE_GATHER) ipart[tid] = 0;
    __syncthreads();
    if (have) {
      ckey[place] = my_key;
      ipart[place] = kept ? my_val : 0;
      if (kept) atomicMax(&sh_last, place);
    }
    __syncthreads();
    const unsigned long long mine = tid < SAMPLE_GATHER ? ipart[tid] : 0;
    __syncthreads();
    if (wave == 0) {          // exclusive scan of the kept masses, in the order of the token ids
      unsigned long long local[SAMPLE_GATHER / 64], run = 0;
#pragma unroll
      for (int j = 0; j < SAMPLE_GATHER / 64; ++j) {
        local[j] = run;
        run += ipart[lane * (SAMPLE_GATHER / 64) + j];
      }
      unsigned long long incl = run;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const unsigned long long w = __shfl_up(incl, o, 64);
        if (lane >= o) incl += w;
      }
#pragma unroll
      for (int j = 0; j < SAMPLE_GATHER / 64; ++j) ipart[lane * (SAMPLE_GATHER / 64) + j] = incl - run + local[j];
      if (lane == 63) sh_itotal = incl;
    }
    __syncthreads();
    const unsigned long long total = sh_itotal;
    unsigned long long goal = share(u, total);
    if (total > 0 && goal >= total) goal = total - 1;
    const unsigned long long base = tid < SAMPLE_GATHER ? ipart[tid] : 0;
    if (mine > 0 && base <= goal && goal < base + mine) sh_result = tid;       // one thread at most
    __syncthreads();
    if (tid == 0) {
      const int pick = sh_result >= 0 ? sh_result : max(sh_last, 0);
      out[rowi] = (int)(~(uint32_t)ckey[pick]);
    }
    return;
  }

  // top-p: the smallest kept key is the last one whose predecessors hold less than p of the mass. The search
  // narrows level by level, at each with a count and a mass for each of 256 bins: first bins an eighth wide
  // of the distance below the row's maximum, then each of these in 256 (over such bins the keys of a row
  // spread, where the first bytes of the key, sign, exponent and first fraction bits, are the same for most of
  // them), then the bytes of the key among the tokens of the chosen bin; the first level's sums give the
  // whole mass.
  if (p < 1.f) {
    // both larger for larger values; 255, 255 for the maximum
    auto below_max = [&](float x, int& coarse, int& fine) {
      if (x != x) x = -INFINITY;      // as in the order of the keys
      const float t = fmaxf((xmax - x * inv_temp) * 8.f, 0.f);
      const float c = fminf(floorf(t), 255.f);
      coarse = 255 - (int)c;
      fine = 255 - (int)fminf((t - c) * 256.f, 255.f);
    };
    unsigned long long target = 0;
    int level = -1, sublevel = -1;
    uint64_t prefix = 0, mask = 0;
    unsigned long long above = 0;
    for (int pass = -2; pass < 8; ++pass) {
      const int shift = 56 - 8 * max(pass, 0);
      for (int j = tid; j < 256 * 8; j += SAMPLE_THREADS) {
        cnt8[j] = 0;
        mass8[j] = 0;
      }
      __syncthreads();
      for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
        const float x = row[i];
        const uint64_t key = order_key(x, i);
        int coarse, fine;
        below_max(x, coarse, fine);
        const bool in = pass == -2 || (coarse == level && (pass == -1 || (fine == sublevel && (key & mask) == prefix)));
        if (key >= floor_key && in) {
          const unsigned int digit = pass == -2 ? coarse : pass == -1 ? fine : (unsigned int)(key >> shift) & 255u;
          const unsigned int d = digit * 8 + copy;
          atomicAdd(&cnt8[d], 1u);
          atomicAdd(&mass8[d], weight(x));
        }
      }
      __syncthreads();
      if (tid < 256) {
        unsigned int c = 0;
        unsigned long long m = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          c += cnt8[tid * 8 + j];
          m += mass8[tid * 8 + j];
        }
        cnt[tid] = c;
        mass[tid] = m;
      }
      __syncthreads();
      // the lowest digit in use with less than the target above it (the highest in use, if none has)
      sums_from_the_top(mass, mass_above, carry_m);
      sums_from_the_top(cnt, cnt_above, carry_u);
      if (pass == -2) target = share(p, mass_above[0]);
      if (tid == 0) sh_digit = 256;
      __syncthreads();
      if (tid < 256 && cnt[tid] > 0) {
        const unsigned long long over = above + (tid < 255 ? mass_above[tid + 1] : 0);     // the mass above this digit
        const bool top = tid == 255 || cnt_above[tid + 1] == 0;                  // no digit in use above it
        if (over < target || top) atomicMin(&sh_digit, tid);
      }
      __syncthreads();
      if (tid == sh_digit) {
        sh_above = above + (tid < 255 ? mass_above[tid + 1] : 0);
        sh_bin = cnt[tid];
      }
      __syncthreads();
      if (pass == -2) {
        level = sh_digit;
      } else if (pass == -1) {
        sublevel = sh_digit;
      } else {
        prefix |= (uint64_t)sh_digit << shift;
        mask |= 0xFFull << shift;
      }
      above = sh_above;
      const unsigned int bin = sh_bin;
      __syncthreads();
      if (pass >= 0 && bin == 1) break;
      if (pass < 7 && bin <= SAMPLE_GATHER) {
        // few keys are left in the bin: they are gathered with their masses, and the threshold is the lowest
        // of them with less than the target above it (the largest of them has: its bin was chosen so)
        if (tid == 0) {
          sh_n = 0;
          sh_key = ~0ull;
        }
        __syncthreads();
        for (int i = tid; i < vocab; i += SAMPLE_THREADS) {
          const float x = row[i];
          const uint64_t key = order_key(x, i);
          int coarse, fine;
          below_max(x, coarse, fine);
          if (key >= floor_key && coarse == level && (sublevel < 0 || fine == sublevel) && (key & mask) == prefix) {
            const int at = atomicAdd(&sh_n, 1);
            tkey[at] = key;
            tmass[at] = weight(x);
          }
        }
        __syncthreads();
        if (tid < (int)bin) {
          const uint64_t mine = tkey[tid];
          unsigned long long over = above;
          bool top = true;
          for (unsigned int j = 0; j < bin; ++j)
            if (tkey[j] > mine) {
              over += tmass[j];
              top = false;
            }
          if (over < target || top) atomicMin(&sh_key, (unsigned long long)mine);
        }
        __syncthreads();
        prefix = sh_key;
        __syncthreads();
        break;
      }
    }
    uint64_t by_mass = prefix > floor_key ? prefix : floor_key;
    if (keep > 1) {
      // at least `keep` tokens stay, the largest ones (sampling.py:232): the floor is no higher than the
      // keep-th largest key, and no lower than what top-k left
      const uint64_t nth = keep < vocab ? kth_largest((unsigned int)keep) : 0;
      const uint64_t least = nth > floor_key ? nth : floor_key;
      by_mass = by_mass < least ? by_mass : least;
    }
    floor_key = by_mass;
  }

  // the draw, over the kept tokens in ascending order of token id; thread t owns a contiguous segment, which
  // it reads four floats a load: segments are counted from the 16-byte boundary at or before the row's start
  // (`lead` floats before it), and a group of four that reaches outside the row is read one by one
  const int lead = (int)(((uintptr_t)row >> 2) & 3);
  const int seg = (((vocab + lead + SAMPLE_THREADS - 1) / SAMPLE_THREADS) + 3) & ~3;
  const int i0 = tid * seg - lead;           // may lie before the row or beyond it
  auto four = [&](int i, float (&x)[4]) {
    if (i >= 0 && i + 3 < vocab) {
      const float4 v = *(const float4*)(row + i);
      x[0] = v.x, x[1] = v.y, x[2] = v.z, x[3] = v.w;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) x[e] = i + e >= 0 && i + e < vocab ? row[i + e] : 0.f;
    }
  };
  // the masses are added as whole numbers of 2^-40: the sums are the same whatever the order, so the thread
  // that owns the drawn point finds it in its segment, and the draw is that of exact arithmetic to 2^-40 a token
  unsigned long long s = 0;
  int last = -1;
#pragma unroll 4
  for (int q = 0; q < seg; q += 4) {
    float x[4];
    four(i0 + q, x);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = i0 + q + e;
      if (i >= 0 && i < vocab && order_key(x[e], i) >= floor_key) {
        s += weight(x[e]);
        last = i;
      }
    }
  }
  if (tid == 0) {
    sh_result = -1;
    sh_last = -1;
    sh_owner = -1;
  }
  ipart[tid] = s;
  __syncthreads();
  if (last >= 0) atomicMax(&sh_last, last);
  // exclusive scan of ipart[] by one wave: 16 values per lane
  if (wave == 0) {
    unsigned long long local[16];
    unsigned long long run = 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      local[j] = run;
      run += ipart[lane * 16 + j];
    }
    unsigned long long incl = run;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const unsigned long long v = __shfl_up(incl, o, 64);
      if (lane >= o) incl += v;
    }
    const unsigned long long base = incl - run;
#pragma unroll
    for (int j = 0; j < 16; ++j) ipart[lane * 16 + j] = base + local[j];
    if (lane == 63) sh_itotal = incl;
  }
  __syncthreads();
  const unsigned long long total = sh_itotal;
  unsigned long long goal = share(u, total);
  if (total > 0 && goal >= total) goal = total - 1;
  // thread t owns [base_t, base_{t+1}): the scanned values tile the line without gaps
  const unsigned long long base = ipart[tid];
  const unsigned long long next = tid + 1 < SAMPLE_THREADS ? ipart[tid + 1] : total;
  // its owner's segment is walked by the first wave, 64 tokens a turn: one trip to memory where the owner alone
  // would make one for every four tokens, each waiting for the one before
  if (last >= 0 && base <= goal && goal < next) {
    sh_owner = tid;
    sh_owner_last = last;
  }
  __syncthreads();
  if (wave == 0 && sh_owner >= 0) {
    const int o0 = sh_owner * seg - lead;
    unsigned long long run = ipart[sh_owner];
    int pick = -1;
    for (int q = 0; q < seg && pick < 0; q += 64) {
      const int i = o0 + q + lane;
      const bool ok = q + lane < seg && i >= 0 && i < vocab;
      const float x = ok ? row[i] : 0.f;
      const bool kept = ok && order_key(x, i) >= floor_key;
      unsigned long long incl = kept ? weight(x) : 0;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const unsigned long long v = __shfl_up(incl, o, 64);
        if (lane >= o) incl += v;
      }
      const unsigned long long hit = __ballot(kept && run + incl > goal);
      if (hit) pick = o0 + q + __ffsll(hit) - 1;
      run += __shfl(incl, 63, 64);
    }
    if (lane == 0) sh_result = pick >= 0 ? pick : sh_owner_last;
  }
  __syncthreads();
  if (tid == 0) out[rowi] = sh_result >= 0 ? sh_result : sh_last >= 0 ? sh_last : arg;
}

extern "C" int tnx_sample(const float* logits, const float* temperature, const int* top_k, const float* top_p,
                          const long long* seeds, const long long* counters, const int* min_keep, int* out,
                          int rows, int vocab, hipStream_t stream) {
  TNX_REQUIRE(rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", rows, vocab);
  TNX_REQUIRE(vocab <= (1 << 22), "sample: a vocabulary of %d is more than the %d that the sums of masses (whole "
              "numbers of 2^-40 in 64 bits) are sized for", vocab, 1 << 22);
  if (rows == 0) return 0;
  sample_kernel<<<rows, SAMPLE_THREADS, 0, stream>>>(logits, temperature, top_k, top_p, seeds, counters, min_keep,
                                                     out, vocab);
  TNX_CHECK_LAUNCH("sample");
  return 0;
}
