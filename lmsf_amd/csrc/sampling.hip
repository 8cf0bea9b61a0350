// Sampling from float32 logits: greedy, temperature, top-k, top-p, min-p, and the penalties.
//
// Pipeline of the reference (core/src/model_executor/layers/sampler.rs:839-971): penalties, divide
// by the temperature, top-k/top-p, min-p, float32 softmax, then argmax for greedy rows and
// argmax(probs / q) with q ~ Exp(1) for random rows (:326-361). The reference sorts the whole
// vocabulary for top-k/top-p (:139-210). Here one workgroup per row finds the two cut values by
// bisection on the order-preserving integer image of the floats, without a sort, and draws with the
// same exponential race written as argmax(x_i - log(-log u_i)), u_i from a counter-based generator
// keyed by (seed of the request, number of the draw, vocabulary index): the token does not depend
// on what else is in the batch.
//
// A bisection step over the whole vocabulary costs a pass over the row; 32 of them per cut are most of a
// millisecond at 128,256 entries. With a top-k of up to 1,024 the row is passed over twice instead: the k-th
// largest of the 1,024 threads' own maxima is a value that at least k entries reach, so everything the cuts
// can keep is among the entries that reach it; those (a few times k) are gathered in LDS, and the cuts and
// the draw work on them alone. Top-p without a top-k does the same from a value below which top-p removes
// everything whatever the rest of the row is; it gains where the distribution is peaked. Masses are added up there as integers (exp scaled by 2^32), so that the
// order in which the entries were gathered does not show. Rows without any cut draw over the whole
// vocabulary, split over several workgroups a row like the greedy search.
//
// Cut rules (ties at a cut value are kept together):
//   top-k : keep x >= k-th largest value                         (sampler.rs:170-178)
//   top-p : keep x whose mass of strictly larger values is < p   (sampler.rs:180-197: ascending
//           cumulative sums <= 1 - p are removed, the largest always stays)
//   min-p : keep x with prob >= min_p * max prob, i.e. x >= max + log(min_p)   (sampler.rs:305-325)
#include "common.h"
#include "no_alloc.h"

#include <math.h>

#include <mutex>

#define SAMP_THREADS 1024

// (-0 and +0 compare equal as numbers and get one key)
__device__ __forceinline__ uint32_t order_key(float f) {
  uint32_t b = __float_as_uint(f);
  if (b == 0x80000000u) b = 0u;
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

// Philox4x32-10; returns the first of the four output words.
__device__ __forceinline__ uint32_t philox_first(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                                 uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

__device__ __forceinline__ float gumbel_noise(uint64_t seed, uint32_t draw, uint32_t index) {
  const uint32_t r = philox_first(index, draw, 0u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32));
  // 23 bits: k + 0.5 is exact in float32 for k < 2^23, so u lies strictly inside (0, 1) and the noise is finite
  // (with 24 bits the largest k + 0.5 rounds up to 2^24, u to 1 and the noise to +inf: that entry would win)
  const float u = ((float)(r >> 9) + 0.5f) * (1.0f / 8388608.0f);
  return -logf(-logf(u));
}

__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* red) {
#pragma unroll
  for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, LMSF_WAVE);
  const int nw = blockDim.x / LMSF_WAVE;
  const int w = threadIdx.x / LMSF_WAVE, l = threadIdx.x % LMSF_WAVE;
  __syncthreads();
  if (l == 0) red[w] = v;
  __syncthreads();
  unsigned long long r = 0;
  for (int i = 0; i < nw; ++i) r += red[i];
  return r;
}

// Largest (value, lowest index) over the block; every thread gets the index.
__device__ __forceinline__ int block_argmax(float v, int idx, float* redv, int* redi) {
#pragma unroll
  for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, LMSF_WAVE);
    const int oi = __shfl_xor(idx, o, LMSF_WAVE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
  const int nw = blockDim.x / LMSF_WAVE;
  const int w = threadIdx.x / LMSF_WAVE, l = threadIdx.x % LMSF_WAVE;
  __syncthreads();
  if (l == 0) { redv[w] = v; redi[w] = idx; }
  __syncthreads();
  float bv = redv[0];
  int bi = redi[0];
  for (int i = 1; i < nw; ++i)
    if (redv[i] > bv || (redv[i] == bv && redi[i] < bi)) { bv = redv[i]; bi = redi[i]; }
  return bi;
}

__device__ __forceinline__ float key_value(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key & 0x7fffffffu) : ~key);
}

#define SAMP_CAND 8192   // entries the small-top-k path gathers in LDS (keys, then indices)

// The largest c with at least ``need`` of keys[0 .. n) >= c (the need-th largest key); every thread gets it.
__device__ __forceinline__ uint32_t lds_kth_largest(const uint32_t* keys, int n, unsigned long long need,
                                                    unsigned long long* redu) {
  uint32_t cur = 0u;
  for (int bit = 31; bit >= 0; --bit) {
    const uint32_t cand = cur | (1u << bit);
    unsigned long long cnt = 0;
    for (int j = threadIdx.x; j < n; j += SAMP_THREADS) cnt += keys[j] >= cand ? 1u : 0u;
    cnt = block_sum_u64(cnt, redu);
    if (cnt >= need) cur = cand;
  }
  return cur;
}

// exp(x - mx) for x <= mx as an integer: 2^32 at the maximum
__device__ __forceinline__ unsigned long long mass_fixed(float x, float mx) {
  return (unsigned long long)(expf(x - mx) * 4294967296.0f);
}

// f(i, row[i]) for this thread's entries i = tid, tid + SAMP_THREADS, ..., in ascending order, eight loads in
// flight at a time: one workgroup passes over a row of half a megabyte, and with a load per wave and trip the
// pass is as slow as the loads' latency.
template <typename F>
__device__ __forceinline__ void for_each_entry(const float* __restrict__ row, int V, F f) {
  if (((size_t)row & 15) == 0) {
    // a row that starts on a 16-byte boundary: four entries a load, four loads in flight
    const int V4 = V >> 2;
    const float4* row4 = reinterpret_cast<const float4*>(row);
    int q = threadIdx.x;
    for (; q + 3 * SAMP_THREADS < V4; q += 4 * SAMP_THREADS) {
      float4 x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) x[u] = row4[q + u * SAMP_THREADS];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = 4 * (q + u * SAMP_THREADS);
        f(i, x[u].x); f(i + 1, x[u].y); f(i + 2, x[u].z); f(i + 3, x[u].w);
      }
    }
    for (; q < V4; q += SAMP_THREADS) {
      const float4 x = row4[q];
      f(4 * q, x.x); f(4 * q + 1, x.y); f(4 * q + 2, x.z); f(4 * q + 3, x.w);
    }
    for (int i = 4 * V4 + threadIdx.x; i < V; i += SAMP_THREADS) f(i, row[i]);
    return;
  }
  int i = threadIdx.x;
  for (; i + 7 * SAMP_THREADS < V; i += 8 * SAMP_THREADS) {
    float x[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) x[u] = row[i + u * SAMP_THREADS];
#pragma unroll
    for (int u = 0; u < 8; ++u) f(i + u * SAMP_THREADS, x[u]);
  }
  for (; i < V; i += SAMP_THREADS) f(i, row[i]);
}

// One workgroup per row. temperature < 1e-5 means greedy (core/src/common/sampling_params.rs:156-163).
__global__ __launch_bounds__(SAMP_THREADS) void sample_kernel(
    const float* __restrict__ logits, long ld, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ min_p,
    const unsigned long long* __restrict__ seeds, const unsigned int* __restrict__ draws, int* __restrict__ out) {
  __shared__ float redf[16];
  __shared__ int redi[16];
  __shared__ unsigned long long redu[16];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + (long)r * ld;
  const float T = temperature ? temperature[r] : 0.f;
  const bool greedy = T < 1e-5f;

  if (greedy) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for_each_entry(row, V, [&](int i, float x) {
      if (x > bv) { bv = x; bi = i; }  // ascending i per thread: the first maximum wins
    });
    const int best = block_argmax(bv, bi, redf, redi);
    if (tid == 0) out[r] = best < V ? best : 0;
    return;
  }

  extern __shared__ __align__(16) uint32_t cand_keys[];   // [SAMP_CAND] keys, [SAMP_CAND] indices, [SAMP_THREADS] maxima
  uint32_t* cand_idx = cand_keys + SAMP_CAND;
  uint32_t* thread_max = cand_idx + SAMP_CAND;
  __shared__ unsigned int n_cand;
  const float invT = 1.0f / T;
  float mx = -INFINITY;
  for_each_entry(row, V, [&](int, float x) { mx = fmaxf(mx, x * invT); });
  thread_max[tid] = order_key(mx);   // (-inf for a thread without entries: below every entry)
  mx = block_max(mx, redf);
  const unsigned long long seed = seeds ? seeds[r] : 0ull;
  const unsigned int draw = draws ? draws[r] : 0u;
  const float p = top_p ? top_p[r] : 1.0f;
  const float mp = min_p ? min_p[r] : 0.f;
  const uint32_t kmax = order_key(mx);

  uint32_t cut = 0u;  // keep order_key(x) >= cut
  const int k = top_k ? top_k[r] : -1;
  const bool small_k = k > 0 && k < V && k <= SAMP_THREADS;
  const bool p_alone = p < 1.0f && !(k > 0 && k < V);
  if (small_k || p_alone) {
    // A value below which nothing can be kept. Top-k: at least k entries reach the k-th largest of the threads'
    // maxima. Top-p alone: entries whose exp(x - max) is below (1 - p) / V add up to less than 1 - p, which
    // is at most (1 - p) of the whole mass (the maximum alone contributes 1): top-p removes them all. With a
    // peaked distribution, as a model's, few entries are above either.
    const uint32_t floor_key = small_k ? lds_kth_largest(thread_max, SAMP_THREADS, (unsigned long long)k, redu)
                                       : order_key(mx + logf((1.0f - p) / (float)V));
    if (tid == 0) n_cand = 0u;
    __syncthreads();
    unsigned long long z_all = 0;   // top-p alone: the mass of every entry
    for_each_entry(row, V, [&](int i, float xr) {
      const float x = xr * invT;
      const uint32_t key = order_key(x);
      if (p_alone) z_all += mass_fixed(x, mx);
      // one addition to the counter per wave, not per entry: a flat row has a hundred thousand takers
      const bool take = key >= floor_key;
      const unsigned long long takers = __ballot(take);
      if (takers) {
        const int lane = threadIdx.x & (LMSF_WAVE - 1), leader = __ffsll((long long)takers) - 1;
        unsigned int base = 0u;
        if (lane == leader) base = atomicAdd(&n_cand, (unsigned int)__popcll(takers));
        base = __shfl(base, leader, LMSF_WAVE);
        const unsigned int at = base + (unsigned int)__popcll(takers & ((1ull << lane) - 1ull));
        if (take && at < SAMP_CAND) {
          cand_keys[at] = key;
          cand_idx[at] = (uint32_t)i;
        }
      }
    });
    __syncthreads();
    const int n = (int)n_cand;
    if (n <= SAMP_CAND) {      // (more: a flat distribution, or thousands of equal values; the passes below take those)
      cut = small_k ? lds_kth_largest(cand_keys, n, (unsigned long long)k, redu) : floor_key;
      if (p < 1.0f) {
        unsigned long long z = 0;
        if (p_alone) {
          z = z_all;
        } else {
          for (int j = tid; j < n; j += SAMP_THREADS)
            if (cand_keys[j] >= cut) z += mass_fixed(key_value(cand_keys[j]), mx);
        }
        z = block_sum_u64(z, redu);
        const unsigned long long target = (unsigned long long)((double)p * (double)z);
        uint32_t cur = 0u;
        for (int bit = 31; bit >= 0; --bit) {
          const uint32_t c = cur | (1u << bit);
          unsigned long long mass = 0;
          for (int j = tid; j < n; j += SAMP_THREADS)
            if (cand_keys[j] >= c && cand_keys[j] >= cut) mass += mass_fixed(key_value(cand_keys[j]), mx);
          mass = block_sum_u64(mass, redu);
          if (mass >= target) cur = c;
        }
        if (cur > cut) cut = cur;
      }
      if (mp > 0.f) {
        const uint32_t c = order_key(mx + logf(mp));
        if (c > cut) cut = c;
      }
      if (cut > kmax) cut = kmax;
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int j = tid; j < n; j += SAMP_THREADS) {
        if (cand_keys[j] < cut) continue;
        const int i = (int)cand_idx[j];
        const float y = key_value(cand_keys[j]) + gumbel_noise(seed, draw, (uint32_t)i);
        if (y > bv || (y == bv && i < bi)) { bv = y; bi = i; }
      }
      const int best = block_argmax(bv, bi, redf, redi);
      if (tid == 0) out[r] = best < V ? best : 0;
      return;
    }
  }
  // The passes over the whole row, for rows with more entries to keep than LDS holds (flat rows: a model with random
  // weights has them). The cut is searched four bits at a time, the 15 candidates of a digit counted in one pass:
  // 8 passes instead of 32 (a flat row of 128,256 entries with top-p 0.9: 1.3 -> 0.58 ms; a peaked one, gathered above:
  // 0.07). A pass costs about 45 us, and what it costs is instructions, not loads: one workgroup has one compute
  // unit's vector units for 128,256 entries. Counts and masses fall as the candidate rises, so the largest digit that
  // still reaches the target is the last one that does.
  if (k > 0 && k < V) {
    uint32_t cur = 0u;
    for (int shift = 28; shift >= 0; shift -= 4) {
      unsigned int cnt[15];
#pragma unroll
      for (int j = 0; j < 15; ++j) cnt[j] = 0u;
      for_each_entry(row, V, [&](int, float x) {
        const uint32_t key = order_key(x * invT);
#pragma unroll
        for (int j = 0; j < 15; ++j) cnt[j] += key >= (cur | ((uint32_t)(j + 1) << shift)) ? 1u : 0u;
      });
      uint32_t digit = 0u;
#pragma unroll
      for (int j = 0; j < 15; ++j)
        if (block_sum_u64(cnt[j], redu) >= (unsigned long long)k) digit = (uint32_t)(j + 1);
      cur |= digit << shift;
    }
    cut = cur;
  }
  if (p < 1.0f) {
    float z = 0.f;
    for_each_entry(row, V, [&](int, float xr) {
      const float x = xr * invT;
      if (order_key(x) >= cut) z += expf(x - mx);
    });
    z = block_sum(z, redf);
    const float target = p * z;
    uint32_t cur = 0u;
    for (int shift = 28; shift >= 0; shift -= 4) {
      float mass[15];
#pragma unroll
      for (int j = 0; j < 15; ++j) mass[j] = 0.f;
      for_each_entry(row, V, [&](int, float xr) {
        const float x = xr * invT;
        const uint32_t key = order_key(x);
        if (key < cut || key < cur) return;
        const float e = expf(x - mx);
#pragma unroll
        for (int j = 0; j < 15; ++j)
          if (key >= (cur | ((uint32_t)(j + 1) << shift))) mass[j] += e;
      });
      uint32_t digit = 0u;
#pragma unroll
      for (int j = 0; j < 15; ++j)
        if (block_sum(mass[j], redf) >= target) digit = (uint32_t)(j + 1);
      cur |= digit << shift;
    }
    if (cur > cut) cut = cur;
  }
  if (mp > 0.f) {
    const uint32_t c = order_key(mx + logf(mp));
    if (c > cut) cut = c;
  }
  // the maximum is always kept, whatever rounding did to the cuts
  if (cut > kmax) cut = kmax;

  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for_each_entry(row, V, [&](int i, float xr) {
    const float x = xr * invT;
    if (order_key(x) < cut) return;
    const float y = x + gumbel_noise(seed, draw, (uint32_t)i);
    if (y > bv) { bv = y; bi = i; }
  });
  const int best = block_argmax(bv, bi, redf, redi);
  if (tid == 0) out[r] = best < V ? best : 0;
}

// Greedy rows of a large vocabulary, in two small kernels: each of SPLIT workgroups finds the first maximum
// of its share of the row, then one wave per row picks among the shares (the lowest index wins ties, as in
// the kernel above). One workgroup per row leaves most of the chip idle when there are few rows.
#define ARGMAX_SPLIT 32
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits, long ld, int V,
                                                             float* __restrict__ pval, int* __restrict__ pidx) {
  __shared__ float redf[16];
  __shared__ int redi[16];
  const int r = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
  const int per = (V + ARGMAX_SPLIT - 1) / ARGMAX_SPLIT;
  const int lo = part * per, hi = min(V, lo + per);
  const float* row = logits + (long)r * ld;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + tid; i < hi; i += 256) {
    const float x = row[i];
    if (x > bv) { bv = x; bi = i; }
  }
  const int best = block_argmax(bv, bi, redf, redi);
  if (tid == 0) {
    pidx[r * ARGMAX_SPLIT + part] = best;
    pval[r * ARGMAX_SPLIT + part] = best < V ? row[best] : -INFINITY;
  }
}
// The same with the draw's noise: rows without any cut (temperature only, or greedy where it is below 1e-5).
__global__ __launch_bounds__(256) void noisy_argmax_partial_kernel(
    const float* __restrict__ logits, long ld, int V, const float* __restrict__ temperature,
    const unsigned long long* __restrict__ seeds, const unsigned int* __restrict__ draws, float* __restrict__ pval,
    int* __restrict__ pidx) {
  __shared__ float redf[16];
  __shared__ int redi[16];
  const int r = blockIdx.x, part = blockIdx.y, tid = threadIdx.x;
  const int per = (V + ARGMAX_SPLIT - 1) / ARGMAX_SPLIT;
  const int lo = part * per, hi = min(V, lo + per);
  const float* row = logits + (long)r * ld;
  const float T = temperature[r];
  const bool greedy = T < 1e-5f;
  const float invT = greedy ? 1.0f : 1.0f / T;
  const unsigned long long seed = seeds ? seeds[r] : 0ull;
  const unsigned int draw = draws ? draws[r] : 0u;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + tid; i < hi; i += 256) {
    const float x = row[i] * invT;
    const float y = greedy ? x : x + gumbel_noise(seed, draw, (uint32_t)i);
    if (y > bv) { bv = y; bi = i; }
  }
  // (the value is carried along: the last kernel compares the shares' best values, noise included)
#pragma unroll
  for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, LMSF_WAVE);
    const int oi = __shfl_xor(bi, o, LMSF_WAVE);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  const int w = tid / LMSF_WAVE, l = tid % LMSF_WAVE;
  if (l == 0) { redf[w] = bv; redi[w] = bi; }
  __syncthreads();
  if (tid == 0) {
    for (int i = 1; i < 256 / LMSF_WAVE; ++i)
      if (redf[i] > bv || (redf[i] == bv && redi[i] < bi)) { bv = redf[i]; bi = redi[i]; }
    pidx[r * ARGMAX_SPLIT + part] = bi;
    pval[r * ARGMAX_SPLIT + part] = bv;
  }
}
__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pval, const int* __restrict__ pidx,
                                                          int V, int* __restrict__ out) {
  const int r = blockIdx.x, l = threadIdx.x;
  float v = l < ARGMAX_SPLIT ? pval[r * ARGMAX_SPLIT + l] : -INFINITY;
  int idx = l < ARGMAX_SPLIT ? pidx[r * ARGMAX_SPLIT + l] : 0x7fffffff;
#pragma unroll
  for (int o = LMSF_WAVE / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(v, o, LMSF_WAVE);
    const int oi = __shfl_xor(idx, o, LMSF_WAVE);
    if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
  }
  if (l == 0) out[r] = idx < V ? idx : 0;
}

// Floats (and as many ints) of scratch that lmsf_sample wants for R greedy rows; 0: none needed.
extern "C" long lmsf_sample_scratch_elems(int R, int V) { return (V >= 16384 && R <= 256) ? (long)R * ARGMAX_SPLIT : 0; }

// logits [R, V] float32 with row stride ld. temperature/top_k/top_p/min_p/seeds/draws are per-row
// device arrays; any of them may be null (greedy, no cut, seed 0, draw 0).
// scratch (optional): lmsf_sample_scratch_elems(R, V) floats followed by as many ints; with it, a large
// vocabulary is searched by several workgroups per row where no row has a cut: with no temperature (all rows
// greedy), or with top_k, top_p and min_p all null.
extern "C" int lmsf_sample(const float* logits, long ld, int R, int V, const float* temperature, const int* top_k,
                           const float* top_p, const float* min_p, const unsigned long long* seeds,
                           const unsigned int* draws, int* out, void* scratch, hipStream_t stream) {
  LMSF_CHECK(logits && out, "sample: null pointer");
  LMSF_CHECK(R >= 0 && V > 0 && ld >= V, "sample: bad sizes R=%d V=%d ld=%ld", R, V, ld);
  if (R == 0) return 0;
  const long elems = lmsf_sample_scratch_elems(R, V);
  if (temperature == nullptr && scratch != nullptr && elems > 0) {
    float* pval = (float*)scratch;
    int* pidx = (int*)(pval + elems);
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(R, ARGMAX_SPLIT), dim3(256), 0, stream, logits, ld, V, pval, pidx);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(R), dim3(64), 0, stream, pval, pidx, V, out);
    LMSF_LAUNCH_CHECK("sample (greedy)");
    return 0;
  }
  if (top_k == nullptr && top_p == nullptr && min_p == nullptr && scratch != nullptr && elems > 0) {
    // no row has a cut: the draw over the whole vocabulary, several workgroups a row
    float* pval = (float*)scratch;
    int* pidx = (int*)(pval + elems);
    hipLaunchKernelGGL(noisy_argmax_partial_kernel, dim3(R, ARGMAX_SPLIT), dim3(256), 0, stream, logits, ld, V,
                       temperature, seeds, draws, pval, pidx);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(R), dim3(64), 0, stream, pval, pidx, V, out);
    LMSF_LAUNCH_CHECK("sample (no cuts)");
    return 0;
  }
  const size_t smem = (size_t)(2 * SAMP_CAND + SAMP_THREADS) * sizeof(uint32_t);
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(sample_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("sample: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  hipLaunchKernelGGL(sample_kernel, dim3(R), dim3(SAMP_THREADS), smem, stream, logits, ld, V, temperature, top_k, top_p,
                     min_p, seeds, draws, out);
  LMSF_LAUNCH_CHECK("sample");
  return 0;
}

// ---------------------------------------------------------------- greedy tokens without an allocation
// The partial results of argmax_partial_kernel in a device array of the library's own (declared in
// no_alloc.h). In host code the array's name is only a stand-in for the symbol; the address on the current
// device comes from hipGetSymbolAddress and is kept per device.
static __device__ __align__(256) unsigned char scratch[(size_t)LMSF_GREEDY_STATIC_MAX_ROWS * ARGMAX_SPLIT * 8];

static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[64] = {nullptr};

// Address of ``scratch`` on the current device, or null (error set).
static void* greedy_static_scratch() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    lmsf_set_error("greedy_tokens_static: cannot tell the current device");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      lmsf_set_error("greedy_tokens_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

extern "C" int lmsf_greedy_tokens_static(const float* logits, long ld, int R, int V, int* out, hipStream_t stream) {
  LMSF_CHECK(logits && out, "greedy_tokens_static: null pointer");
  LMSF_CHECK(R >= 0 && V > 0 && ld >= V, "greedy_tokens_static: bad sizes R=%d V=%d ld=%ld", R, V, ld);
  LMSF_CHECK(R <= LMSF_GREEDY_STATIC_MAX_ROWS,
             "greedy_tokens_static: %d rows, the library's own buffer holds the partial results of %d at most", R,
             LMSF_GREEDY_STATIC_MAX_ROWS);
  if (R == 0) return 0;
  void* ptr = greedy_static_scratch();
  if (ptr == nullptr) return 2;
  // values first, then indices, each R * ARGMAX_SPLIT entries: every entry is written by the first kernel
  // before the second reads it, so the last call's contents do not matter
  float* pval = (float*)ptr;
  int* pidx = (int*)(pval + (size_t)R * ARGMAX_SPLIT);
  hipLaunchKernelGGL(argmax_partial_kernel, dim3(R, ARGMAX_SPLIT), dim3(256), 0, stream, logits, ld, V, pval, pidx);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(R), dim3(64), 0, stream, pval, pidx, V, out);
  LMSF_LAUNCH_CHECK("greedy_tokens_static");
  return 0;
}

// ---------------------------------------------------------------- penalties
// counts[r, v] = (times v occurs in the output tokens of row r) | PROMPT_BIT if v occurs in the
// prompt. tokens is the concatenation over rows of [prompt tokens, output tokens];
// offsets[r] .. offsets[r+1] is row r's range and prompt_lens[r] how many of them are prompt.
#define PROMPT_BIT 0x40000000

__global__ __launch_bounds__(256) void penalty_count_kernel(const int* __restrict__ tokens,
                                                            const int* __restrict__ offsets,
                                                            const int* __restrict__ prompt_lens,
                                                            int* __restrict__ counts, int V) {
  const int r = blockIdx.x;
  const int b = offsets[r], e = offsets[r + 1], np = prompt_lens[r];
  int* c = counts + (long)r * V;
  for (int i = b + threadIdx.x; i < e; i += blockDim.x) {
    const int tok = tokens[i];
    if (tok < 0 || tok >= V) continue;
    if (i - b < np)
      atomicOr(&c[tok], PROMPT_BIT);
    else
      atomicAdd(&c[tok], 1);
  }
}

// core/src/model_executor/layers/sampler.rs:48-137: seen tokens: x > 0 ? x / rep : x * rep;
// then x -= frequency * output count; then x -= presence * [output count > 0].
__global__ __launch_bounds__(256) void penalty_apply_kernel(float* __restrict__ logits, long ld,
                                                            const int* __restrict__ counts, int V,
                                                            const float* __restrict__ presence,
                                                            const float* __restrict__ frequency,
                                                            const float* __restrict__ repetition) {
  const int r = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= V) return;
  const int c = counts[(long)r * V + i];
  if (c == 0) return;
  const int n_out = c & (PROMPT_BIT - 1);
  float x = logits[(long)r * ld + i];
  const float rep = repetition[r];
  x = x > 0.f ? x / rep : x * rep;
  x -= frequency[r] * (float)n_out;
  if (n_out > 0) x -= presence[r];
  logits[(long)r * ld + i] = x;
}

// counts must be an int32 [R, V] buffer filled with zeros before the call.
extern "C" int lmsf_apply_penalties(float* logits, long ld, int R, int V, const int* tokens, const int* offsets,
                                    const int* prompt_lens, int* counts, const float* presence,
                                    const float* frequency, const float* repetition, hipStream_t stream) {
  LMSF_CHECK(logits && tokens && offsets && prompt_lens && counts && presence && frequency && repetition,
             "apply_penalties: null pointer");
  LMSF_CHECK(R >= 0 && V > 0 && ld >= V, "apply_penalties: bad sizes R=%d V=%d ld=%ld", R, V, ld);
  LMSF_CHECK((V + 255) / 256 <= 65535, "apply_penalties: vocabulary too large");
  if (R == 0) return 0;
  hipLaunchKernelGGL(penalty_count_kernel, dim3(R), dim3(256), 0, stream, tokens, offsets, prompt_lens, counts, V);
  hipLaunchKernelGGL(penalty_apply_kernel, dim3(R, (V + 255) / 256), dim3(256), 0, stream, logits, ld, counts, V,
                     presence, frequency, repetition);
  LMSF_LAUNCH_CHECK("apply_penalties");
  return 0;
}
