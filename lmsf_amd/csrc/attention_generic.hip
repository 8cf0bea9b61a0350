// Paged attention, general form: any number of query tokens per request, any head size that is a
// multiple of 4 up to 256, any page size, float32 or bfloat16 storage, float32 arithmetic.
//
// Query token t belongs to request segment seg[t] and stands at position pos[t]. It attends to
// the keys at positions j in [max(0, pos - window + 1), pos] of that request, read from the pages
// (key j lives in page block_table[seg][j / page_size] at offset j % page_size; K pages are
// [page, kv_head, offset, d], V pages [page, kv_head, d, offset]). All keys of a step
// are written to the pages before this kernel runs, so prompts, portions of prompts and single
// decoded tokens are one case.
//
// Function computed, per query head h with kv head g = h / (nh / nkv)
// (core/src/model_executor/layers/attention.rs:91-103, :139-155 for prompts;
// vllm/kernels/attention/attention_kernels.cu:82-414 for decoding):
//   s_j = scale * <q, k_j>;  p = softmax_j(s);  out = sum_j p_j v_j
// with an exact softmax (the reference's decode kernel divides by sum + 1e-6, :279).
//
// One workgroup of 256 threads per (token, head): keys are taken 256 at a time, one key per
// thread for the scores, an online softmax across chunks, and the P V product with the threads
// arranged as (key group, output dim).
#include "common.h"

#include <math.h>

#define GEN_THREADS 256

template <typename T>
__global__ __launch_bounds__(GEN_THREADS) void paged_attention_generic_kernel(
    const T* __restrict__ q, long q_stride, T* __restrict__ out, long out_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, const int* __restrict__ block_tables, int bt_width, const int* __restrict__ seg,
    const int* __restrict__ pos, int nh, int nkv, int d, int ps, float scale, int window) {
  extern __shared__ float smem[];
  float* sq = smem;                       // [d] query, pre-scaled
  float* sp = sq + d;                     // [256] scores, then probabilities
  int* srow = (int*)(sp + GEN_THREADS);   // [256] (page * nkv + g) * ps + offset of each key
  float* sacc = (float*)(srow + GEN_THREADS);  // [256] partial outputs of the key groups
  __shared__ float red[16];

  const int t = blockIdx.x, h = blockIdx.y;
  const int tid = threadIdx.x;
  const int s = seg[t], p = pos[t];
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int g = h / (nh / nkv);
  const int* bt = block_tables + (long)s * bt_width;

  for (int i = tid; i < d; i += GEN_THREADS) sq[i] = to_f32<T>(q[(long)t * q_stride + h * d + i]) * scale;

  const int ngroups = GEN_THREADS / d > 0 ? GEN_THREADS / d : 1;  // d <= 256
  const int og = tid / d, oi = tid % d;                            // (key group, output dim) of this thread
  const bool pv_active = og < ngroups;
  float acc = 0.f, m = -INFINITY, l = 0.f;
  __syncthreads();

  for (int j0 = lo; j0 <= p; j0 += GEN_THREADS) {
    const int j = j0 + tid;
    float sc = -INFINITY;
    if (j <= p) {
      const int page = bt[j / ps];
      const int row = (page * nkv + g) * ps + j % ps;
      srow[tid] = row;
      const T* kr = k_pages + (long)row * d;
      float dot = 0.f;
      for (int i = 0; i < d; i += 4) {
        dot += sq[i] * to_f32<T>(kr[i]) + sq[i + 1] * to_f32<T>(kr[i + 1]) + sq[i + 2] * to_f32<T>(kr[i + 2]) +
               sq[i + 3] * to_f32<T>(kr[i + 3]);
      }
      sc = dot;
    }
    const float cmax = block_max(sc, red);
    const float m_new = fmaxf(m, cmax);
    const float e = (j <= p) ? expf(sc - m_new) : 0.f;
    sp[tid] = e;
    const float csum = block_sum(e, red);  // has barriers: sp and srow are visible afterwards
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + csum;
    acc *= corr;
    m = m_new;
    __syncthreads();
    if (pv_active) {
      const int n = min(GEN_THREADS, p - j0 + 1);
      for (int jj = og; jj < n; jj += ngroups) {
        const int row = srow[jj], head_base = row / ps, off = row - head_base * ps;
        acc += sp[jj] * to_f32<T>(v_pages[((long)head_base * d + oi) * ps + off]);
      }
    }
    __syncthreads();
  }
  sacc[tid] = pv_active ? acc : 0.f;
  __syncthreads();
  if (tid < d) {
    float o = 0.f;
    for (int gg = 0; gg < ngroups; ++gg) o += sacc[gg * d + tid];
    out[(long)t * out_stride + h * d + tid] = from_f32<T>(o / l);
  }
}

extern "C" int lmsf_paged_attention_generic(const void* q, long q_stride, void* out, long out_stride,
                                            const void* k_pages, const void* v_pages, long num_pages,
                                            const int* block_tables, int bt_width, const int* seg, const int* pos,
                                            int n_tokens, int nh, int nkv, int d, int ps, float scale, int window,
                                            int dtype, hipStream_t stream) {
  LMSF_CHECK(q && out && k_pages && v_pages && block_tables && seg && pos, "paged_attention: null pointer");
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "paged_attention: unknown dtype code %d", dtype);
  LMSF_CHECK(nh > 0 && nkv > 0 && nh % nkv == 0, "paged_attention: heads %d not a multiple of kv heads %d", nh, nkv);
  LMSF_CHECK(d > 0 && d % 4 == 0 && d <= 256, "paged_attention: head size %d not supported (multiple of 4, <= 256)", d);
  LMSF_CHECK(ps > 0 && bt_width > 0 && num_pages > 0, "paged_attention: bad page geometry");
  LMSF_CHECK(num_pages * nkv * ps < 2147483647L, "paged_attention: cache too large for 32-bit row indices");
  LMSF_CHECK(q_stride >= (long)nh * d && out_stride >= (long)nh * d, "paged_attention: row strides too small");
  LMSF_CHECK(nh <= 65535, "paged_attention: too many heads");
  LMSF_CHECK(window >= 0, "paged_attention: negative window");
  if (n_tokens == 0) return 0;
  const size_t smem = (size_t)(d + 3 * GEN_THREADS) * 4;
  dim3 grid(n_tokens, nh), block(GEN_THREADS);
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((paged_attention_generic_kernel<float>), grid, block, smem, stream, (const float*)q, q_stride,
                       (float*)out, out_stride, (const float*)k_pages, (const float*)v_pages, block_tables, bt_width,
                       seg, pos, nh, nkv, d, ps, scale, window);
  else
    hipLaunchKernelGGL((paged_attention_generic_kernel<bf16_t>), grid, block, smem, stream, (const bf16_t*)q, q_stride,
                       (bf16_t*)out, out_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_tables,
                       bt_width, seg, pos, nh, nkv, d, ps, scale, window);
  LMSF_LAUNCH_CHECK("paged_attention_generic");
  return 0;
}
