// Embedding gather and gated activation.
#include "common.h"

// ---------------------------------------------------------------- embedding
// out[t, :] = float32(table[ids[t], :]) * scale. The output is the float32 residual stream.
// The reference gathers rows with candle's index_select
// (core/src/model_executor/layers/vocab_parallel_embedding.rs:28-38). An id outside [0, V)
// gives a row of zeros and raises a flag that the host reads (ids are also checked on the host
// before a step; the kernel never reads outside the table).
template <typename TW>
__global__ __launch_bounds__(256) void embedding_kernel(const int* __restrict__ ids, const TW* __restrict__ table,
                                                        float* __restrict__ out, int H, int V, float scale,
                                                        int* __restrict__ bad_flag) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* o = out + (long)t * H;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = 0.f;
    if (threadIdx.x == 0 && bad_flag) atomicOr(bad_flag, 1);
    return;
  }
  const TW* row = table + (long)id * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32<TW>(row[i]) * scale;
}

extern "C" int lmsf_embedding(const int* ids, const void* table, int table_dtype, float* out, int n_tokens, int H,
                              int V, float scale, int* bad_flag, hipStream_t stream) {
  LMSF_CHECK(ids && table && out, "embedding: null pointer");
  LMSF_CHECK(n_tokens >= 0 && H > 0 && V > 0, "embedding: bad sizes n=%d H=%d V=%d", n_tokens, H, V);
  LMSF_CHECK(table_dtype == LMSF_F32 || table_dtype == LMSF_BF16, "embedding: unknown dtype code %d", table_dtype);
  if (n_tokens == 0) return 0;
  if (table_dtype == LMSF_F32)
    hipLaunchKernelGGL((embedding_kernel<float>), dim3(n_tokens), dim3(256), 0, stream, ids, (const float*)table, out,
                       H, V, scale, bad_flag);
  else
    hipLaunchKernelGGL((embedding_kernel<bf16_t>), dim3(n_tokens), dim3(256), 0, stream, ids, (const bf16_t*)table,
                       out, H, V, scale, bad_flag);
  LMSF_LAUNCH_CHECK("embedding");
  return 0;
}

// ---------------------------------------------------------------- token ids from the step before
// ids[i] = prev[src[i]] where src[i] >= 0: a step that is launched before the host has read the tokens that the
// step before it sampled takes them from where the sampler left them on the device.
__global__ __launch_bounds__(256) void patch_tokens_kernel(int* __restrict__ ids, const int* __restrict__ src,
                                                           const int* __restrict__ prev, int n, int n_prev) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int s = src[i];
  if (s >= 0 && s < n_prev) ids[i] = prev[s];
}

extern "C" int lmsf_patch_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t stream) {
  LMSF_CHECK(ids && src && prev, "patch_tokens: null pointer");
  LMSF_CHECK(n >= 0 && n_prev >= 0, "patch_tokens: bad sizes n=%d n_prev=%d", n, n_prev);
  if (n == 0) return 0;
  hipLaunchKernelGGL(patch_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, ids, src, prev, n, n_prev);
  LMSF_LAUNCH_CHECK("patch_tokens");
  return 0;
}

// ---------------------------------------------------------------- gated activation
// out[t, i] = act(in[t, i]) * in[t, I + i], act computed in float32.
// kind 0: silu(x) = x / (1 + exp(-x))   (vllm/kernels/activation_kernels.cu:26-42)
// kind 1: gelu(x) = x/2 (1 + erf(x / sqrt 2)) (vllm/kernels/activation_kernels.cu:44-51)
template <typename T, int KIND>
__global__ __launch_bounds__(256) void gated_act_kernel(const T* __restrict__ in, T* __restrict__ out, int I,
                                                        long in_stride) {
  const long t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= I) return;
  const float g = to_f32<T>(in[t * in_stride + i]);
  const float u = to_f32<T>(in[t * in_stride + I + i]);
  float a;
  if (KIND == 0)
    a = g / (1.0f + expf(-g));
  else
    a = 0.5f * g * (1.0f + erff(g * 0.70710678118654752f));
  out[t * (long)I + i] = from_f32<T>(a * u);
}

// The same with 16-byte accesses: 8 bfloat16 or 4 float32 per thread.
template <typename T, int KIND>
__global__ __launch_bounds__(256) void gated_act_vec_kernel(const T* __restrict__ in, T* __restrict__ out, int I,
                                                            long in_stride) {
  constexpr int N = Vec16<T>::N;
  const long t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * N;
  if (i >= I) return;
  Vec16<T> g, u, o;
  g.load(in + t * in_stride + i);
  u.load(in + t * in_stride + I + i);
#pragma unroll
  for (int e = 0; e < N; ++e) {
    const float x = g.get(e);
    float a;
    if (KIND == 0)
      a = x / (1.0f + expf(-x));
    else
      a = 0.5f * x * (1.0f + erff(x * 0.70710678118654752f));
    o.set(e, a * u.get(e));
  }
  o.store(out + t * (long)I + i);
}

extern "C" int lmsf_gated_act(const void* in, void* out, int dtype, int n_tokens, int I, long in_stride, int kind,
                              hipStream_t stream) {
  LMSF_CHECK(in && out, "gated_act: null pointer");
  LMSF_CHECK(n_tokens >= 0 && I > 0 && in_stride >= 2L * I, "gated_act: bad sizes n=%d I=%d stride=%ld", n_tokens, I,
             in_stride);
  LMSF_CHECK((I + 255) / 256 <= 65535, "gated_act: intermediate size %d too large", I);
  LMSF_CHECK(kind == 0 || kind == 1, "gated_act: unknown activation %d", kind);
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "gated_act: unknown dtype code %d", dtype);
  if (n_tokens == 0) return 0;
  const int per = dtype == LMSF_F32 ? 4 : 8;   // elements of a 16-byte access
  if (I % per == 0 && in_stride % per == 0 && lmsf_aligned16(in) && lmsf_aligned16(out)) {
    const int vecs = I / per;
    dim3 vgrid(n_tokens, (vecs + 255) / 256), vblock(256);
#define GAV(T, K) \
  hipLaunchKernelGGL((gated_act_vec_kernel<T, K>), vgrid, vblock, 0, stream, (const T*)in, (T*)out, I, in_stride)
    if (dtype == LMSF_F32) {
      if (kind == 0) GAV(float, 0); else GAV(float, 1);
    } else {
      if (kind == 0) GAV(bf16_t, 0); else GAV(bf16_t, 1);
    }
#undef GAV
    LMSF_LAUNCH_CHECK("gated_act");
    return 0;
  }
  dim3 grid(n_tokens, (I + 255) / 256), block(256);
#define GA(T, K) hipLaunchKernelGGL((gated_act_kernel<T, K>), grid, block, 0, stream, (const T*)in, (T*)out, I, in_stride)
  if (dtype == LMSF_F32) {
    if (kind == 0) GA(float, 0); else GA(float, 1);
  } else {
    if (kind == 0) GA(bf16_t, 0); else GA(bf16_t, 1);
  }
#undef GA
  LMSF_LAUNCH_CHECK("gated_act");
  return 0;
}
