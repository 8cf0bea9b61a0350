// RMSNorm, with the residual addition fused in.
//
//   r = branch + residual          (float32; either operand may be absent)
//   residual <- r                  (kept in float32, written only when both are present)
//   out = r * rsqrt(mean(r^2) + eps) * (w + weight_offset)
//
// The reference has the two forms as separate kernels (vllm/kernels/layernorm_kernels.cu:13-38
// rms_norm_kernel, :41-68 fused_add_rms_norm_kernel), rounds the residual to the model's dtype
// and rounds the normalised value before the weight multiply. Here the residual stream stays in
// float32 and the row is rounded once, at the store.
//
// One workgroup per output row. ``rows`` (optional) gathers: output row i is computed from input
// row rows[i], and the residual is then left untouched.
#include "common.h"

template <typename TB, typename TO, typename TW>
__global__ __launch_bounds__(1024) void add_rms_norm_kernel(
    const TB* __restrict__ branch, float* __restrict__ residual, const TW* __restrict__ weight,
    TO* __restrict__ out, const int* __restrict__ rows, int H, float eps, float weight_offset) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const long src = rows ? (long)rows[r] : (long)r;
  const TB* b = branch ? branch + src * H : nullptr;
  float* res = residual ? residual + src * H : nullptr;
  const bool write_res = (b != nullptr) && (res != nullptr) && (rows == nullptr);
  // When the sum cannot be written back to the residual (gather, or no residual), the second
  // pass recomputes it from the inputs.
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float x = 0.f;
    if (b) x += to_f32<TB>(b[i]);
    if (res) x += res[i];
    if (write_res) res[i] = x;
    ss += x * x;
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)H + eps);
  TO* o = out + (long)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float x;
    if (write_res) {
      x = res[i];
    } else {
      x = 0.f;
      if (b) x += to_f32<TB>(b[i]);
      if (res) x += res[i];
    }
    o[i] = from_f32<TO>(x * inv * (to_f32<TW>(weight[i]) + weight_offset));
  }
}

// The same for rows whose length is a multiple of 4 and at most 4 * 4 * 1024: every thread keeps its
// elements in registers between the two passes (at most VPT vectors of 4), so the row is read once and
// nothing is read back from memory that was just written. One workgroup per output row.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float* p, float* x) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
  }
  static __device__ __forceinline__ void store(float* p, const float* x) {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
  }
};
template <> struct Vec4<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float* x) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    x[0] = __uint_as_float(v.x << 16); x[1] = __uint_as_float(v.x & 0xffff0000u);
    x[2] = __uint_as_float(v.y << 16); x[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float* x) {
    uint2 v;
    v.x = (uint32_t)f32_to_bf16(x[0]) | ((uint32_t)f32_to_bf16(x[1]) << 16);
    v.y = (uint32_t)f32_to_bf16(x[2]) | ((uint32_t)f32_to_bf16(x[3]) << 16);
    *reinterpret_cast<uint2*>(p) = v;
  }
};

// PART: the branch is a product left as partial sums (``partial``; ``branch`` is not read).
template <typename TB, typename TO, typename TW, int VPT, bool PART>
__global__ __launch_bounds__(1024) void add_rms_norm_vec_kernel(
    const TB* __restrict__ branch, float* __restrict__ residual, const TW* __restrict__ weight,
    TO* __restrict__ out, const int* __restrict__ rows, int H, float eps, float weight_offset,
    LmsfPartialSum partial) {
  __shared__ float red[16];
  const int r = blockIdx.x;
  const long src = rows ? (long)rows[r] : (long)r;
  const TB* b = (!PART && branch) ? branch + src * H : nullptr;
  float* res = residual ? residual + src * H : nullptr;
  const bool write_res = (PART || b != nullptr) && (res != nullptr) && (rows == nullptr);
  const int nvec = H / 4;
  float x[VPT][4];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int v = threadIdx.x + k * blockDim.x;
#pragma unroll
    for (int e = 0; e < 4; ++e) x[k][e] = 0.f;
    if (v < nvec) {
      if (PART) partial_sum_value4(partial, (int)src, v * 4, x[k]);
      else if (b) Vec4<TB>::load(b + v * 4, x[k]);
      if (res) {
        float y[4];
        Vec4<float>::load(res + v * 4, y);
#pragma unroll
        for (int e = 0; e < 4; ++e) x[k][e] += y[e];
      }
      if (write_res) Vec4<float>::store(res + v * 4, x[k]);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += x[k][e] * x[k][e];
    }
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)H + eps);
  TO* o = out + (long)r * H;
#pragma unroll
  for (int k = 0; k < VPT; ++k) {
    const int v = threadIdx.x + k * blockDim.x;
    if (v < nvec) {
      float w[4], y[4];
      Vec4<TW>::load(weight + v * 4, w);
#pragma unroll
      for (int e = 0; e < 4; ++e) y[e] = x[k][e] * inv * (w[e] + weight_offset);
      Vec4<TO>::store(o + v * 4, y);
    }
  }
}

template <typename TB, typename TO, typename TW>
static void launch_norm(const void* branch, float* residual, const void* weight, void* out, const int* rows,
                        int n_out, int H, float eps, float woff, hipStream_t stream) {
  const LmsfPartialSum none = {nullptr, nullptr, 0, 0, 0};
  const bool aligned = (branch == nullptr || (((uintptr_t)branch) & 15u) == 0) &&
                       (residual == nullptr || (((uintptr_t)residual) & 15u) == 0) &&
                       (((uintptr_t)weight) & 15u) == 0 && (((uintptr_t)out) & 15u) == 0;
  if (H % 4 == 0 && H <= 16384 && aligned) {
    const int nvec = H / 4;
    int threads = (nvec + 63) / 64 * 64;
    if (threads > 1024) threads = 1024;
    // few vectors per thread also for short rows: at most 256 threads while one vector each suffices
    const int vpt = (nvec + threads - 1) / threads;
#define NORM_VEC(V)                                                                                          \
  hipLaunchKernelGGL((add_rms_norm_vec_kernel<TB, TO, TW, V, false>), dim3(n_out), dim3(threads), 0, stream,  \
                     (const TB*)branch, residual, (const TW*)weight, (TO*)out, rows, H, eps, woff, none)
    if (vpt <= 1) NORM_VEC(1);
    else if (vpt == 2) NORM_VEC(2);
    else if (vpt == 3) NORM_VEC(3);
    else NORM_VEC(4);
#undef NORM_VEC
    return;
  }
  int threads = ((H + 3) / 4 + 63) / 64 * 64;
  if (threads > 1024) threads = 1024;
  if (threads < 64) threads = 64;
  hipLaunchKernelGGL((add_rms_norm_kernel<TB, TO, TW>), dim3(n_out), dim3(threads), 0, stream,
                     (const TB*)branch, residual, (const TW*)weight, (TO*)out, rows, H, eps, woff);
}

// branch [n_in, H] of branch_dtype or null; residual [n_in, H] float32 or null (not both null);
// weight [H]; out [n_out, H]; rows int32 [n_out] or null (then n_out rows are rows 0..n_out-1).
extern "C" int lmsf_add_rms_norm(const void* branch, int branch_dtype, float* residual, const void* weight,
                                 int weight_dtype, void* out, int out_dtype, const int* rows, int n_out, int H,
                                 float eps, float weight_offset, hipStream_t stream) {
  LMSF_CHECK(branch != nullptr || residual != nullptr, "add_rms_norm: neither branch nor residual given");
  LMSF_CHECK(weight != nullptr && out != nullptr, "add_rms_norm: null weight or out");
  LMSF_CHECK(H > 0 && n_out >= 0, "add_rms_norm: bad sizes n_out=%d H=%d", n_out, H);
  LMSF_CHECK(eps > 0.f, "add_rms_norm: eps must be > 0");
  LMSF_CHECK((branch_dtype == LMSF_F32 || branch_dtype == LMSF_BF16) &&
                 (weight_dtype == LMSF_F32 || weight_dtype == LMSF_BF16) &&
                 (out_dtype == LMSF_F32 || out_dtype == LMSF_BF16),
             "add_rms_norm: unknown dtype code");
  if (n_out == 0) return 0;
  const int key = branch_dtype * 4 + out_dtype * 2 + weight_dtype;
  switch (key) {
    case 0: launch_norm<float, float, float>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 1: launch_norm<float, float, bf16_t>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 2: launch_norm<float, bf16_t, float>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 3: launch_norm<float, bf16_t, bf16_t>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 4: launch_norm<bf16_t, float, float>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 5: launch_norm<bf16_t, float, bf16_t>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 6: launch_norm<bf16_t, bf16_t, float>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    default: launch_norm<bf16_t, bf16_t, bf16_t>(branch, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
  }
  LMSF_LAUNCH_CHECK("add_rms_norm");
  return 0;
}

template <typename TO, typename TW>
static void launch_norm_partial(const LmsfPartialSum& ps, float* residual, const void* weight, void* out,
                                const int* rows, int n_out, int H, float eps, float woff, hipStream_t stream) {
  const int nvec = H / 4;
  int threads = (nvec + 63) / 64 * 64;
  if (threads > 1024) threads = 1024;
  const int vpt = (nvec + threads - 1) / threads;
#define NORM_PART(V)                                                                                              \
  hipLaunchKernelGGL((add_rms_norm_vec_kernel<bf16_t, TO, TW, V, true>), dim3(n_out), dim3(threads), 0, stream,   \
                     (const bf16_t*)nullptr, residual, (const TW*)weight, (TO*)out, rows, H, eps, woff, ps)
  if (vpt <= 1) NORM_PART(1);
  else if (vpt == 2) NORM_PART(2);
  else if (vpt == 3) NORM_PART(3);
  else NORM_PART(4);
#undef NORM_PART
}

// The same with the branch given as the partial sums of a bfloat16 product [M, H] whose K was split
// (lmsf_gemm_mid_partial): the reduction, the addition and the norm in one kernel. part: float32
// [n_split, M, H]; bias bfloat16 [H] or null. residual [M, H] float32 or null; rows as above, entries < M.
// Needs H a multiple of 4 and at most 16,384 and 16-byte aligned operands.
extern "C" int lmsf_add_rms_norm_partial(const float* part, const void* bias, int n_split, int M, float* residual,
                                         const void* weight, int weight_dtype, void* out, int out_dtype,
                                         const int* rows, int n_out, int H, float eps, float weight_offset,
                                         hipStream_t stream) {
  LMSF_CHECK(part != nullptr && weight != nullptr && out != nullptr, "add_rms_norm_partial: null pointer");
  LMSF_CHECK(n_split >= 1 && M >= 0 && n_out >= 0 && (rows != nullptr || n_out <= M),
             "add_rms_norm_partial: bad sizes splits=%d M=%d n_out=%d", n_split, M, n_out);
  LMSF_CHECK(H > 0 && H % 4 == 0 && H <= 16384, "add_rms_norm_partial: H=%d must be a multiple of 4 up to 16384", H);
  LMSF_CHECK(eps > 0.f, "add_rms_norm_partial: eps must be > 0");
  LMSF_CHECK((weight_dtype == LMSF_F32 || weight_dtype == LMSF_BF16) && (out_dtype == LMSF_F32 || out_dtype == LMSF_BF16),
             "add_rms_norm_partial: unknown dtype code");
  LMSF_CHECK(lmsf_aligned16(part) && lmsf_aligned16(weight) && lmsf_aligned16(out) &&
                 (residual == nullptr || lmsf_aligned16(residual)) && (bias == nullptr || (((uintptr_t)bias) & 7u) == 0),
             "add_rms_norm_partial: operands must be 16-byte aligned");
  if (n_out == 0) return 0;
  const LmsfPartialSum ps = {part, (const bf16_t*)bias, n_split, M, H};
  const int key = out_dtype * 2 + weight_dtype;
  switch (key) {
    case 0: launch_norm_partial<float, float>(ps, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 1: launch_norm_partial<float, bf16_t>(ps, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    case 2: launch_norm_partial<bf16_t, float>(ps, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
    default: launch_norm_partial<bf16_t, bf16_t>(ps, residual, weight, out, rows, n_out, H, eps, weight_offset, stream); break;
  }
  LMSF_LAUNCH_CHECK("add_rms_norm_partial");
  return 0;
}
