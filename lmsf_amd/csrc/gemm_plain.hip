// Linear layer C[M, N] = A[M, K] W[N, K]^T (+ bias[N]) with float32 multiply-adds.
//
// This is the true 32-bit matrix product of the float32 path (no matrix-core instruction, no
// reduced-precision input mode), and the fallback of the bfloat16 path for shapes the fast kernels
// refuse. Inputs may be float32 or bfloat16; products and sums are float32, summed over k in
// ascending order inside each 16-wide slab. The reference calls cuBLASLt with float32 compute
// (tops/csrc/tops/tensorrt_llm/common/cublasMMWrapper.cpp:182-210) and adds the bias afterwards
// (core/src/model_executor/layers/linear.rs:101-104).
//
// 64x64 output tile per workgroup of 256 threads, 4x4 outputs per thread, K in slabs of 16 staged
// through LDS. Any M, N, K; rows may be strided (lda, ldw, ldc in elements).
#include "common.h"

#define GP_TILE 64
#define GP_BK 16

template <typename TA, typename TW, typename TO>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const TA* __restrict__ A, long lda, const TW* __restrict__ W,
                                                         long ldw, const TW* __restrict__ bias, TO* __restrict__ C,
                                                         long ldc, int M, int N, int K) {
  __shared__ float As[GP_BK][GP_TILE + 4];
  __shared__ float Ws[GP_BK][GP_TILE + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * GP_TILE, n0 = blockIdx.x * GP_TILE;
  const int lrow = tid / 4, lk = (tid % 4) * 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GP_BK) {
    const int gm = m0 + lrow, gn = n0 + lrow;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      As[lk + e][lrow] = (gm < M && k < K) ? to_f32<TA>(A[(long)gm * lda + k]) : 0.f;
      Ws[lk + e][lrow] = (gn < N && k < K) ? to_f32<TW>(W[(long)gn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GP_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + ty * 4 + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tx * 4 + j;
      if (gn >= N) continue;
      float r = acc[i][j];
      if (bias) r += to_f32<TW>(bias[gn]);
      C[(long)gm * ldc + gn] = from_f32<TO>(r);
    }
  }
}

// The same product for up to 16 rows of bfloat16 operands that the weight-streaming kernels refuse (a K that is no
// multiple of 8, rows that do not start on 16-byte boundaries): with so few rows the tiles above leave most of the
// chip idle (N / 64 workgroups, each walking all of K: 4,160 x 11,100 at 8 rows 1,290 us). Here a wave owns one output
// column; lane l takes k = l, l + 64, ... with 2-byte loads, which need no alignment, and the lanes' sums are added
// up in a fixed order. float32 products and sums.
#define GP_FEW_ROWS 16
// MT: rows the kernel walks (M rounded up to 1, 2, 4, 8 or 16; the rows beyond M repeat row M - 1 and are not written),
// so that the loop has no tests and the loads of several steps are in flight together. VEC: elements a load (2 where K
// and the row strides are even and the operands start on 4-byte boundaries, else 1). COLS: output columns a wave owns,
// more with more rows: every column's wave reads all of x from the caches, and with 16 rows and one column a wave that
// is 16 loads of x for each of W (4,160 x 11,100 at 16 rows: 1.5 GB through the caches).
template <typename TO, int MT, int VEC, int COLS>
__global__ __launch_bounds__(256) void gemm_plain_few_kernel(const bf16_t* __restrict__ A, long lda,
                                                             const bf16_t* __restrict__ W, long ldw,
                                                             const bf16_t* __restrict__ bias, TO* __restrict__ C,
                                                             long ldc, int M, int N, int K) {
  const int lane = threadIdx.x & 63;
  const int n0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * COLS;
  if (n0 >= N) return;
  float acc[MT][COLS];
  const bf16_t* a[MT];
  const bf16_t* w[COLS];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    a[m] = A + (long)min(m, M - 1) * lda;
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[m][c] = 0.f;
  }
#pragma unroll
  for (int c = 0; c < COLS; ++c) w[c] = W + (long)min(n0 + c, N - 1) * ldw;   // columns beyond N repeat the last one
  if (VEC == 2) {
#pragma unroll 2
    for (int k = 2 * lane; k < K; k += 128) {   // K is even: a pair never straddles the end
      float w0[COLS], w1[COLS];
#pragma unroll
      for (int c = 0; c < COLS; ++c) {
        const unsigned wp = *reinterpret_cast<const unsigned*>(w[c] + k);
        w0[c] = __uint_as_float(wp << 16);
        w1[c] = __uint_as_float(wp & 0xffff0000u);
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const unsigned xp = *reinterpret_cast<const unsigned*>(a[m] + k);
        const float x0 = __uint_as_float(xp << 16), x1 = __uint_as_float(xp & 0xffff0000u);
#pragma unroll
        for (int c = 0; c < COLS; ++c) acc[m][c] = fmaf(x1, w1[c], fmaf(x0, w0[c], acc[m][c]));
      }
    }
  } else {
#pragma unroll 2
    for (int k = lane; k < K; k += 64) {
      float wv[COLS];
#pragma unroll
      for (int c = 0; c < COLS; ++c) wv[c] = bf16_to_f32(w[c][k]);
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const float xv = bf16_to_f32(a[m][k]);
#pragma unroll
        for (int c = 0; c < COLS; ++c) acc[m][c] = fmaf(xv, wv[c], acc[m][c]);
      }
    }
  }
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int c = 0; c < COLS; ++c) {
      float r = acc[m][c];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) r += __shfl_xor(r, off, 64);
      if (lane == 0 && m < M && n0 + c < N) {
        if (bias) r += bf16_to_f32(bias[n0 + c]);
        C[(long)m * ldc + n0 + c] = from_f32<TO>(r);
      }
    }
}

template <typename TO>
static void launch_gemm_plain_few(const void* A, long lda, const void* W, long ldw, const void* bias, void* C, long ldc,
                                  int M, int N, int K, hipStream_t stream) {
  const dim3 block(256);
  const bool pairs = K % 2 == 0 && lda % 2 == 0 && ldw % 2 == 0 && (size_t)A % 4 == 0 && (size_t)W % 4 == 0;
#define FEW(MT_, COLS_)                                                                                                \
  do {                                                                                                                 \
    const dim3 grid((N + 4 * COLS_ - 1) / (4 * COLS_));                                                                \
    if (pairs)                                                                                                         \
      hipLaunchKernelGGL((gemm_plain_few_kernel<TO, MT_, 2, COLS_>), grid, block, 0, stream, (const bf16_t*)A, lda,    \
                         (const bf16_t*)W, ldw, (const bf16_t*)bias, (TO*)C, ldc, M, N, K);                            \
    else                                                                                                               \
      hipLaunchKernelGGL((gemm_plain_few_kernel<TO, MT_, 1, COLS_>), grid, block, 0, stream, (const bf16_t*)A, lda,    \
                         (const bf16_t*)W, ldw, (const bf16_t*)bias, (TO*)C, ldc, M, N, K);                            \
  } while (0)
  if (M <= 1) FEW(1, 1); else if (M <= 2) FEW(2, 1); else if (M <= 4) FEW(4, 2); else if (M <= 8) FEW(8, 4); else FEW(16, 4);
#undef FEW
}

template <typename TA, typename TW, typename TO>
static void launch_gemm_plain(const void* A, long lda, const void* W, long ldw, const void* bias, void* C, long ldc,
                              int M, int N, int K, hipStream_t stream) {
  dim3 grid((N + GP_TILE - 1) / GP_TILE, (M + GP_TILE - 1) / GP_TILE), block(256);
  hipLaunchKernelGGL((gemm_plain_kernel<TA, TW, TO>), grid, block, 0, stream, (const TA*)A, lda, (const TW*)W, ldw,
                     (const TW*)bias, (TO*)C, ldc, M, N, K);
}

// Supported (a, w, c) dtypes: (f32,f32,f32), (bf16,bf16,bf16), (bf16,bf16,f32), (f32,bf16,f32),
// (bf16,f32,bf16), (bf16,f32,f32). bias has the dtype of the weight or is null.
extern "C" int lmsf_gemm_plain(const void* A, int a_dtype, long lda, const void* W, int w_dtype, long ldw,
                               const void* bias, void* C, int c_dtype, long ldc, int M, int N, int K,
                               hipStream_t stream) {
  LMSF_CHECK(A && W && C, "gemm_plain: null pointer");
  LMSF_CHECK(M >= 0 && N > 0 && K > 0, "gemm_plain: bad sizes M=%d N=%d K=%d", M, N, K);
  LMSF_CHECK(lda >= K && ldw >= K && ldc >= N, "gemm_plain: leading dimensions too small");
  LMSF_CHECK((M + GP_TILE - 1) / GP_TILE <= 65535, "gemm_plain: M=%d too large", M);
  if (M == 0) return 0;
  if (M <= GP_FEW_ROWS && a_dtype == LMSF_BF16 && w_dtype == LMSF_BF16) {
    if (c_dtype == LMSF_BF16)
      launch_gemm_plain_few<bf16_t>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream);
    else
      launch_gemm_plain_few<float>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream);
    LMSF_LAUNCH_CHECK("gemm_plain");
    return 0;
  }
  const int key = a_dtype * 100 + w_dtype * 10 + c_dtype;
  switch (key) {
    case 0: launch_gemm_plain<float, float, float>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream); break;
    case 111: launch_gemm_plain<bf16_t, bf16_t, bf16_t>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream); break;
    case 110: launch_gemm_plain<bf16_t, bf16_t, float>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream); break;
    case 10: launch_gemm_plain<float, bf16_t, float>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream); break;
    case 101: launch_gemm_plain<bf16_t, float, bf16_t>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream); break;
    case 100: launch_gemm_plain<bf16_t, float, float>(A, lda, W, ldw, bias, C, ldc, M, N, K, stream); break;
    default:
      lmsf_set_error("gemm_plain: dtype combination a=%d w=%d c=%d not supported", a_dtype, w_dtype, c_dtype);
      return 1;
  }
  LMSF_LAUNCH_CHECK("gemm_plain");
  return 0;
}
