// Linear layer for 17 to 128 rows (decoding at larger batches): y[M, N] = x[M, K] W[N, K]^T (+ bias),
// bfloat16 inputs, float32 accumulation on the matrix cores, bfloat16 or float32 output; up to 64 rows
// optionally with the gated activation of a feed-forward as epilogue (beyond that its stages do not fit LDS).
//
// The product is still a stream of the weight matrix, but with this many rows the activations are no
// longer negligible: a workgroup that owns 16 rows of W reads four times as many bytes of x as of W. Here
// a workgroup owns 64 rows of W (16 per wave) and all rows of x, so x is read once per 64 rows of W; where
// that leaves too few workgroups to fill the chip (N = 4096: 64 of them), K is split over several
// workgroups, which write float32 partial sums that a second small kernel adds in a fixed order (and
// applies bias and activation to). The reference leaves these products to cuBLASLt
// (tops/src/cublas.rs:29-114).
//
// Tiles of 64 k travel from global memory straight into LDS (global_load_lds_dwordx4: lane i of a wave
// writes its 16 bytes at the wave's LDS base + 16 i), four steps ahead of the one being multiplied (three in the
// form whose waves own two tiles of each projection); each wave moves its own rows of W and a quarter of x. A tile is 16 rows of 128 bytes; the 16-byte piece c of
// row r lies in slot (c + r) mod 8 of its row, which keeps the operand reads of a wave on distinct
// banks without padding (the transfer cannot pad). One barrier per step.
//
// v_mfma_f32_16x16x32_bf16: A = 16 rows of W, B = 16 rows of x, both with lane (r, g) = (l % 16, l / 16)
// holding row r, elements 8 g .. 8 g + 7 of a 32-wide step; D[n][m]: lane l holds token m = l % 16 and the
// four outputs n = (l / 16) * 4 .. + 3.
#include "common.h"

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // m0 is named as clobbered on purpose
// The transfer is inline assembly: through the compiler's builtin every LDS read that follows would first
// wait for all transfers in flight. The waits are explicit (s_waitcnt vmcnt before each step's barrier).
__device__ __forceinline__ void mid_global_to_lds_16(const void* src, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base_uniform)
               : "memory", "m0");
}
// The same for data that is read once (the weights): marked non-temporal, it does not push out of the caches what
// is read again and again (x).
__device__ __forceinline__ void mid_global_to_lds_16_once(const void* src, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(src), "s"(lds_base_uniform)
               : "memory", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ unsigned mid_lds_address(const void* p) {
  return (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)p;
}

__device__ __forceinline__ float mid_activation(float g, float u, int act) {
  // the two products are rounded to the storage type before the activation, as the unfused path stores them
  g = bf16_to_f32(f32_to_bf16(g));
  u = bf16_to_f32(f32_to_bf16(u));
  const float a = act == 1 ? g / (1.0f + expf(-g)) : 0.5f * g * (1.0f + erff(g * 0.70710678118654752f));
  return a * u;
}

// four consecutive outputs of a row
__device__ __forceinline__ void mid_store4(bf16_t* p, const float* o) {
  uint2 v;
  v.x = pack2_bf16(o[0], o[1]);
  v.y = pack2_bf16(o[2], o[3]);
  *reinterpret_cast<uint2*>(p) = v;
}
__device__ __forceinline__ void mid_store4(float* p, const float* o) {
  *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
}

#define MID_STAGES_OF(TW) ((TW) == 2 ? 4 : 5)   // stages of the ring: what fits into the 160 KB of LDS
#define MID_TILE 2048

// MT: tiles of 16 rows of x (2, 4, 6 or 8). ACT: 0 none, 1 silu-gated, 2 gelu-gated (W = [gate rows; up rows], N
// outputs). PARTIAL: write float32 partial sums of this workgroup's part of K instead of the result. TW: tiles of 16
// outputs a wave owns (of each projection), so 64 TW outputs a workgroup.
// (A form of the gated product with 32 outputs a workgroup, waves 0 and 1 on the gate rows and 2 and 3 on the up rows
// of the same outputs, twice as many workgroups, two to a compute unit, was ahead at 17 to 48 rows while the
// weights' rows lay back to back and were loaded like anything else: 4.7 -> 5.0 TB/s. With the rows apart and the
// transfers non-temporal it is behind at every number of rows, 42.3 against 40.5 us at 17 rows and 50.1 against 42.7
// at 48, and is gone.)
// What the gated product takes when it stands after a norm whose row factor it applies itself (up to 16 rows): x is
// then bf16(stream * w), sumsq [tiles][16] the sums of stream^2 over 16 columns per row (rows >= M: 0), and the rows
// of both products are multiplied by rsqrt(sum / H + eps) before bias and activation, as the few-rows product does
// (gemm_skinny.hip). sumsq null: no factor.
struct MidRowScale {
  const float* sumsq;
  int tiles;
  float eps;
  int H;
};
#define MID_SCALE_HELD 32   // sums a thread holds: thread t has row t % 16 of the tiles t / 16, t / 16 + 16, ...

template <int MT, int ACT, bool PARTIAL, typename TOut, int TW>
__global__ __launch_bounds__(256) void gemm_mid_kernel(const bf16_t* __restrict__ x, long ldx,
                                                       const bf16_t* __restrict__ W, long ldw,
                                                       const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                       long ldy, float* __restrict__ part, int M, int N, int K,
                                                       int n_split, MidRowScale rs) {
  constexpr int WP = ACT ? 2 : 1;      // projections: gate and up, or the only one
  constexpr int WT = WP * TW;          // tiles of 16 rows of W per wave: TW of each projection
  constexpr int STAGES = MID_STAGES_OF(TW);
  constexpr int STAGE = (4 * WT + MT) * MID_TILE;
  constexpr int XL = MT / 2;           // halves of x tiles this wave moves per step (2 MT halves over 4 waves)
  constexpr int LPW = 2 * WT + XL;     // transfers per wave and step
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
  const int n0 = blockIdx.x * (64 * TW), split = blockIdx.y;
  const int chunks = K / 64;
  const int c_begin = (int)((long)split * chunks / n_split), c_end = (int)((long)(split + 1) * chunks / n_split);
  const int n_steps = c_end - c_begin;

  // what this lane moves in every step: lane i of a transfer fills slot i % 8 of row i / 8 of half a tile
  const int trow = l >> 3, tslot = l & 7;
  const bf16_t* src[LPW];
  unsigned dst[LPW];                   // byte offset inside a stage; the same for all lanes of the wave
#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int row = 8 * h + trow, piece = (tslot - row) & 7;
      // tile t of this wave: projection t / TW (0 the gate's rows or the only ones, 1 the up projection's), the
      // wave's 16 outputs number t % TW
      int n = n0 + 16 * (w * TW + t % TW) + row;
      if (n > N - 1) n = N - 1;        // rows beyond the matrix repeat the last row and are not stored
      src[t * 2 + h] = W + (long)(n + (t / TW) * N) * ldw + piece * 8 + (long)c_begin * 64;
      dst[t * 2 + h] = (w * WT + t) * MID_TILE + h * 1024;
    }
#pragma unroll
  for (int j = 0; j < XL; ++j) {
    const int qh = w * XL + j, tile = qh >> 1, h = qh & 1;
    const int row = 8 * h + trow, piece = (tslot - row) & 7;
    int m = tile * 16 + row;
    if (m > M - 1) m = M - 1;
    src[2 * WT + j] = x + (long)m * ldx + piece * 8 + (long)c_begin * 64;
    dst[2 * WT + j] = (4 * WT + tile) * MID_TILE + h * 1024;
  }
  // where this lane reads its operands in a tile: row r, pieces 4 s + g of the two 32-wide steps
  int foff[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) foff[s] = r * 128 + (((s * 4 + g) + r) & 7) * 16;

  f32x4_t acc[WT][MT];
#pragma unroll
  for (int t = 0; t < WT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  // The row factor's sums are asked for before the first weights (loads come back in the order they were asked for)
  // and added up after the last step, when nothing waits for them any more.
  constexpr bool MAY_SCALE = ACT != 0 && !PARTIAL;
  float held[MID_SCALE_HELD];
  if (MAY_SCALE && rs.sumsq) {
#pragma unroll
    for (int k = 0; k < MID_SCALE_HELD; ++k) {
      const int t = (tid >> 4) + 16 * k;
      held[k] = t < rs.tiles ? rs.sumsq[t * 16 + (tid & 15)] : 0.f;
    }
  }
  const unsigned lds0 = mid_lds_address(lds);
  auto issue = [&](int step, int stage_byte) {
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const unsigned to = __builtin_amdgcn_readfirstlane(lds0 + stage_byte + dst[i]);
      if (i < 2 * WT)
        mid_global_to_lds_16_once(src[i] + (long)step * 64, to);
      else
        mid_global_to_lds_16(src[i] + (long)step * 64, to);
    }
  };
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < n_steps) issue(s, s * STAGE);

  int consume = 0, produce = (STAGES - 1) * STAGE;
  for (int it = 0; it < n_steps; ++it) {
    // step ``it`` has arrived when at most the transfers of the later steps are outstanding
    if (it + STAGES - 2 < n_steps)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LPW) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // everybody's part of step ``it`` is there, and everybody is done with step ``it - 1``
    if (it + STAGES - 1 < n_steps) issue(it + STAGES - 1, produce);
    produce = produce + STAGE == STAGES * STAGE ? 0 : produce + STAGE;
    const unsigned char* st = lds + consume;
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      bf16x8_t a[WT], b[MT];
#pragma unroll
      for (int t = 0; t < WT; ++t) a[t] = *reinterpret_cast<const bf16x8_t*>(st + (w * WT + t) * MID_TILE + foff[s]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[mt] = *reinterpret_cast<const bf16x8_t*>(st + (4 * WT + mt) * MID_TILE + foff[s]);
#pragma unroll
      for (int t = 0; t < WT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t], b[mt], acc[t][mt], 0, 0, 0);
    }
    consume = consume + STAGE == STAGES * STAGE ? 0 : consume + STAGE;
  }

  float inv = 1.f;                     // the factor of row r (rows of the first tile only: up to 16 rows)
  if (MAY_SCALE && rs.sumsq) {
    float sum = 0.f;
#pragma unroll
    for (int k = 0; k < MID_SCALE_HELD; ++k) sum += held[k];
    __syncthreads();                   // everybody is done with the last stage
    float* red = reinterpret_cast<float*>(lds);
    red[tid] = sum;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int k = 0; k < 16; ++k) total += red[k * 16 + r];   // in a fixed order
    inv = rsqrtf(total / (float)rs.H + rs.eps);
  }
  // this lane holds, for token m = mt * 16 + r, the outputs n = n0 + 16 (w TW + tw) + 4 g .. + 3
#pragma unroll
  for (int tw = 0; tw < TW; ++tw) {
    const int n = n0 + 16 * (w * TW + tw) + 4 * g;
    if (n >= N) continue;              // N is a multiple of 4 where it is not a multiple of 64 (checked by the host)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      if (m >= M) continue;
      if (PARTIAL) {
        // partial sums: [split][projection (gate, up)][M][N]
#pragma unroll
        for (int p = 0; p < WP; ++p)
          *reinterpret_cast<f32x4_t*>(part + (((long)split * WP + p) * M + m) * N + n) = acc[p * TW + tw][mt];
      } else {
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (ACT == 0) {
            o[i] = acc[tw][mt][i] + (bias ? bf16_to_f32(bias[n + i]) : 0.f);
          } else {
            const float gg = acc[tw][mt][i] * inv + (bias ? bf16_to_f32(bias[n + i]) : 0.f);
            const float uu = acc[(WP - 1) * TW + tw][mt][i] * inv + (bias ? bf16_to_f32(bias[N + n + i]) : 0.f);
            o[i] = mid_activation(gg, uu, ACT);
          }
        }
        mid_store4(y + (long)m * ldy + n, o);
      }
    }
  }
}

// y[m][n] = (act of) the sum over the splits of the partial sums, in the order of the splits, plus bias.
template <typename TOut>
__global__ __launch_bounds__(256) void gemm_mid_reduce_kernel(const float* __restrict__ part,
                                                              const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                              long ldy, int M, int N, int n_split, int act) {
  const long idx = ((long)blockIdx.x * 256 + threadIdx.x) * 4;   // over M * N, four outputs of a row at a time
  if (idx >= (long)M * N) return;
  const int m = (int)(idx / N), n = (int)(idx - (long)m * N);
  const int wt = act ? 2 : 1;
  f32x4_t sg = (f32x4_t){0.f, 0.f, 0.f, 0.f}, su = sg;
  for (int s = 0; s < n_split; ++s) {
    sg += *reinterpret_cast<const f32x4_t*>(part + (((long)s * wt) * M + m) * N + n);
    if (act) su += *reinterpret_cast<const f32x4_t*>(part + (((long)s * wt + 1) * M + m) * N + n);
  }
  float o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float gg = sg[i] + (bias ? bf16_to_f32(bias[n + i]) : 0.f);
    if (act) {
      const float uu = su[i] + (bias ? bf16_to_f32(bias[N + n + i]) : 0.f);
      o[i] = mid_activation(gg, uu, act);
    } else {
      o[i] = gg;
    }
  }
  mid_store4(y + (long)m * ldy + n, o);
}

template <int MT, int ACT, bool PARTIAL, typename TOut, int TW = 1>
static int launch_mid(dim3 grid, hipStream_t stream, const bf16_t* x, long ldx, const bf16_t* W, long ldw,
                      const bf16_t* bias, TOut* y, long ldy, float* part, int M, int N, int K, int n_split,
                      MidRowScale rs) {
  static_assert(TW == 1 || TW == 2, "one or two tiles of each projection per wave");
  constexpr int WT = (ACT ? 2 : 1) * TW;
  const size_t smem = (size_t)MID_STAGES_OF(TW) * (4 * WT + MT) * MID_TILE;
  auto kernel = gemm_mid_kernel<MT, ACT, PARTIAL, TOut, TW>;
  static bool configured = false;   // per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("gemm_mid: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(256), smem, stream, x, ldx, W, ldw, bias, y, ldy, part, M, N, K, n_split, rs);
  return 0;
}

// Splits of K proposed for these sizes (1: no partial sums, no second kernel). The time of the product is
// that of the compute unit with the most workgroups, so the number of workgroups should fill the last round
// over the 256 compute units; against that stand the partial sums, which are written and read once. The
// proposal minimises bytes / (share of the last round that is filled) + bytes of the partial sums.
extern "C" int lmsf_gemm_mid_splits(int M, int N, int K, int act) {
  const int wt = act ? 2 : 1;
  const long blocks = (N + 63) / 64, chunks = K / 64;
  const double w_bytes = 2.0 * wt * (double)N * K;
  int best = 1;
  double best_cost = 0;
  for (int s = 1; s <= 8; ++s) {
    if (s > 1 && chunks / s < 8) break;       // at least 8 steps per workgroup
    const long wg = blocks * s, rounds = (wg + 255) / 256;
    const double fill = (double)wg / (256.0 * rounds);
    // partial sums are written and read again, and a byte of them costs about three of the weights' (measured: QKV of
    // 6,144 x 4,096 at 64 rows 18.5 us in 2 parts against 20.8 in 5, of 12,288 x 4,096 26.3 in one piece against 31.8
    // in 4; o and down of 4,096 columns stay at 4 parts); the gated form also needs a kernel of its own to add them
    // up (about 5 us, the time of 40 MB), the plain form's are added up by the kernel that takes the product
    const double cost = w_bytes / fill + (s > 1 ? 6.0 * s * wt * (double)M * N * 4 + (act ? 40e6 : 0.0) : 0.0);
    if (s == 1 || cost < best_cost) {
      best = s;
      best_cost = cost;
    }
  }
  return best;
}
extern "C" long lmsf_gemm_mid_scratch_floats(int M, int N, int n_split, int act) {
  return n_split > 1 ? (long)n_split * (act ? 2 : 1) * M * N : 0;
}

// x [M, K] bfloat16 (row stride ldx), W [N, K] (act 0) or [2 N, K] (act 1 silu, 2 gelu: gate rows first),
// bias [N] or [2 N] or null, y [M, N] of out_dtype (float32 only without activation). Needs 1 <= M <= 128 (64 with an activation), K a multiple of 64, N a multiple of 4,
// 16-byte aligned x and W, row strides of x and W that are multiples of 8 and of y of 4; anything else is
// refused. n_split: parts of K that go to different workgroups (lmsf_gemm_mid_splits proposes a number);
// scratch: lmsf_gemm_mid_scratch_floats floats (may be null when that is 0).
static int mid_check(const void* x, long ldx, const void* W, long ldw, int M, int N, int K, int n_split,
                     const float* scratch, int act = 0) {
  LMSF_CHECK(x && W, "gemm_mid: null pointer");
  LMSF_CHECK(M >= 0 && M <= (act ? 64 : 128), "gemm_mid: M=%d outside [0, %d]", M, act ? 64 : 128);
  LMSF_CHECK(N > 0 && N % 4 == 0 && K > 0 && K % 64 == 0, "gemm_mid: N=%d must be a multiple of 4 and K=%d of 64", N, K);
  LMSF_CHECK(ldx >= K && ldw >= K && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_mid: row strides of x and W must cover the rows and be multiples of 8");
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W), "gemm_mid: operands must be 16-byte aligned");
  LMSF_CHECK(n_split >= 1 && n_split <= 64 && n_split <= K / 64, "gemm_mid: %d splits of K=%d", n_split, K);
  LMSF_CHECK(n_split == 1 || (scratch != nullptr && lmsf_aligned16(scratch)),
             "gemm_mid: %d splits need 16-byte aligned scratch", n_split);
  return 0;
}

// The product's kernel: the result into y (n_split == 1) or partial sums into scratch.
static int mid_product(const bf16_t* xb, long ldx, const bf16_t* Wb, long ldw, const bf16_t* bb, void* y, int out_dtype,
                       long ldy, int M, int N, int K, int act, int n_split, float* scratch, hipStream_t stream,
                       MidRowScale rs = MidRowScale{nullptr, 0, 0.f, 0}) {
  dim3 grid((N + 63) / 64, n_split);
  int rc = 0;
#define MID(MT_, ACT_, T_)                                                                                          \
  rc = n_split > 1                                                                                                  \
           ? launch_mid<MT_, ACT_, true, T_>(grid, stream, xb, ldx, Wb, ldw, bb, (T_*)y, ldy, scratch, M, N, K, n_split, rs) \
           : launch_mid<MT_, ACT_, false, T_>(grid, stream, xb, ldx, Wb, ldw, bb, (T_*)y, ldy, scratch, M, N, K, n_split, rs)
  if (out_dtype == LMSF_F32) {
    if (M <= 32) MID(2, 0, float); else if (M <= 64) MID(4, 0, float); else if (M <= 96) MID(6, 0, float); else MID(8, 0, float);
  } else if (M <= 32) {
    if (act == 0) MID(2, 0, bf16_t); else if (act == 1) MID(2, 1, bf16_t); else MID(2, 2, bf16_t);
  } else if (M <= 64) {
    if (act == 0) MID(4, 0, bf16_t); else if (act == 1) MID(4, 1, bf16_t); else MID(4, 2, bf16_t);
  } else if (M <= 96) {
    MID(6, 0, bf16_t);
  } else {
    MID(8, 0, bf16_t);
  }
#undef MID
  if (rc) return rc;
  LMSF_LAUNCH_CHECK("gemm_mid");
  return 0;
}

static int mid_reduce(const float* scratch, const bf16_t* bb, void* y, int out_dtype, long ldy, int M, int N,
                      int act, int n_split, hipStream_t stream) {
  const long quads = ((long)M * N + 3) / 4;
  const dim3 rgrid((unsigned)((quads + 255) / 256));
  if (out_dtype == LMSF_F32)
    hipLaunchKernelGGL(gemm_mid_reduce_kernel<float>, rgrid, dim3(256), 0, stream, scratch, bb, (float*)y, ldy, M, N,
                       n_split, act);
  else
    hipLaunchKernelGGL(gemm_mid_reduce_kernel<bf16_t>, rgrid, dim3(256), 0, stream, scratch, bb, (bf16_t*)y, ldy, M,
                       N, n_split, act);
  LMSF_LAUNCH_CHECK("gemm_mid_reduce");
  return 0;
}

extern "C" int lmsf_gemm_mid(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y,
                             int out_dtype, long ldy, int M, int N, int K, int act, int n_split, float* scratch,
                             hipStream_t stream) {
  LMSF_CHECK(act >= 0 && act <= 2, "gemm_mid: unknown activation %d", act);
  if (int rc = mid_check(x, ldx, W, ldw, M, N, K, M == 0 ? 1 : n_split, scratch, act)) return rc;
  LMSF_CHECK(y != nullptr && lmsf_aligned16(y) && ldy >= N && ldy % 4 == 0,
             "gemm_mid: y must be 16-byte aligned with a row stride that covers N and is a multiple of 4");
  LMSF_CHECK(out_dtype == LMSF_BF16 || (out_dtype == LMSF_F32 && act == 0),
             "gemm_mid: output is bfloat16, or float32 without activation");
  if (M == 0) return 0;
  const bf16_t *xb = (const bf16_t*)x, *Wb = (const bf16_t*)W, *bb = (const bf16_t*)bias;
  if (int rc = mid_product(xb, ldx, Wb, ldw, bb, y, out_dtype, ldy, M, N, K, act, n_split, scratch, stream)) return rc;
  if (n_split > 1) return mid_reduce(scratch, bb, y, out_dtype, ldy, M, N, act, n_split, stream);
  return 0;
}

// The two halves of a product without activation whose K is split (n_split >= 2): the partial sums alone,
// scratch[(s * M + m) * N + n], for a kernel that reduces them while it loads its operand (LmsfPartialSum);
// and the reduction alone, y = sum over s + bias, for a caller that turns out to need the plain result.
// Whether the gated product after a norm should run here rather than in the few-rows kernel: when its workgroups (64
// outputs each) fit on the chip at once, so that every compute unit streams one share of the weights from the first
// step to the last (gate_up of 28,672 x 4,096 at 8 rows: 39.5 us against 43.9, at 16 rows 39.4 against 47.3; of
// 57,344 x 8,192, 448 workgroups: 158.7 against 144.8), and when they do not leave too many compute units without
// one (22,016 x 4,096, 172 workgroups on 256 units: 39.0 against 33.7 us at 8 rows, 35.2 against 38.5 at 16): from
// 0.8 of the units on with up to 8 rows, from 0.58 on beyond. Where workgroups of 64 outputs are too many, those of
// 128 take over beyond 8 rows (57,344 x 8,192 in 224 workgroups: a decode step of 80 such layers at 16 rows 25.6 ms
// against 26.7, about 14 us a layer; at 4 and 8 rows 23.7 against 23.6 and 24.0 against 24.0, left to the few-rows
// kernel).
// Outputs a workgroup of the gated product after a norm takes: 64, or 128 (each wave two tiles of either projection,
// a ring of 4 stages) where workgroups of 64 would be more than the chip holds at once.
static int mid_scaled_outputs(int N) { return (N + 63) / 64 <= lmsf_compute_units() ? 64 : 128; }
extern "C" int lmsf_gemm_mid_scaled_fits(int M, int N, int K, int in_tiles) {
  const long per = mid_scaled_outputs(N), blocks = (N + per - 1) / per, cus = lmsf_compute_units();
  return M >= 1 && M <= 16 && N > 0 && N % 4 == 0 && K > 0 && K % 64 == 0 && in_tiles == (K + 15) / 16 &&
         in_tiles <= 16 * MID_SCALE_HELD && blocks <= cus && blocks * 100 >= cus * (M <= 8 ? 80 : 58) &&
         (per == 64 || M > 8);
}

// The gated product (act 1 silu, 2 gelu) after a norm, with up to 16 rows: x [M, K] is bf16(stream * w) and sumsq
// [in_tiles][16] its sums of squares, as the few-rows product before the norm writes them (lmsf_gemm_skinny_add_norm);
// the rows of both products are multiplied by rsqrt(sum / K + eps) before bias and activation. K = 16 in_tiles at
// most 8,192 (each thread holds 32 of the sums). In one piece, no split of K.
extern "C" int lmsf_gemm_mid_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
                                    int M, int N, int K, int act, const float* sumsq, int in_tiles, float eps,
                                    hipStream_t stream) {
  LMSF_CHECK(act == 1 || act == 2, "gemm_mid_scaled: activation %d (1 silu, 2 gelu)", act);
  LMSF_CHECK(M >= 0 && M <= 16, "gemm_mid_scaled: M=%d outside [0, 16]", M);
  if (int rc = mid_check(x, ldx, W, ldw, M, N, K, 1, nullptr, act)) return rc;
  LMSF_CHECK(y != nullptr && lmsf_aligned16(y) && ldy >= N && ldy % 4 == 0,
             "gemm_mid_scaled: y must be 16-byte aligned with a row stride that covers N and is a multiple of 4");
  LMSF_CHECK(sumsq != nullptr && in_tiles > 0 && in_tiles == (K + 15) / 16 && in_tiles <= 16 * MID_SCALE_HELD,
             "gemm_mid_scaled: %d sums of squares must cover %d columns (at most %d)", in_tiles, K, 16 * 16 * MID_SCALE_HELD);
  if (M == 0) return 0;
  const MidRowScale rs = {sumsq, in_tiles, eps, K};
  if (mid_scaled_outputs(N) == 128) {
    const dim3 grid((N + 127) / 128, 1);
    const int rc = act == 1 ? launch_mid<2, 1, false, bf16_t, 2>(grid, stream, (const bf16_t*)x, ldx, (const bf16_t*)W, ldw,
                                                                 (const bf16_t*)bias, (bf16_t*)y, ldy, nullptr, M, N, K, 1, rs)
                            : launch_mid<2, 2, false, bf16_t, 2>(grid, stream, (const bf16_t*)x, ldx, (const bf16_t*)W, ldw,
                                                                 (const bf16_t*)bias, (bf16_t*)y, ldy, nullptr, M, N, K, 1, rs);
    if (rc) return rc;
    LMSF_LAUNCH_CHECK("gemm_mid_scaled");
    return 0;
  }
  return mid_product((const bf16_t*)x, ldx, (const bf16_t*)W, ldw, (const bf16_t*)bias, y, LMSF_BF16, ldy, M, N, K, act, 1,
                     nullptr, stream, rs);
}

extern "C" int lmsf_gemm_mid_partial(const void* x, long ldx, const void* W, long ldw, int M, int N, int K,
                                     int n_split, float* scratch, hipStream_t stream) {
  if (int rc = mid_check(x, ldx, W, ldw, M, N, K, n_split, scratch)) return rc;
  LMSF_CHECK(n_split >= 2, "gemm_mid_partial: needs at least two splits, got %d", n_split);
  if (M == 0) return 0;
  return mid_product((const bf16_t*)x, ldx, (const bf16_t*)W, ldw, nullptr, nullptr, LMSF_BF16, N, M, N, K, 0, n_split,
                     scratch, stream);
}
extern "C" int lmsf_gemm_mid_reduce(const float* scratch, const void* bias, void* y, int out_dtype, long ldy, int M,
                                    int N, int n_split, hipStream_t stream) {
  LMSF_CHECK(scratch && y && lmsf_aligned16(scratch) && lmsf_aligned16(y), "gemm_mid_reduce: null or unaligned pointer");
  LMSF_CHECK(M >= 0 && N > 0 && N % 4 == 0 && ldy >= N && ldy % 4 == 0 && n_split >= 1,
             "gemm_mid_reduce: bad sizes M=%d N=%d ldy=%ld splits=%d", M, N, ldy, n_split);
  LMSF_CHECK(out_dtype == LMSF_BF16 || out_dtype == LMSF_F32, "gemm_mid_reduce: unknown dtype code %d", out_dtype);
  if (M == 0) return 0;
  return mid_reduce(scratch, (const bf16_t*)bias, y, out_dtype, ldy, M, N, 0, n_split, stream);
}
