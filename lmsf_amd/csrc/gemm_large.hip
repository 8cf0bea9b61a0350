// Linear layer for many rows (portions of prompts): y[M, N] = x[M, K] W[N, K]^T (+ bias), bfloat16 in and out,
// float32 accumulation on the matrix cores; optionally with the gated activation of a feed-forward as epilogue
// (W = [gate rows; up rows], y = act(x Wg^T) * (x Wu^T)), or left as float32 partial sums over parts of K.
// The reference leaves these products to cuBLASLt (tops/src/cublas.rs:29-114,
// tops/csrc/tops/tensorrt_llm/common/cublasMMWrapper.cpp:182-210); so did this engine, through the BLAS library,
// which is weak between a hundred and a thousand rows, and no library product can carry these epilogues.
//
// A workgroup of four waves owns BM rows of x (128 or 256) and BN rows of W (128 or 256); the waves stand 2 x 2,
// each with BM / 2 rows of x and BN / 2 rows of W: (BN / 32) x (BM / 32) accumulator tiles of 16 x 16. Tiles of 64 k
// (two steps of the matrix instruction) travel from global memory straight into LDS (global_load_lds_dwordx4: lane i
// of a wave writes its 16 bytes at the wave's LDS base + 16 i), STAGES - 1 steps ahead of the one being multiplied.
// A tile row is 128 bytes; the 16-byte piece c of row r lies in slot (c + r) mod 8 of its row, so that the operand
// reads of a wave fall on distinct banks without padding. One barrier per step.
//
// What limits it: with wave tiles of 128 x 64 the operand reads ask LDS for 96 bytes a cycle at the full rate of the
// matrix cores and the arriving tiles write 47 more, against the 128 it has; the kernel reaches 0.9 to 1.0 PFLOP/s
// at 2,048 rows where the library's 256 x 256 tiles (wave tiles of 128 x 128) reach 1.2. Tried and measured, not
// kept: steps of 32 k with rows of 64 bytes and the next step's operands read under the multiplications (0.56);
// the same prefetch within steps of 64 k with the barrier in the middle of a step (0.74); tiles of 256 x 256 with two
// stages, which is all LDS holds of them (0.6, the compiler spills around 256 accumulators); the same tiles with the
// 32 x 32 x 16 instruction, wave tiles of 128 x 128 and no spills (0.85 to 1.0: two stages do not cover the way from
// memory); and those tiles again with four or five stages of 32 k (rows of 64 bytes), the accumulators in the 256
// accumulation registers and the next step's operands read from LDS under the current step's multiplications: 0.91
// PFLOP/s on gate_up at 2,048 rows against the library's 1.38 to 1.44, 0.55 on o (128 tiles: half the chip). The
// same loop without its transfers reaches 1.20, without transfers and barriers 1.31 (1.7 a compute unit on o), the
// same whether the transfers bring new data or the same lines again: what costs is the transfers' instructions
// themselves, six to eight each with their addresses, issued in a burst during which the matrix pipe runs dry, and
// the barrier of four waves every 1,024 cycles. The library stages through registers and places every instruction
// by hand; with 3.5 rounds of tiles over the chip (896 tiles) the ceiling here would be 1.2 to 1.25.
//
// Counters of this kernel and of the library's on the same product (2,048 x 14,336 x 4,096, the weight in cache):
// the same 1.47e7 matrix instructions; beside each of them 0.71 other vector instructions here and 0.06 there; the
// matrix pipe busy 42 percent of the time here, with 1.6 waves a SIMD that wait 39 percent of their time, and 62
// percent there, with one wave a SIMD. The library's loop is scheduled by hand around every wait; here two groups
// of waves cover some of each other's (they share the step's barrier, so they wait at the same moments).
//
// Workgroups that share rows of W run on the same XCD, one after the other in launch order, so that a panel of W
// comes from memory once and from that XCD's L2 afterwards: with 8 XCDs taking workgroups in turn, workgroup b
// runs on XCD b mod 8, and the tiles are numbered so that all row tiles of one panel of W differ by multiples of 8.
//
// v_mfma_f32_16x16x32_bf16: A = 16 rows of W, B = 16 rows of x, both with lane (r, g) = (l % 16, l / 16)
// holding row r, elements 8 g .. 8 g + 7 of a 32-wide step; D[n][m]: lane l holds row m = l % 16 of x and the
// four outputs n = (l / 16) * 4 .. + 3.
#include "common.h"

#include <type_traits>

#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // m0 is named as clobbered on purpose
__device__ __forceinline__ void large_global_to_lds_16(const void* src, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base_uniform)
               : "memory", "m0");
}
// The same for data that this launch reads once: marked non-temporal, it does not push out of the caches what is
// read again and again.
__device__ __forceinline__ void large_global_to_lds_16_once(const void* src, unsigned lds_base_uniform) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt" ::"v"(src), "s"(lds_base_uniform)
               : "memory", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ unsigned large_lds_address(const void* p) {
  return (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)p;
}

__device__ __forceinline__ float large_activation(float g, float u, int act) {
  // the two products are rounded to the storage type before the activation, as the unfused path stores them
  g = bf16_to_f32(f32_to_bf16(g));
  u = bf16_to_f32(f32_to_bf16(u));
  const float a = act == 1 ? g / (1.0f + expf(-g)) : 0.5f * g * (1.0f + erff(g * 0.70710678118654752f));
  return a * u;
}

#define LARGE_ROW 128         // bytes of a tile row: 64 k, two steps of the matrix instruction

// BM: rows of x per workgroup (128 or 256). BN: rows of W per workgroup (128 or 256; with ACT half of them gate rows
// and half the up rows of the same outputs). ACT: 0 none, 1 SiLU-gated, 2 GELU-gated. PARTIAL: float32 partial sums
// of this workgroup's part of K instead of the result (not with ACT).
template <int BM, int BN, int STAGES, int ACT, bool PARTIAL, int KG>
__global__ __launch_bounds__(256 * KG) void gemm_large_kernel(const bf16_t* __restrict__ x, long ldx,
                                                         const bf16_t* __restrict__ W, long ldw,
                                                         const bf16_t* __restrict__ bias, bf16_t* __restrict__ y,
                                                         long ldy, float* __restrict__ part, int M, int N, int K,
                                                         int n_split, int tiles_m, int tiles_n) {
  static_assert(!(ACT != 0 && PARTIAL), "the gated product is made in one piece");
  constexpr int MT = BM / 32;                      // accumulator tiles along x per wave
  constexpr int NT = BN / 32;                      // along W
  constexpr int W_BYTES = BN * LARGE_ROW, X_BYTES = BM * LARGE_ROW, STAGE = W_BYTES + X_BYTES;
  // KG groups of four waves: with two, both hold the same tile of outputs and each multiplies one 32-wide half of
  // every step, so that a SIMD has two waves and one's matrix instructions run while the other waits for its
  // operands; the groups' sums are added through LDS at the end.
  constexpr int W_LOADS = BN / 8 / (4 * KG), X_LOADS = BM / 8 / (4 * KG);   // transfers of 8 rows per wave and step
  static_assert(W_LOADS * 8 * 4 * KG == BN && X_LOADS * 8 * 4 * KG == BM, "the waves share the transfers evenly");
  constexpr int LPW = W_LOADS + X_LOADS;
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x, wave = tid >> 6, l = tid & 63, r = l & 15, g = l >> 4;
  const int kg = KG == 1 ? 0 : wave >> 2, w = wave & 3;
  const int wm = w & 1, wn = w >> 1;

  // which tile: all row tiles of one panel of W on one XCD, next to each other in time
  const int b = blockIdx.x;
  const int lane8 = b & 7, rest = b >> 3;
  const int mt_idx = rest % tiles_m, ngroup = rest / tiles_m;
  const int nt_idx = ngroup * 8 + lane8;
  if (nt_idx >= tiles_n) return;                   // the last group of eight may be short (uniform for the workgroup)
  constexpr int n_out = ACT ? BN / 2 : BN;         // outputs of a workgroup
  const int n0 = nt_idx * n_out, m0 = mt_idx * BM;
  const int split = blockIdx.y;
  const int chunks = K / 64;
  const int c_begin = (int)((long)split * chunks / n_split), c_end = (int)((long)(split + 1) * chunks / n_split);
  const int n_steps = c_end - c_begin;

  // LDS row j of the W tile (j = BN / 2 wn + 16 t + r) holds, without ACT, row n0 + j of W; with ACT the wave wn owns
  // the outputs n0 + BN / 4 wn .. + BN / 4 - 1: the first half of its tiles t are their gate rows, the second half
  // their up rows (N further down in W)
  auto w_row = [&](int j) {
    int n;
    if (ACT) {
      const int jn = j / (BN / 2), t = (j % (BN / 2)) >> 4, rr = j & 15;
      const int up = t >= NT / 2 ? 1 : 0;
      n = n0 + (BN / 4) * jn + 16 * (t - up * (NT / 2)) + rr;
      if (n > N - 1) n = N - 1;                    // rows beyond the matrix repeat the last row and are not stored
      n += up * N;
    } else {
      n = n0 + j;
      if (n > N - 1) n = N - 1;
    }
    return n;
  };

  // what this lane moves in every step: lane i of a transfer fills slot i % 8 of row i / 8 of eight rows
  const int trow = l >> 3, tslot = l & 7;
  const bf16_t* src[LPW];
  unsigned dst[LPW];                               // byte offset inside a stage; the same for all lanes of the wave
#pragma unroll
  for (int i = 0; i < W_LOADS; ++i) {
    const int j = (wave * W_LOADS + i) * 8 + trow, piece = (tslot - j) & 7;
    src[i] = W + (long)w_row(j) * ldw + piece * 8 + (long)c_begin * 64;
    dst[i] = (wave * W_LOADS + i) * 8 * LARGE_ROW;
  }
#pragma unroll
  for (int i = 0; i < X_LOADS; ++i) {
    const int j = (wave * X_LOADS + i) * 8 + trow, piece = (tslot - j) & 7;
    int m = m0 + j;
    if (m > M - 1) m = M - 1;
    src[W_LOADS + i] = x + (long)m * ldx + piece * 8 + (long)c_begin * 64;
    dst[W_LOADS + i] = W_BYTES + (wave * X_LOADS + i) * 8 * LARGE_ROW;
  }
  // where this lane reads its operands in a 16-row tile: row r, pieces 4 s + g of the two 32-wide halves of a step
  int foff[2];
#pragma unroll
  for (int s = 0; s < 2; ++s) foff[s] = r * LARGE_ROW + (((s * 4 + g) + r) & 7) * 16;
  const int foff_mine = foff[kg];                  // with two groups: the half of a step that this group multiplies

  f32x4_t acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const unsigned lds0 = large_lds_address(lds);
  // (with one tile of rows every row of W is read once by the whole launch; with several, the later tiles find W in
  // the die's L2, where it should stay)
  const bool w_once = tiles_m == 1;
  auto issue = [&](int step, int stage_byte) {
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const unsigned to = __builtin_amdgcn_readfirstlane(lds0 + stage_byte + dst[i]);
      if (i < W_LOADS && w_once)
        large_global_to_lds_16_once(src[i] + (long)step * 64, to);
      else
        large_global_to_lds_16(src[i] + (long)step * 64, to);
    }
  };
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < n_steps) issue(s, s * STAGE);

  const int a_base = (BN / 2 * wn) * LARGE_ROW, b_base = W_BYTES + (BM / 2 * wm) * LARGE_ROW;
  // One step; SI: which stage holds it (a constant, so that the operands' places in LDS are constants in the
  // instructions and cost no additions).
  auto step = [&](auto SI, int it) {
    constexpr int consume = decltype(SI)::value * STAGE;
    constexpr int produce = ((decltype(SI)::value + STAGES - 1) % STAGES) * STAGE;
    // step ``it`` has arrived when at most the transfers of the later steps are outstanding
    if (it + STAGES - 2 < n_steps)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LPW) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // everybody's part of step ``it`` is there, and everybody is done with step ``it - 1``
    if (it + STAGES - 1 < n_steps) issue(it + STAGES - 1, produce);
    const unsigned char* st = lds + consume;
#pragma unroll
    for (int s = 0; s < 2 / KG; ++s) {
      const int fo = KG == 2 ? foff_mine : foff[s];
      bf16x8_t a[NT], bb[MT];
#pragma unroll
      for (int t = 0; t < NT; ++t)
        a[t] = *reinterpret_cast<const bf16x8_t*>(st + a_base + t * 16 * LARGE_ROW + fo);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        bb[mt] = *reinterpret_cast<const bf16x8_t*>(st + b_base + mt * 16 * LARGE_ROW + fo);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int t = 0; t < NT; ++t) acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t], bb[mt], acc[t][mt], 0, 0, 0);
    }
  };
  static_assert(STAGES == 3 || STAGES == 4, "the loop is unrolled by three or four stages");
  for (int it = 0; it < n_steps; it += STAGES) {
    step(std::integral_constant<int, 0>(), it);
    if (it + 1 < n_steps) step(std::integral_constant<int, 1>(), it + 1);
    if (it + 2 < n_steps) step(std::integral_constant<int, 2>(), it + 2);
    if constexpr (STAGES == 4)
      if (it + 3 < n_steps) step(std::integral_constant<int, 3>(), it + 3);
  }

  if constexpr (KG == 2) {
    // the second group's sums go to the first through LDS (the stages are done with), lane to lane
    static_assert((size_t)4 * NT * MT * 1024 <= (size_t)STAGES * STAGE, "the exchange fits the stages");
    __syncthreads();
    f32x4_t* xch = reinterpret_cast<f32x4_t*>(lds) + (size_t)w * NT * MT * 64 + l;
    if (kg == 1) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) xch[(t * MT + mt) * 64] = acc[t][mt];
    }
    __syncthreads();
    if (kg == 1) return;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[t][mt] += xch[(t * MT + mt) * 64];
  }
  // this lane holds, for row m = m0 + BM / 2 wm + 16 mt + r of x, four neighbouring outputs per tile t
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = m0 + BM / 2 * wm + 16 * mt + r;
    if (m >= M) continue;
    if (ACT) {
#pragma unroll
      for (int t = 0; t < NT / 2; ++t) {
        const int n = n0 + (BN / 4) * wn + 16 * t + 4 * g;
        if (n >= N) continue;                      // N is a multiple of 4 (checked by the host)
        uint2 v;
        float o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float gg = acc[t][mt][i] + (bias ? bf16_to_f32(bias[n + i]) : 0.f);
          const float uu = acc[t + NT / 2][mt][i] + (bias ? bf16_to_f32(bias[N + n + i]) : 0.f);
          o[i] = large_activation(gg, uu, ACT);
        }
        v.x = pack2_bf16(o[0], o[1]);
        v.y = pack2_bf16(o[2], o[3]);
        *reinterpret_cast<uint2*>(y + (long)m * ldy + n) = v;
      }
    } else {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const int n = n0 + (BN / 2) * wn + 16 * t + 4 * g;
        if (n >= N) continue;
        if (PARTIAL) {
          *reinterpret_cast<f32x4_t*>(part + ((long)split * M + m) * N + n) = acc[t][mt];
        } else {
          uint2 v;
          float o[4];
#pragma unroll
          for (int i = 0; i < 4; ++i) o[i] = acc[t][mt][i] + (bias ? bf16_to_f32(bias[n + i]) : 0.f);
          v.x = pack2_bf16(o[0], o[1]);
          v.y = pack2_bf16(o[2], o[3]);
          *reinterpret_cast<uint2*>(y + (long)m * ldy + n) = v;
        }
      }
    }
  }
}

template <int BM, int BN, int STAGES, int ACT, bool PARTIAL, int KG = 1>
static int launch_large(hipStream_t stream, const bf16_t* x, long ldx, const bf16_t* W, long ldw, const bf16_t* bias,
                        bf16_t* y, long ldy, float* part, int M, int N, int K, int n_split) {
  const size_t smem = (size_t)STAGES * (BN + BM) * LARGE_ROW;
  auto kernel = gemm_large_kernel<BM, BN, STAGES, ACT, PARTIAL, KG>;
  static bool configured = false;   // per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("gemm_large: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  constexpr int n_out = ACT ? BN / 2 : BN;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + n_out - 1) / n_out;
  const int groups = (tiles_n + 7) / 8;
  hipLaunchKernelGGL(kernel, dim3(groups * tiles_m * 8, n_split), dim3(256 * KG), smem, stream, x, ldx, W, ldw, bias, y, ldy,
                     part, M, N, K, n_split, tiles_m, tiles_n);
  return 0;
}

// The tilings: rows of x, rows of W per workgroup; 3 to 5 are 0 to 2 with two groups of four waves (at 129 to 256
// rows 2 to 6 percent faster where K is long, the same elsewhere; at 2,048 rows 6 to 14 percent, which is still
// 0.75 to 1.0 PFLOP/s against the library's 1.05 to 1.2).
static const int kLargeTiles[6][2] = {{128, 128}, {256, 128}, {192, 128}, {128, 128}, {256, 128}, {192, 128}};

template <int ACT, bool PARTIAL>
static int launch_tiling(int tiling, hipStream_t stream, const bf16_t* x, long ldx, const bf16_t* W, long ldw,
                         const bf16_t* bias, bf16_t* y, long ldy, float* part, int M, int N, int K, int n_split) {
  switch (tiling) {
    case 0: return launch_large<128, 128, 4, ACT, PARTIAL>(stream, x, ldx, W, ldw, bias, y, ldy, part, M, N, K, n_split);
    case 1: return launch_large<256, 128, 3, ACT, PARTIAL>(stream, x, ldx, W, ldw, bias, y, ldy, part, M, N, K, n_split);
    case 2: return launch_large<192, 128, 4, ACT, PARTIAL>(stream, x, ldx, W, ldw, bias, y, ldy, part, M, N, K, n_split);
    // the same tiles with two groups of four waves
    case 3: return launch_large<128, 128, 4, ACT, PARTIAL, 2>(stream, x, ldx, W, ldw, bias, y, ldy, part, M, N, K, n_split);
    case 4: return launch_large<256, 128, 3, ACT, PARTIAL, 2>(stream, x, ldx, W, ldw, bias, y, ldy, part, M, N, K, n_split);
    default: return launch_large<192, 128, 4, ACT, PARTIAL, 2>(stream, x, ldx, W, ldw, bias, y, ldy, part, M, N, K, n_split);
  }
}

// Parts of K for these sizes (1: the result in one piece). Few columns leave too few workgroups to fill the chip;
// then K is split and the float32 partial sums are added up by gemm_mid's reduction kernel or by the kernel that
// takes the product next. The partial sums are written and read once, which costs what 2 * 4 * M * N bytes cost.
// Tiling and parts of K proposed for these sizes: plan = tiling * 16 + parts. Few columns leave too few workgroups to
// fill the chip; then K is split and the float32 partial sums are added up by gemm_mid's reduction kernel or by the
// kernel that takes the product next. The estimate: rounds of workgroups over the 256 compute units times what a
// workgroup's product takes at the rate its tiling sustains, plus what the partial sums' traffic costs.
extern "C" int lmsf_gemm_large_plan(int M, int N, int K, int act) {
  static const double rate[3] = {3.0e12, 3.7e12, 3.4e12};   // flops a second a compute unit sustains with each tiling (measured)
  const int chunks = K / 64;
  int best = 16 + 1;
  double best_cost = 1e30;
  for (int tiling = 0; tiling < 3; ++tiling) {
    const int bm = kLargeTiles[tiling][0], bn = kLargeTiles[tiling][1];
    if (tiling == 0 && M > 128) continue;      // (two tiles of 128 rows lose against one of 192 or 256)
    const int n_out = act ? bn / 2 : bn;
    const long tiles = (long)((M + bm - 1) / bm) * ((N + n_out - 1) / n_out);
    const double wg_seconds = 2.0 * bm * bn * (double)K / rate[tiling];
    for (int s = 1; s <= (act ? 1 : 8) && s * 8 <= chunks; ++s) {
      const long rounds = (tiles * s + 255) / 256;
      const double product = (double)rounds / s * wg_seconds;
      const double traffic = s > 1 ? (double)M * N * 8.0 * s / 4.0e12 + 4.0e-6 : 0.0;
      if (product + traffic < best_cost - 1e-9) {
        best_cost = product + traffic;
        best = (tiling + 3) * 16 + s;             // (the tilings with two groups of waves)
      }
    }
  }
  return best;
}

extern "C" long lmsf_gemm_large_scratch_floats(int M, int N, int n_split) {
  return n_split > 1 ? (long)n_split * M * N : 0;
}

// y [M, N] bfloat16 with row stride ldy. act 0: y = x W^T + bias, W [N, K]; act 1 / 2: W [2 N, K] = [gate; up], bias
// [2 N], y = act(gate) * up with SiLU / GELU. n_split > 1 (act 0 only): K in that many parts; ``scratch`` then holds
// lmsf_gemm_large_scratch_floats floats; with ``reduce`` 0 the sums stay there ([n_split, M, N], for a kernel that
// adds them up itself, bias not yet added) and y is not written. ``plan``: tiling * 16 + n_split, as
// lmsf_gemm_large_plan proposes. K a multiple of 64, N of 8, row strides of 8, 16-byte aligned bases.
extern "C" int lmsf_gemm_large(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
                               int M, int N, int K, int act, int plan, float* scratch, int reduce,
                               hipStream_t stream);
extern "C" int lmsf_gemm_mid_reduce(const float* scratch, const void* bias, void* y, int out_dtype, long ldy, int M,
                                    int N, int n_split, hipStream_t stream);

extern "C" int lmsf_gemm_large(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
                               int M, int N, int K, int act, int plan, float* scratch, int reduce,
                               hipStream_t stream) {
  const int tiling = plan / 16, n_split = plan % 16;
  LMSF_CHECK(tiling >= 0 && tiling < 6, "gemm_large: unknown tiling %d", tiling);
  LMSF_CHECK(x && W && (y || (n_split > 1 && !reduce)), "gemm_large: null pointer");
  LMSF_CHECK(M > 0 && N > 0 && K > 0, "gemm_large: bad sizes M=%d N=%d K=%d", M, N, K);
  LMSF_CHECK(K % 64 == 0 && N % 8 == 0, "gemm_large: K must be a multiple of 64 and N of 8, got K=%d N=%d", K, N);
  LMSF_CHECK(ldx >= K && ldw >= K && ldx % 8 == 0 && ldw % 8 == 0 && (!y || (ldy >= N && ldy % 4 == 0)),
             "gemm_large: bad row strides");
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W) && (!y || (((uintptr_t)y) & 7u) == 0), "gemm_large: operands must be 16-byte aligned");
  LMSF_CHECK(act >= 0 && act <= 2, "gemm_large: unknown activation %d", act);
  LMSF_CHECK(n_split >= 1 && n_split <= K / 64 && (n_split == 1 || act == 0), "gemm_large: bad split %d", n_split);
  LMSF_CHECK(n_split == 1 || (scratch && lmsf_aligned16(scratch)), "gemm_large: a split product needs scratch");
  const bf16_t* xp = (const bf16_t*)x;
  const bf16_t* wp = (const bf16_t*)W;
  const bf16_t* bp = (const bf16_t*)bias;
  bf16_t* yp = (bf16_t*)y;
  int rc;
  if (n_split > 1)
    rc = launch_tiling<0, true>(tiling, stream, xp, ldx, wp, ldw, nullptr, nullptr, 0, scratch, M, N, K, n_split);
  else if (act == 0)
    rc = launch_tiling<0, false>(tiling, stream, xp, ldx, wp, ldw, bp, yp, ldy, nullptr, M, N, K, 1);
  else if (act == 1)
    rc = launch_tiling<1, false>(tiling, stream, xp, ldx, wp, ldw, bp, yp, ldy, nullptr, M, N, K, 1);
  else
    rc = launch_tiling<2, false>(tiling, stream, xp, ldx, wp, ldw, bp, yp, ldy, nullptr, M, N, K, 1);
  if (rc != 0) return rc;
  LMSF_LAUNCH_CHECK("gemm_large");
  if (n_split > 1 && reduce) return lmsf_gemm_mid_reduce(scratch, bias, y, LMSF_BF16, ldy, M, N, n_split, stream);
  return 0;
}
