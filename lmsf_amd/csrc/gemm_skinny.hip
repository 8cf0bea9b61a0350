// Linear layer for few rows (decoding): y[M, N] = x[M, K] W[N, K]^T (+ bias), M <= 64, bfloat16
// inputs, float32 accumulation on the matrix cores, bfloat16 or float32 output.
//
// With so few rows the product is a stream of the weight matrix: every weight is read once from
// HBM and used M times, so the kernel is built around the memory system, not the arithmetic.
// The reference leaves these products to cuBLASLt with an offline-tuned algorithm per shape
// (tops/src/cublas.rs:29-114, tops/csrc/tops/tensorrt_llm/c_api/gemm.cc:43-150).
//
// Decomposition. One workgroup owns 16 rows of W (16 outputs per token) over the whole K. Its NW
// waves split K in chunks of KC elements, wave w taking chunks w, w + NW, ...: at any moment the
// workgroup reads NW * KC contiguous elements of each of its rows. Partial sums of the waves are
// added in a fixed order through LDS, so the result does not depend on timing.
//
// Data path of one chunk in one wave. W tile (16 rows x KC) and x tile (16 tokens x KC, per token
// tile) are fetched with 16-byte loads in which consecutive lanes read consecutive addresses of one
// row (KC/8 lanes per row), so every load instruction covers whole cache lines. The matrix-core
// operand layout wants lane (r, g) to hold row r, elements g*8..g*8+7 of a 32-wide step; the tiles go
// through a wave-private LDS area (row stride padded by 16 bytes: conflict-free for both the write
// and the read pattern) to change layout. The loads of the next chunk are issued before the current
// chunk's LDS traffic and MFMAs, so a chunk per wave is always in flight.
//
// Gated form (GATED): W holds 2 N rows, the gate's N rows first and then the up projection's N rows (the
// fused gate_up weight of a gated feed-forward). A workgroup then owns rows n0 .. n0 + 15 of both halves and
// writes y[m][n] = act(g) * u with g and u the two products: the activation kernel and its traffic are gone
// (the reference runs silu_and_mul as a kernel of its own, vllm/kernels/activation_kernels.cu:31-42).
//
// Rotary form (ACT == 3): the product is the fused QKV projection of an attention layer with NeoX rotary
// embedding over the whole head. A workgroup owns rows i .. i + 15 and i + d/2 .. i + d/2 + 15 of one head,
// that is, both members of 16 rotation pairs, and its epilogue rotates q and k by the token's position,
// stores q (and k, v) in the output and k, v in the token's slot of the paged cache: the kernel that
// would do this afterwards (vllm/kernels/pos_encoding_kernels.cu:38-77 and cache_kernels.cu:190-232 in the
// reference) and its launch are gone from a decode step.
//
// Norm around the products (ACT == 4 and SCALED, up to 16 rows). An RMSNorm between two products is
// x' = r * inv(r) * w with inv(r) = rsqrt(mean(r^2) + eps) one number per row, so inv can be taken out of the
// product that follows: (r * w * inv) W^T = inv * ((r * w) W^T). The product before the norm (o, down:
// ACT == 4) adds its rounded result to the float32 stream r in place and writes bf16(r * w) for the next
// product and, per 16 columns, the sum of r^2; the product after it (SCALED: the gated and the rotary form)
// adds up those sums while its first weights are on their way and multiplies its rows by inv before the bias.
// The norm and the addition are then no kernel of their own (vllm/kernels/layernorm_kernels.cu:41-68 in the
// reference); the values differ from the kernel's only in where the rounding to bfloat16 falls.
//
// MFMA: v_mfma_f32_16x16x32_bf16, A = W tile (16 rows x 32 k), B = x tile (32 k x 16 tokens), D[n][m]:
// lane l holds token m = l % 16 and the four outputs n = (l / 16) * 4 .. + 3.
#include "common.h"

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));   // a 16-byte piece in flight

template <int KC>
struct SkinnyTile {
  static constexpr int LANES_PER_ROW = KC / 8;              // 16-byte pieces per row of a tile
  static constexpr int ROWS_PER_LOAD = 64 / LANES_PER_ROW;  // rows one load instruction covers
  static constexpr int LOADS = 16 / ROWS_PER_LOAD;          // load instructions per tile
  static constexpr int ROW_BYTES = KC * 2 + 16;             // padded LDS row
  static constexpr int TILE_BYTES = 16 * ROW_BYTES;
  static constexpr int STEPS = KC / 32;                     // MFMA steps per chunk
};

// What the forms around a norm take beside the product's operands.
struct NormAroundArgs {
  // ACT == 4: the product before the norm
  float* stream;              // [M, N] float32 residual stream, updated in place
  long ld_stream;
  const bf16_t* norm_weight;  // [N] of the norm that follows
  float weight_offset;
  float* sumsq_out;           // [ceil(N / 16)][16]: sums of stream^2 over 16 columns, per row (rows >= M: 0)
  // SCALED: the product after the norm (its x is the bf16(stream * w) written above)
  const float* sumsq_in;      // [in_tiles][16]
  int in_tiles;
  float eps;
  int H;                      // columns of the stream: the mean is over these
};

// ACT: 0 none (plain linear layer), 1 silu-gated, 2 gelu-gated, 3 rotary embedding and cache write,
// 4 add to the stream and prepare the norm that follows (y receives bf16(stream * w))
// XROWS: rows of a tile of x that are fetched and staged, 16 or (one row tile of up to 8 rows) 8; the columns of the
// result that belong to the others are never stored.
template <int MT, int KC, int NW, typename TOut, int ACT, int DEPTH, bool SCALED, int XROWS>
__global__ __launch_bounds__(NW * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ x, long ldx,
                                                              const bf16_t* __restrict__ W, long ldw,
                                                              const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                              long ldy, int M, int N, int K, RopeCacheArgs rc,
                                                              NormAroundArgs na) {
  using T = SkinnyTile<KC>;
  constexpr int WT = (ACT >= 1 && ACT <= 3) ? 2 : 1;   // W tiles per chunk: gate and up, the two halves of a head, or one
  constexpr int XLOADS = (XROWS + T::ROWS_PER_LOAD - 1) / T::ROWS_PER_LOAD;   // load instructions per tile of x
  static_assert(XROWS == 16 || (XROWS == 8 && MT == 1 && XLOADS < T::LOADS), "8 rows of x: one row tile, and a whole load fewer");
  static_assert(!(SCALED || ACT == 4) || MT == 1, "the forms around a norm take up to 16 rows");
  static_assert(ACT != 4 || NW >= 4, "the epilogue of the product before a norm has a thread for each of the tile's 256 elements");
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int wave = tid / 64, lane = tid % 64;
  const int half = rc.d / 2;
  // first row of the first tile; the second tile starts tile_step rows further
  const int n0 = ACT == 3 ? (blockIdx.x / (half / 16)) * rc.d + (blockIdx.x % (half / 16)) * 16 : blockIdx.x * 16;
  const int tile_step = ACT == 3 ? half : N;
  unsigned char* my = lds + (size_t)wave * (WT + MT) * T::TILE_BYTES;

  // global load coordinates of this lane inside a tile
  const int lrow = lane / T::LANES_PER_ROW;      // + i * ROWS_PER_LOAD
  const int lcol = (lane % T::LANES_PER_ROW) * 8;  // element offset inside the chunk
  // LDS read coordinates (MFMA operand layout)
  const int fr = lane % 16, fg = lane / 16;

  // row offsets (in elements) of this lane's 16-byte pieces; rows beyond the matrix repeat the last row
  long woff[WT][T::LOADS], xoff[MT][T::LOADS];
#pragma unroll
  for (int i = 0; i < T::LOADS; ++i) {
    int r = n0 + lrow + i * T::ROWS_PER_LOAD;
    if (r > N - 1) r = N - 1;
#pragma unroll
    for (int wt = 0; wt < WT; ++wt) woff[wt][i] = (long)(r + wt * tile_step) * ldw + lcol;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      int m = mt * 16 + lrow + i * T::ROWS_PER_LOAD;
      if (m > M - 1) m = M - 1;
      xoff[mt][i] = (long)m * ldx + lcol;
    }
  }

  f32x4_t acc[WT][MT];
#pragma unroll
  for (int wt = 0; wt < WT; ++wt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[wt][mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  const int nchunks = (K + KC - 1) / KC;
  // DEPTH chunks per wave are in flight: while chunk c is multiplied, c + NW .. c + DEPTH * NW are on their way
  u32x4_t wreg[DEPTH][WT][T::LOADS], xreg[DEPTH][MT][T::LOADS];

  // K is a multiple of 8, so a 16-byte piece is inside or outside the row as a whole; a piece outside
  // is read from the start of the row instead and multiplied by nothing (its x piece is zeroed)
  // The weights are read once: their loads are marked non-temporal, so that they do not push out of the caches what is
  // read again and again (x). A fetch that is only made to keep the loop in one shape (live == false: the wave has
  // no further chunk) asks for a piece of x instead, which the caches hold, and its result is never used.
#define SKINNY_FETCH(buf, chunk, live)                                                          \
  {                                                                                             \
    const int k_ = (chunk) * KC;                                                                \
    const bool ok_ = (k_ + lcol) < K;                                                           \
    const int kk_ = ok_ ? k_ : -lcol;                                                           \
    const unsigned keep_ = ok_ ? 0xffffffffu : 0u;                                              \
    const bool live_ = (live);                                                                  \
    _Pragma("unroll") for (int i = 0; i < T::LOADS; ++i) {                                      \
      _Pragma("unroll") for (int wt = 0; wt < WT; ++wt) {                                       \
        const bf16_t* from_ = live_ ? W + woff[wt][i] : x + xoff[0][i];                         \
        wreg[buf][wt][i] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(from_ + kk_)); \
      }                                                                                         \
      _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) {                                       \
        if (i < XLOADS)                                                                         \
          xreg[buf][mt][i] = *reinterpret_cast<const u32x4_t*>(x + xoff[mt][i] + kk_) & keep_;  \
      }                                                                                         \
    }                                                                                           \
  }

  // Every fetch is unconditional, which keeps the staged pieces in registers across the loop.
  // SCALED: this thread's share of the sums of squares (row tid % 16). Loads come back in the order they were
  // asked for: these go first and are added up once the first weights have been asked for, so that waiting
  // for them does not wait for the weights.
  constexpr int SQ_HELD = 8;
  float sq_held[SQ_HELD];
  if (SCALED) {
#pragma unroll
    for (int i = 0; i < SQ_HELD; ++i) {
      const int e = tid + i * NW * 64;
      sq_held[i] = e < na.in_tiles * 16 ? na.sumsq_in[e] : 0.f;
    }
  }
  // ACT == 4: what the epilogue adds to and multiplies by does not hang on the product; it is asked for here, ahead
  // of the weights, so that the epilogue does not end on a trip to memory (thread e < 256 owns element e of the tile):
  // a decode step of 8 requests 3.628 -> 3.611 ms. (The same for the rotary form, position and slot here, cosine and
  // sine after the products: 3.608 -> 3.624, not kept.)
  // (kept as they come and converted where they are used: a conversion here would wait for them here)
  float held_stream = 0.f;
  bf16_t held_norm_w = 0, held_bias = 0;
  if (ACT == 4 && tid < 256) {
    const int l = tid / 4, n = n0 + (l / 16) * 4 + tid % 4, m = l % 16;
    if (n < N && m < M) {
      held_stream = na.stream[(long)m * na.ld_stream + n];
      held_norm_w = na.norm_weight[n];
      if (bias) held_bias = bias[n];
    }
  }
  int c = wave;
#pragma unroll
  for (int b = 0; b < DEPTH; ++b) SKINNY_FETCH(b, c + b * NW < nchunks ? c + b * NW : 0, c + b * NW < nchunks);
  float ssq = 0.f;
  if (SCALED) {
#pragma unroll
    for (int i = 0; i < SQ_HELD; ++i) ssq += sq_held[i];
    for (int e = tid + SQ_HELD * NW * 64; e < na.in_tiles * 16; e += NW * 64) ssq += na.sumsq_in[e];   // wider streams
    ssq += __shfl_xor(ssq, 16, 64);
    ssq += __shfl_xor(ssq, 32, 64);
  }
  while (c < nchunks) {
#pragma unroll
    for (int b = 0; b < DEPTH; ++b) {
      if (c >= nchunks) break;
      // registers -> LDS (load layout)
#pragma unroll
      for (int i = 0; i < T::LOADS; ++i) {
        const int off = (lrow + i * T::ROWS_PER_LOAD) * T::ROW_BYTES + lcol * 2;
#pragma unroll
        for (int wt = 0; wt < WT; ++wt) *reinterpret_cast<u32x4_t*>(my + wt * T::TILE_BYTES + off) = wreg[b][wt][i];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          if (i < XLOADS) *reinterpret_cast<u32x4_t*>(my + (WT + mt) * T::TILE_BYTES + off) = xreg[b][mt][i];
      }
      const int ahead = c + DEPTH * NW;
      SKINNY_FETCH(b, ahead < nchunks ? ahead : c, ahead < nchunks);
      // LDS -> operands (MFMA layout), multiply
#pragma unroll
      for (int s = 0; s < T::STEPS; ++s) {
        const int off = fr * T::ROW_BYTES + s * 64 + fg * 16;
        bf16x8_t a[WT];
#pragma unroll
        for (int wt = 0; wt < WT; ++wt) a[wt] = *reinterpret_cast<const bf16x8_t*>(my + wt * T::TILE_BYTES + off);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const bf16x8_t bb = *reinterpret_cast<const bf16x8_t*>(my + (WT + mt) * T::TILE_BYTES + off);
#pragma unroll
          for (int wt = 0; wt < WT; ++wt) acc[wt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[wt], bb, acc[wt][mt], 0, 0, 0);
        }
      }
      c += NW;
    }
  }
#undef SKINNY_FETCH

  // add the waves' partial sums in wave order
  __syncthreads();
  float* red = reinterpret_cast<float*>(lds);   // [NW][WT][MT][64 lanes][4]
  float* extra = red + (size_t)NW * WT * MT * 256;   // SCALED: [NW][16] sums of squares; ACT 4: [256] squares
#pragma unroll
  for (int wt = 0; wt < WT; ++wt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      *reinterpret_cast<f32x4_t*>(red + ((((size_t)wave * WT + wt) * MT + mt) * 64 + lane) * 4) = acc[wt][mt];
  if (SCALED && lane < 16) extra[wave * 16 + lane] = ssq;
  __syncthreads();
  for (int e = tid; e < MT * 256; e += NW * 64) {
    const int mt = e / 256, l = (e % 256) / 4, j = e % 4;
    float sum[WT];
#pragma unroll
    for (int wt = 0; wt < WT; ++wt) {
      sum[wt] = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) sum[wt] += red[((((size_t)w * WT + wt) * MT + mt) * 64 + l) * 4 + j];
    }
    const int n = n0 + (l / 16) * 4 + j, m = mt * 16 + l % 16;
    if (SCALED) {
      float total = 0.f;
#pragma unroll
      for (int w = 0; w < NW; ++w) total += extra[w * 16 + (l % 16)];
      const float inv = rsqrtf(total / (float)na.H + na.eps);
#pragma unroll
      for (int wt = 0; wt < WT; ++wt) sum[wt] *= inv;
    }
    if (ACT == 4) {
      // (MT == 1: thread e holds element e of the tile, row m = l % 16, column n)
      float sq = 0.f;
      if (n < N && m < M) {
        float r = sum[0];
        if (bias) r += bf16_to_f32(held_bias);
        const float v = held_stream + bf16_to_f32(f32_to_bf16(r));   // the product rounded as it is where it is stored first
        na.stream[(long)m * na.ld_stream + n] = v;
        reinterpret_cast<bf16_t*>(y)[(long)m * ldy + n] = f32_to_bf16(v * (bf16_to_f32(held_norm_w) + na.weight_offset));
        sq = v * v;
      }
      extra[e] = sq;
      continue;
    }
    if (ACT == 3) {
      if (m >= M) continue;
      float a = sum[0], b = sum[WT - 1];
      if (bias) {
        a += bf16_to_f32(bias[n]);
        b += bf16_to_f32(bias[n + half]);
      }
      // rounded to the storage type first, as the product stores them when the rotation is a kernel of its own
      a = bf16_to_f32(f32_to_bf16(a));
      b = bf16_to_f32(f32_to_bf16(b));
      const int head = n / rc.d, i = n - head * rc.d;   // i < d / 2: index of the rotation pair
      bf16_t lo, hi;
      if (head < rc.nh + rc.nkv) {
        const float* cs = rc.table + (long)rc.positions[m] * rc.d;
        const float c = cs[i], sn = cs[half + i];
        float xr, yr;
        rope_rotate(a, b, c, sn, &xr, &yr);
        lo = f32_to_bf16(xr);
        hi = f32_to_bf16(yr);
      } else {
        lo = f32_to_bf16(a);
        hi = f32_to_bf16(b);
      }
      bf16_t* yo = reinterpret_cast<bf16_t*>(y);   // this form writes bfloat16 only
      yo[(long)m * ldy + n] = lo;
      yo[(long)m * ldy + n + half] = hi;
      const int slot = rc.slots[m];
      if (head >= rc.nh && slot >= 0) {
        const int page = slot / rc.ps, off = slot - page * rc.ps;
        if (head < rc.nh + rc.nkv) {
          bf16_t* dst = rc.k_pages + (((long)page * rc.nkv + (head - rc.nh)) * rc.ps + off) * rc.d;
          dst[i] = lo;
          dst[i + half] = hi;
        } else {
          bf16_t* dst = rc.v_pages + ((long)page * rc.nkv + (head - rc.nh - rc.nkv)) * rc.d * rc.ps + off;
          dst[(long)i * rc.ps] = lo;
          dst[(long)(i + half) * rc.ps] = hi;
        }
      }
      continue;
    }
    if (n < N && m < M) {
      float r;
      if (ACT == 0) {
        r = sum[0];
        if (bias) r += bf16_to_f32(bias[n]);
      } else {
        float g = sum[0], u = sum[WT - 1];
        if (bias) {
          g += bf16_to_f32(bias[n]);
          u += bf16_to_f32(bias[N + n]);
        }
        // the two products are rounded to the storage type before the activation, as the unfused path
        // stores them (so both paths give the same bits)
        g = bf16_to_f32(f32_to_bf16(g));
        u = bf16_to_f32(f32_to_bf16(u));
        const float a = ACT == 1 ? g / (1.0f + expf(-g)) : 0.5f * g * (1.0f + erff(g * 0.70710678118654752f));
        r = a * u;
      }
      y[(long)m * ldy + n] = from_f32<TOut>(r);
    }
  }
  if (ACT == 4) {
    // the tile's sum of squares per row, in a fixed order: element e = 4 l + j is row l % 16
    __syncthreads();
    if (tid < 16) {
      float t = 0.f;
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) t += extra[(g * 16 + tid) * 4 + j];
      na.sumsq_out[(long)blockIdx.x * 16 + tid] = t;
    }
  }
}

template <int MT, int KC, int NW, typename TOut, int ACT, int DEPTH, bool SCALED, int XROWS>
static int launch_skinny_x(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int M,
                           int N, int K, hipStream_t stream, RopeCacheArgs rc, NormAroundArgs na) {
  using T = SkinnyTile<KC>;
  constexpr int WT = (ACT >= 1 && ACT <= 3) ? 2 : 1;
  const size_t stage = (size_t)NW * (WT + MT) * T::TILE_BYTES;
  const size_t red = (size_t)NW * WT * MT * 64 * 4 * sizeof(float) + ((SCALED || ACT == 4) ? 256 * sizeof(float) : 0);
  const size_t smem = stage > red ? stage : red;
  auto kernel = gemm_skinny_kernel<MT, KC, NW, TOut, ACT, DEPTH, SCALED, XROWS>;
  static bool configured = false;   // per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("gemm_skinny: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  // the gated form has a workgroup per 16 outputs, the rotary form one per 32 rows of W, the plain one per 16
  const int blocks = ACT == 3 ? N / 32 : (N + 15) / 16;
  hipLaunchKernelGGL(kernel, dim3(blocks), dim3(NW * 64), smem, stream, (const bf16_t*)x, ldx, (const bf16_t*)W, ldw,
                     (const bf16_t*)bias, (TOut*)y, ldy, M, N, K, rc, na);
  return 0;
}

template <int MT, int KC, int NW, typename TOut, int ACT, int DEPTH = 1, bool SCALED = false>
static int launch_skinny(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int M,
                         int N, int K, hipStream_t stream, RopeCacheArgs rc = RopeCacheArgs(),
                         NormAroundArgs na = NormAroundArgs()) {
  // up to 8 rows (and tiles whose loads cover 8 rows each): half of x's tile is neither fetched nor staged
  if constexpr (MT == 1 && SkinnyTile<KC>::ROWS_PER_LOAD <= 8) {
    if (M <= 8)
      return launch_skinny_x<MT, KC, NW, TOut, ACT, DEPTH, SCALED, 8>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream, rc, na);
  }
  return launch_skinny_x<MT, KC, NW, TOut, ACT, DEPTH, SCALED, 16>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream, rc, na);
}

// x [M, K] bfloat16 (row stride ldx), W [N, K] bfloat16 (row stride ldw), bias [N] bfloat16 or null,
// y [M, N] of out_dtype. Needs M <= 64, K a multiple of 8, 16-byte aligned x and W and row strides
// that are multiples of 8 elements; anything else is refused. ``variant`` picks the tiling (0: default).
// act 0: y = x W^T + bias. act 1 (silu) or 2 (gelu): W is [2 N, K] and bias [2 N], gate rows first;
// y = act(x Wgate^T + bgate) * (x Wup^T + bup), bfloat16 output only.
extern "C" int lmsf_gemm_skinny(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y,
                                int out_dtype, long ldy, int M, int N, int K, int variant, int act,
                                hipStream_t stream) {
  LMSF_CHECK(x && W && y, "gemm_skinny: null pointer");
  LMSF_CHECK(M >= 0 && M <= 64, "gemm_skinny: M=%d outside [0, 64]", M);
  LMSF_CHECK(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: K=%d must be a positive multiple of 8 (N=%d)", K, N);
  LMSF_CHECK(ldx >= K && ldw >= K && ldy >= N && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_skinny: row strides must cover K and be multiples of 8");
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W), "gemm_skinny: x and W must be 16-byte aligned");
  LMSF_CHECK(out_dtype == LMSF_F32 || out_dtype == LMSF_BF16, "gemm_skinny: unknown output dtype %d", out_dtype);
  LMSF_CHECK(act >= 0 && act <= 2, "gemm_skinny: unknown activation %d", act);
  LMSF_CHECK(act == 0 || out_dtype == LMSF_BF16, "gemm_skinny: the gated form writes bfloat16 only");
  if (M == 0) return 0;
  const int mt = (M + 15) / 16;
  int rc = 0;
  if (act) {
#define SKG(MT_, KC_, NW_)                                                                                     \
  rc = act == 1 ? launch_skinny<MT_, KC_, NW_, bf16_t, 1>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream)       \
                : launch_skinny<MT_, KC_, NW_, bf16_t, 2>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream)
    if (mt == 1) {
      // 8 waves with two chunks each in flight: measured 3 % ahead of 16 waves with one (deeper: slower)
      if (variant == 1) SKG(1, 128, 8);
      else if (variant == 3) SKG(1, 64, 16);
      else   // (variant 2 of the plain product splits K over 8 waves as well: the same order of summation)
        rc = act == 1 ? launch_skinny<1, 64, 8, bf16_t, 1, 2>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream)
                      : launch_skinny<1, 64, 8, bf16_t, 2, 2>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream);
    } else if (mt == 2) {
      SKG(2, 64, 16);
    } else if (mt == 3) {
      SKG(3, 64, 8);
    } else {
      SKG(4, 64, 8);
    }
#undef SKG
    if (rc) return rc;
    LMSF_LAUNCH_CHECK("gemm_skinny (gated)");
    return 0;
  }
#define SK(MT_, KC_, NW_)                                                                                          \
  rc = out_dtype == LMSF_F32 ? launch_skinny<MT_, KC_, NW_, float, 0>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream) \
                             : launch_skinny<MT_, KC_, NW_, bf16_t, 0>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream)
  if (mt == 1) {
    if (variant == 1) SK(1, 128, 8);
    else if (variant == 2) SK(1, 64, 8);
    else if (variant == 3) SK(1, 128, 16);
    else SK(1, 64, 16);
  } else if (mt == 2) {
    if (variant == 1) SK(2, 128, 8);
    else SK(2, 64, 16);
  } else if (mt == 3) {
    SK(3, 64, 8);
  } else {
    SK(4, 64, 8);
  }
#undef SK
  if (rc) return rc;
  LMSF_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

// The fused QKV projection with rotary embedding and cache write as its epilogue, for M <= 16 tokens:
// y[M, (nh + 2 nkv) d] = x W^T (+ bias), then q and k heads rotated in NeoX style over the whole head by
// table[positions[m]] ([max_pos, d] = cos | sin, float32), k and v stored in the pages at slots[m]
// (negative: not stored). Needs what lmsf_gemm_skinny needs and d a multiple of 32.
extern "C" int lmsf_gemm_qkv_rope_cache(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y,
                                        long ldy, int M, int K, const int* positions, const float* table, int max_pos,
                                        const int* slots, void* k_pages, void* v_pages, long num_pages, int nh,
                                        int nkv, int d, int ps, int variant, hipStream_t stream) {
  LMSF_CHECK(x && W && y && positions && table && slots && k_pages && v_pages, "gemm_qkv_rope_cache: null pointer");
  LMSF_CHECK(M >= 0 && M <= 64, "gemm_qkv_rope_cache: M=%d outside [0, 64]", M);
  LMSF_CHECK(nh > 0 && nkv > 0 && d >= 32 && d % 32 == 0, "gemm_qkv_rope_cache: head size %d must be a multiple of 32", d);
  const long N = (long)(nh + 2 * nkv) * d;
  LMSF_CHECK(N / 32 <= 2147483647L, "gemm_qkv_rope_cache: too many rows");
  LMSF_CHECK(K > 0 && K % 8 == 0, "gemm_qkv_rope_cache: K=%d must be a positive multiple of 8", K);
  LMSF_CHECK(ldx >= K && ldw >= K && ldy >= N && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_qkv_rope_cache: row strides must cover K and be multiples of 8");
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W), "gemm_qkv_rope_cache: x and W must be 16-byte aligned");
  LMSF_CHECK(ps > 0 && num_pages > 0 && max_pos > 0, "gemm_qkv_rope_cache: bad page geometry or empty table");
  if (M == 0) return 0;
  RopeCacheArgs rc;
  rc.positions = positions; rc.table = table; rc.slots = slots;
  rc.k_pages = (bf16_t*)k_pages; rc.v_pages = (bf16_t*)v_pages;
  rc.nh = nh; rc.nkv = nkv; rc.d = d; rc.ps = ps;
  int r;
  if (M > 48)       // (eight waves: the stages of sixteen would not fit LDS beside three and four tiles of x)
    r = launch_skinny<4, 64, 8, bf16_t, 3>(x, ldx, W, ldw, bias, y, ldy, M, (int)N, K, stream, rc);
  else if (M > 32)
    r = launch_skinny<3, 64, 8, bf16_t, 3>(x, ldx, W, ldw, bias, y, ldy, M, (int)N, K, stream, rc);
  else if (M > 16)
    r = launch_skinny<2, 64, 16, bf16_t, 3>(x, ldx, W, ldw, bias, y, ldy, M, (int)N, K, stream, rc);
  else if (variant == 1)
    r = launch_skinny<1, 64, 8, bf16_t, 3>(x, ldx, W, ldw, bias, y, ldy, M, (int)N, K, stream, rc);
  else
    r = launch_skinny<1, 64, 16, bf16_t, 3>(x, ldx, W, ldw, bias, y, ldy, M, (int)N, K, stream, rc);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemm_qkv_rope_cache");
  return 0;
}

// The forms around a norm (up to 16 rows; see the top of the file).

// The product before the norm: stream [M, N] float32 += bf16(x W^T + bias) in place; xw [M, N] = bf16(stream *
// (norm_weight + weight_offset)); sumsq [ceil(N / 16)][16] = per 16 columns and row the sum of stream^2.
extern "C" int lmsf_gemm_skinny_add_norm(const void* x, long ldx, const void* W, long ldw, const void* bias,
                                         void* stream_f32, long ld_stream, const void* norm_weight,
                                         float weight_offset, void* xw, long ld_xw, float* sumsq, int M, int N, int K,
                                         int variant, hipStream_t stream) {
  LMSF_CHECK(x && W && stream_f32 && norm_weight && xw && sumsq, "gemm_skinny_add_norm: null pointer");
  LMSF_CHECK(M >= 0 && M <= 16, "gemm_skinny_add_norm: M=%d outside [0, 16]", M);
  LMSF_CHECK(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny_add_norm: K=%d must be a positive multiple of 8 (N=%d)", K, N);
  LMSF_CHECK(ldx >= K && ldw >= K && ld_stream >= N && ld_xw >= N && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_skinny_add_norm: row strides must cover the rows and those of x and W be multiples of 8");
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W), "gemm_skinny_add_norm: x and W must be 16-byte aligned");
  if (M == 0) return 0;
  NormAroundArgs na = NormAroundArgs();
  na.stream = (float*)stream_f32; na.ld_stream = ld_stream;
  na.norm_weight = (const bf16_t*)norm_weight; na.weight_offset = weight_offset;
  na.sumsq_out = sumsq;
  int r;
  if (variant == 2)
    r = launch_skinny<1, 64, 8, bf16_t, 4>(x, ldx, W, ldw, bias, xw, ld_xw, M, N, K, stream, RopeCacheArgs(), na);
  else
    r = launch_skinny<1, 64, 16, bf16_t, 4>(x, ldx, W, ldw, bias, xw, ld_xw, M, N, K, stream, RopeCacheArgs(), na);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemm_skinny_add_norm");
  return 0;
}

static int scaled_check(const char* who, const float* sumsq, int in_tiles, int H) {
  LMSF_CHECK(sumsq != nullptr && in_tiles > 0 && H > 0 && in_tiles == (H + 15) / 16,
             "%s: %d sums of squares do not cover %d columns", who, in_tiles, H);
  return 0;
}

// lmsf_gemm_skinny's gated form (act 1 silu, 2 gelu) after a norm: x [M, K] is bf16(stream * w) as written by
// lmsf_gemm_skinny_add_norm, sumsq [in_tiles][16] its sums of squares; the two products' rows are multiplied
// by rsqrt(sum / H + eps) before bias and activation. K == H.
extern "C" int lmsf_gemm_skinny_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y,
                                       long ldy, int M, int N, int K, int act, const float* sumsq, int in_tiles,
                                       float eps, int variant, hipStream_t stream) {
  LMSF_CHECK(x && W && y, "gemm_skinny_scaled: null pointer");
  LMSF_CHECK(M >= 0 && M <= 16, "gemm_skinny_scaled: M=%d outside [0, 16]", M);
  LMSF_CHECK(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny_scaled: K=%d must be a positive multiple of 8 (N=%d)", K, N);
  LMSF_CHECK(ldx >= K && ldw >= K && ldy >= N && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_skinny_scaled: row strides must cover K and be multiples of 8");
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W), "gemm_skinny_scaled: x and W must be 16-byte aligned");
  LMSF_CHECK(act == 1 || act == 2, "gemm_skinny_scaled: activation %d (1 silu, 2 gelu)", act);
  if (int rc = scaled_check("gemm_skinny_scaled", sumsq, in_tiles, K)) return rc;
  if (M == 0) return 0;
  NormAroundArgs na = NormAroundArgs();
  na.sumsq_in = sumsq; na.in_tiles = in_tiles; na.eps = eps; na.H = K;
  int r;
  if (variant == 3)
    r = act == 1 ? launch_skinny<1, 64, 16, bf16_t, 1, 1, true>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream, RopeCacheArgs(), na)
                 : launch_skinny<1, 64, 16, bf16_t, 2, 1, true>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream, RopeCacheArgs(), na);
  else
    r = act == 1 ? launch_skinny<1, 64, 8, bf16_t, 1, 2, true>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream, RopeCacheArgs(), na)
                 : launch_skinny<1, 64, 8, bf16_t, 2, 2, true>(x, ldx, W, ldw, bias, y, ldy, M, N, K, stream, RopeCacheArgs(), na);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemm_skinny_scaled");
  return 0;
}

// lmsf_gemm_qkv_rope_cache after a norm: x and sumsq as in lmsf_gemm_skinny_scaled.
extern "C" int lmsf_gemm_qkv_rope_cache_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias,
                                               void* y, long ldy, int M, int K, const int* positions,
                                               const float* table, int max_pos, const int* slots, void* k_pages,
                                               void* v_pages, long num_pages, int nh, int nkv, int d, int ps,
                                               const float* sumsq, int in_tiles, float eps, hipStream_t stream) {
  LMSF_CHECK(x && W && y && positions && table && slots && k_pages && v_pages, "gemm_qkv_rope_cache_scaled: null pointer");
  LMSF_CHECK(M >= 0 && M <= 16, "gemm_qkv_rope_cache_scaled: M=%d outside [0, 16]", M);
  LMSF_CHECK(nh > 0 && nkv > 0 && d >= 32 && d % 32 == 0, "gemm_qkv_rope_cache_scaled: head size %d must be a multiple of 32", d);
  const long N = (long)(nh + 2 * nkv) * d;
  LMSF_CHECK(N / 32 <= 2147483647L, "gemm_qkv_rope_cache_scaled: too many rows");
  LMSF_CHECK(K > 0 && K % 8 == 0, "gemm_qkv_rope_cache_scaled: K=%d must be a positive multiple of 8", K);
  LMSF_CHECK(ldx >= K && ldw >= K && ldy >= N && ldx % 8 == 0 && ldw % 8 == 0,
             "gemm_qkv_rope_cache_scaled: row strides must cover K and be multiples of 8");
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W), "gemm_qkv_rope_cache_scaled: x and W must be 16-byte aligned");
  LMSF_CHECK(ps > 0 && num_pages > 0 && max_pos > 0, "gemm_qkv_rope_cache_scaled: bad page geometry or empty table");
  if (int rc = scaled_check("gemm_qkv_rope_cache_scaled", sumsq, in_tiles, K)) return rc;
  if (M == 0) return 0;
  RopeCacheArgs rc;
  rc.positions = positions; rc.table = table; rc.slots = slots;
  rc.k_pages = (bf16_t*)k_pages; rc.v_pages = (bf16_t*)v_pages;
  rc.nh = nh; rc.nkv = nkv; rc.d = d; rc.ps = ps;
  NormAroundArgs na = NormAroundArgs();
  na.sumsq_in = sumsq; na.in_tiles = in_tiles; na.eps = eps; na.H = K;
  // (up to 8 rows 8 waves are ahead of 16, a decode step of 8 requests 3.298 -> 3.266 ms; at 16 rows behind, 3.62 -> 3.71)
  int r = M <= 8 ? launch_skinny<1, 64, 8, bf16_t, 3, 1, true>(x, ldx, W, ldw, bias, y, ldy, M, (int)N, K, stream, rc, na)
                 : launch_skinny<1, 64, 16, bf16_t, 3, 1, true>(x, ldx, W, ldw, bias, y, ldy, M, (int)N, K, stream, rc, na);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemm_qkv_rope_cache_scaled");
  return 0;
}
