// Linear layer for one or two rows (decoding a single request, or two): y[M, N] = x[M, K] W[N, K]^T (+ bias),
// bfloat16 inputs, float32 accumulation, bfloat16 or float32 output, with the same fused epilogues as the
// few-rows product (gated activation; rotary embedding and cache write for the fused QKV projection).
//
// With one row there is nothing for the matrix cores to share: every weight is used once. The product is a
// pure stream of W, and the kernel is shaped like the fastest reader of memory that was measured on this
// chip: a wave owns one row of W at a time and reads it 1 KB per instruction (64 lanes x 16 bytes,
// consecutive), eight instructions in flight; x lies in LDS (bfloat16, read 16 bytes per lane beside every 16
// bytes of W); the lanes' partial sums are added across the wave at the end of the row. No LDS staging of W,
// no layout change, no barrier after the first. The few-rows kernel (matrix cores, W through LDS) reaches 80 %
// of that reader's rate, which is why these one or two rows get a kernel of their own.
// The reference leaves these products to cuBLASLt (tops/src/cublas.rs:29-114).
//
// Two more forms take the kernels between two products of a decoder block into the products themselves:
// ACT 4 adds the result, rounded to bfloat16 as a product would store it, to the float32 residual stream in
// place (every element of the stream belongs to one wave), and can write what the norm that follows needs;
// SC takes that norm's row factor out of the product (see GemvNorm). The addition and the norm are then no
// kernels of their own (vllm/kernels/layernorm_kernels.cu:41-68 in the reference).
//
// A "unit" is what one wave produces: ACT 0: output n (one row of W); ACT 1, 2: output n of the gated form
// (rows n and N + n: gate and up); ACT 3: the rotation pair (i, i + d/2) of one head of the fused QKV
// projection (rows head * d + i and head * d + i + d/2).
#include "common.h"

typedef __bf16 gemv_bf16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned int gemv_u32x4_t __attribute__((ext_vector_type(4)));

#define GEMV_WAVES 8
#define GEMV_UNROLL 8   // 16-byte pieces per lane in flight per row: 8 x 512 = 4,096 elements of K

// A wave's work is a list of pieces: for each of its units, for each of the unit's rows (one, or two with an
// epilogue that joins two rows), the row's K in pieces of GEMV_UNROLL x 512 elements. The loads of the next
// piece are issued before the current one is multiplied, and those of the very first before the workgroup
// has x in LDS, so the memory pipe never waits for arithmetic, a reduction or the start of a workgroup.
struct GemvCursor {
  int unit, row, kb;
};

// The forms around a norm: ACT 4 with xw_out also writes bf16(stream * (weight + offset)) for the next product
// and, per workgroup and row, the sum of the squares of the stream's elements it produced (sumsq_out
// [workgroups][NX]); SC multiplies its rows by rsqrt(sum of sumsq_in / K + eps) before the bias, its x being
// that bf16(stream * w): RMSNorm is r * inv(r) * w with one inv per row, and (r * w * inv) W^T =
// inv * ((r * w) W^T).
struct GemvNorm {
  const bf16_t* weight;   // [N] of the norm that follows (ACT 4)
  float eps, offset;
  bf16_t* xw_out;
  long ld_xw;
  float* sumsq_out;
  const float* sumsq_in;
  int n_partials;
};

template <int NX, int ACT, typename TOut, bool SC>
__global__ __launch_bounds__(GEMV_WAVES * 64) void gemv_kernel(const bf16_t* __restrict__ x, long ldx,
                                                               const bf16_t* __restrict__ W, long ldw,
                                                               const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                               long ldy, int N, int K, int n_units, RopeCacheArgs rc,
                                                               GemvNorm nm) {
  constexpr int ROWS = (ACT == 0 || ACT == 4) ? 1 : 2;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  bf16_t* xs = reinterpret_cast<bf16_t*>(lds_raw);             // [NX][K]
  __shared__ float norm_red[GEMV_WAVES][NX];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int half = rc.d / 2;
  const int unit_step = (int)(gridDim.x * GEMV_WAVES);

  auto row_of = [&](const GemvCursor& c) -> int {
    if (ACT == 3) {
      const int head = c.unit / half, i = c.unit - head * half;
      return head * rc.d + i + c.row * half;
    }
    return c.unit + c.row * N;
  };
  auto fetch = [&](const GemvCursor& c, uint4* wv) {
    const bf16_t* w_row = W + (long)row_of(c) * ldw;
#pragma unroll
    for (int j = 0; j < GEMV_UNROLL; ++j) {
      const int k = c.kb + j * 512 + lane * 8;
      // (read once: marked non-temporal, so that the weights do not push x and the stream out of the caches)
      if (k < K) {
        const gemv_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const gemv_u32x4_t*>(w_row + k));
        wv[j] = make_uint4(v.x, v.y, v.z, v.w);
      } else {
        wv[j] = make_uint4(0u, 0u, 0u, 0u);
      }
    }
  };
  auto advance = [&](GemvCursor& c) {
    c.kb += GEMV_UNROLL * 512;
    if (c.kb >= K) {
      c.kb = 0;
      if (++c.row == ROWS) {
        c.row = 0;
        c.unit += unit_step;
      }
    }
  };

  float acc0[NX], acc1[NX];   // the sums of the unit's first and second row (kept apart: registers, not an indexed array)
  auto multiply_into = [&](float (&acc)[NX], const GemvCursor& c, const uint4* wv) {
    if (c.kb == 0) {
#pragma unroll
      for (int m = 0; m < NX; ++m) acc[m] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < GEMV_UNROLL; ++j) {
      if (c.kb + j * 512 >= K) break;              // the same for every lane
      const int k = c.kb + j * 512 + lane * 8;
      const uint32_t ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
#pragma unroll
      for (int m = 0; m < NX; ++m) {
        // beyond K the weights are zeros; x is read from a valid place all the same
        const uint4 xv = *reinterpret_cast<const uint4*>(xs + (long)m * K + (k < K ? k : 0));
        const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
        // two products and the addition to the float32 sum in one instruction (v_dot2c_f32_bf16)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          acc[m] = __builtin_amdgcn_fdot2_f32_bf16(*reinterpret_cast<const gemv_bf16x2_t*>(&ww[e]),
                                                   *reinterpret_cast<const gemv_bf16x2_t*>(&xw[e]), acc[m], false);
      }
    }
  };
  auto multiply = [&](const GemvCursor& c, const uint4* wv) {
    if (c.row == 0) multiply_into(acc0, c, wv);
    else multiply_into(acc1, c, wv);
  };
  float inv_rms[NX];   // SC: the rows' factors
  float sq_acc[NX];    // ACT 4 with xw_out: squares of what this wave added to the stream
#pragma unroll
  for (int m = 0; m < NX; ++m) {
    inv_rms[m] = 1.f;
    sq_acc[m] = 0.f;
  }
  // the unit's rows are complete: add the lanes' sums, apply the epilogue, store
  auto finish = [&](int unit) {
    float p[NX], q[NX];
#pragma unroll
    for (int m = 0; m < NX; ++m) {
      p[m] = wave_sum(acc0[m]);
      q[m] = ROWS == 2 ? wave_sum(acc1[m]) : 0.f;
      if (SC) {
        p[m] *= inv_rms[m];
        q[m] *= inv_rms[m];
      }
    }
    if (lane != 0) return;
    GemvCursor c0 = {unit, 0, 0}, c1 = {unit, ROWS - 1, 0};
    const int n = row_of(c0), n2 = row_of(c1);
#pragma unroll
    for (int m = 0; m < NX; ++m) {
      float a = p[m], b = q[m];
      if (bias) {
        a += bf16_to_f32(bias[n]);
        if (ROWS == 2) b += bf16_to_f32(bias[n2]);
      }
      if (ACT == 0) {
        y[(long)m * ldy + n] = from_f32<TOut>(a);
      } else if (ACT == 4) {
        float* st = reinterpret_cast<float*>(y) + (long)m * ldy + n;   // this form's output is the float32 stream
        const float v = *st + bf16_to_f32(f32_to_bf16(a));
        *st = v;
        if (nm.xw_out) {
          nm.xw_out[(long)m * nm.ld_xw + n] = f32_to_bf16(v * (bf16_to_f32(nm.weight[n]) + nm.offset));
          sq_acc[m] += v * v;
        }
      } else if (ACT == 1 || ACT == 2) {
        // the two products are rounded to the storage type before the activation, as the unfused path stores them
        const float g = bf16_to_f32(f32_to_bf16(a)), u = bf16_to_f32(f32_to_bf16(b));
        const float act = ACT == 1 ? g / (1.0f + expf(-g)) : 0.5f * g * (1.0f + erff(g * 0.70710678118654752f));
        y[(long)m * ldy + n] = from_f32<TOut>(act * u);
      } else {
        // rounded to the storage type first, as the product stores them when the rotation is a kernel of its own
        a = bf16_to_f32(f32_to_bf16(a));
        b = bf16_to_f32(f32_to_bf16(b));
        const int head = n / rc.d, i = n - head * rc.d;
        bf16_t lo, hi;
        if (head < rc.nh + rc.nkv) {
          const float* cs = rc.table + (long)rc.positions[m] * rc.d;
          float xr, yr;
          rope_rotate(a, b, cs[i], cs[half + i], &xr, &yr);
          lo = f32_to_bf16(xr);
          hi = f32_to_bf16(yr);
        } else {
          lo = f32_to_bf16(a);
          hi = f32_to_bf16(b);
        }
        bf16_t* yo = reinterpret_cast<bf16_t*>(y);   // this form writes bfloat16 only
        yo[(long)m * ldy + n] = lo;
        yo[(long)m * ldy + n2] = hi;
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
      }
    }
  };

  GemvCursor cur = {(int)(blockIdx.x * GEMV_WAVES) + wave, 0, 0};
  uint4 wa[GEMV_UNROLL], wb[GEMV_UNROLL];
  {
    float part[NX];
    if (SC) {
      // this thread's share of the sums of squares, asked for first (loads come back in order)
#pragma unroll
      for (int m = 0; m < NX; ++m) part[m] = 0.f;
      for (int i = tid; i < nm.n_partials; i += GEMV_WAVES * 64) {
#pragma unroll
        for (int m = 0; m < NX; ++m) part[m] += nm.sumsq_in[(long)i * NX + m];
      }
    }
    if (cur.unit < n_units) fetch(cur, wa);
    for (int i = tid; i < NX * (K / 8); i += GEMV_WAVES * 64) {
      const int m = i / (K / 8), p = i - m * (K / 8);
      *reinterpret_cast<uint4*>(xs + (long)m * K + p * 8) = *reinterpret_cast<const uint4*>(x + (long)m * ldx + p * 8);
    }
    if (SC) {
#pragma unroll
      for (int m = 0; m < NX; ++m) {
        const float t = wave_sum(part[m]);
        if (lane == 0) norm_red[wave][m] = t;
      }
    }
  }
  __syncthreads();
  if (SC) {
#pragma unroll
    for (int m = 0; m < NX; ++m) {
      float tot = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < GEMV_WAVES; ++w2) tot += norm_red[w2][m];
      inv_rms[m] = rsqrtf(tot / (float)K + nm.eps);
    }
  }
  // one piece per half of the loop body, the two register sets taking turns
#define GEMV_HALF(mine, other)                                                       \
  {                                                                                  \
    GemvCursor nxt = cur;                                                            \
    advance(nxt);                                                                    \
    if (nxt.unit < n_units) fetch(nxt, other);                                       \
    multiply(cur, mine);                                                             \
    if (nxt.unit != cur.unit) finish(cur.unit);                                      \
    cur = nxt;                                                                       \
  }
  while (cur.unit < n_units) {
    GEMV_HALF(wa, wb);
    if (cur.unit >= n_units) break;
    GEMV_HALF(wb, wa);
  }
#undef GEMV_HALF
  if (ACT == 4 && nm.sumsq_out) {
    // the workgroup's sums of squares, the waves' in wave order (every wave comes here, with or without units)
    if (lane == 0) {
#pragma unroll
      for (int m = 0; m < NX; ++m) norm_red[wave][m] = sq_acc[m];
    }
    __syncthreads();
    if (tid < NX) {
      float t = 0.f;
#pragma unroll
      for (int w2 = 0; w2 < GEMV_WAVES; ++w2) t += norm_red[w2][tid];
      nm.sumsq_out[(long)blockIdx.x * NX + tid] = t;
    }
  }
}

// workgroups of a launch over n_units units: every wave takes one unit at a time
static long gemv_blocks(long n_units) {
  long blocks = (n_units + GEMV_WAVES - 1) / GEMV_WAVES;
  return blocks > 2048 ? 2048 : blocks;
}

template <int NX, int ACT, typename TOut, bool SC = false>
static int launch_gemv(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int N,
                       int K, int n_units, hipStream_t stream, RopeCacheArgs rc = RopeCacheArgs(),
                       GemvNorm nm = GemvNorm()) {
  const size_t smem = (size_t)NX * K * sizeof(bf16_t);
  auto kernel = gemv_kernel<NX, ACT, TOut, SC>;
  static size_t configured = 0;   // per instantiation: the largest LDS size asked for so far
  if (smem > configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("gemv: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = smem;
  }
  const long blocks = gemv_blocks(n_units);   // at most 8 workgroups per compute unit's worth of them
  hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(GEMV_WAVES * 64), smem, stream, (const bf16_t*)x, ldx,
                     (const bf16_t*)W, ldw, (const bf16_t*)bias, (TOut*)y, ldy, N, K, n_units, rc, nm);
  return 0;
}

static int gemv_check(const char* who, const void* x, long ldx, const void* W, long ldw, int M, long N, int K) {
  LMSF_CHECK(x && W, "%s: null pointer", who);
  LMSF_CHECK(M >= 0 && M <= 2, "%s: M=%d outside [0, 2]", who, M);
  LMSF_CHECK(N > 0 && N <= 2147483647L / 2 && K > 0 && K % 8 == 0, "%s: K=%d must be a positive multiple of 8 (N=%ld)", who, K, N);
  LMSF_CHECK((long)M * K * 2 <= 160 * 1024 - 1024, "%s: x (%d x %d) does not fit LDS", who, M, K);
  LMSF_CHECK(ldx >= K && ldw >= K && ldx % 8 == 0 && ldw % 8 == 0, "%s: row strides must cover K and be multiples of 8", who);
  LMSF_CHECK(lmsf_aligned16(x) && lmsf_aligned16(W), "%s: x and W must be 16-byte aligned", who);
  return 0;
}

// x [M, K] bfloat16, M <= 2; W [N, K] (act 0) or [2 N, K] (act 1 silu, 2 gelu: gate rows first); bias likewise or
// null; y [M, N] of out_dtype (float32 only without activation). K a multiple of 8, x and W 16-byte aligned
// with row strides that are multiples of 8; M * K * 2 bytes must fit LDS.
extern "C" int lmsf_gemv(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, int out_dtype,
                         long ldy, int M, int N, int K, int act, hipStream_t stream) {
  if (int rc = gemv_check("gemv", x, ldx, W, ldw, M, N, K)) return rc;
  LMSF_CHECK(y != nullptr && ldy >= N, "gemv: bad output");
  LMSF_CHECK(act >= 0 && act <= 2, "gemv: unknown activation %d", act);
  LMSF_CHECK(out_dtype == LMSF_BF16 || (out_dtype == LMSF_F32 && act == 0),
             "gemv: output is bfloat16, or float32 without activation");
  if (M == 0) return 0;
  int r;
#define GV(NX_)                                                                                              \
  r = act == 1   ? launch_gemv<NX_, 1, bf16_t>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream)                 \
      : act == 2 ? launch_gemv<NX_, 2, bf16_t>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream)                 \
      : out_dtype == LMSF_F32 ? launch_gemv<NX_, 0, float>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream)     \
                              : launch_gemv<NX_, 0, bf16_t>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream)
  if (M == 1) GV(1); else GV(2);
#undef GV
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemv");
  return 0;
}

// The fused QKV projection with rotary embedding (NeoX pairing over the whole head) and cache write as its
// epilogue, for M <= 2 tokens; arguments as lmsf_gemm_qkv_rope_cache. Needs an even head size.
extern "C" int lmsf_gemv_qkv_rope_cache(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y,
                                        long ldy, int M, int K, const int* positions, const float* table, int max_pos,
                                        const int* slots, void* k_pages, void* v_pages, long num_pages, int nh,
                                        int nkv, int d, int ps, hipStream_t stream) {
  LMSF_CHECK(y && positions && table && slots && k_pages && v_pages, "gemv_qkv_rope_cache: null pointer");
  LMSF_CHECK(nh > 0 && nkv > 0 && d >= 2 && d % 2 == 0, "gemv_qkv_rope_cache: head size %d must be even", d);
  const long N = (long)(nh + 2 * nkv) * d;
  if (int rc = gemv_check("gemv_qkv_rope_cache", x, ldx, W, ldw, M, N, K)) return rc;
  LMSF_CHECK(ldy >= N, "gemv_qkv_rope_cache: row stride of y below %ld", N);
  LMSF_CHECK(ps > 0 && num_pages > 0 && max_pos > 0, "gemv_qkv_rope_cache: bad page geometry or empty table");
  if (M == 0) return 0;
  RopeCacheArgs rc;
  rc.positions = positions; rc.table = table; rc.slots = slots;
  rc.k_pages = (bf16_t*)k_pages; rc.v_pages = (bf16_t*)v_pages;
  rc.nh = nh; rc.nkv = nkv; rc.d = d; rc.ps = ps;
  const int n_units = (int)(N / 2);
  int r = M == 1 ? launch_gemv<1, 3, bf16_t>(x, ldx, W, ldw, bias, y, ldy, (int)N, K, n_units, stream, rc)
                 : launch_gemv<2, 3, bf16_t>(x, ldx, W, ldw, bias, y, ldy, (int)N, K, n_units, stream, rc);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemv_qkv_rope_cache");
  return 0;
}

// y += bf16(x W^T + bias): y is the float32 residual stream [M, N] with row stride ldy, updated in place; the
// product is rounded to bfloat16 first, as it is where it is stored before it is added. x, W as in lmsf_gemv.
extern "C" int lmsf_gemv_add(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
                             int M, int N, int K, hipStream_t stream) {
  if (int rc = gemv_check("gemv_add", x, ldx, W, ldw, M, N, K)) return rc;
  LMSF_CHECK(y != nullptr && ldy >= N, "gemv_add: bad output");
  if (M == 0) return 0;
  int r = M == 1 ? launch_gemv<1, 4, float>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream)
                 : launch_gemv<2, 4, float>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemv_add");
  return 0;
}

// The forms around a norm for one or two rows (see GemvNorm).

// Workgroups, and so sums of squares per row, of lmsf_gemv_add_norm with N outputs.
extern "C" int lmsf_gemv_partials(int N) { return (int)gemv_blocks(N); }

// lmsf_gemv_add that also writes xw [M, N] = bf16(stream * (norm_weight + weight_offset)) and
// sumsq [lmsf_gemv_partials(N)][M]: per workgroup and row the sum of the squares of the stream's elements
// that the workgroup produced.
extern "C" int lmsf_gemv_add_norm(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y,
                                  long ldy, const void* norm_weight, float weight_offset, void* xw, long ld_xw,
                                  float* sumsq, int M, int N, int K, hipStream_t stream) {
  if (int rc = gemv_check("gemv_add_norm", x, ldx, W, ldw, M, N, K)) return rc;
  LMSF_CHECK(y != nullptr && ldy >= N && norm_weight && xw && ld_xw >= N && sumsq, "gemv_add_norm: bad output");
  if (M == 0) return 0;
  GemvNorm nm = GemvNorm();
  nm.weight = (const bf16_t*)norm_weight; nm.offset = weight_offset;
  nm.xw_out = (bf16_t*)xw; nm.ld_xw = ld_xw; nm.sumsq_out = sumsq;
  int r = M == 1 ? launch_gemv<1, 4, float>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream, RopeCacheArgs(), nm)
                 : launch_gemv<2, 4, float>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream, RopeCacheArgs(), nm);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemv_add_norm");
  return 0;
}

// lmsf_gemv's gated forms (act 1 silu, 2 gelu) after a norm: x is the xw of lmsf_gemv_add_norm, sumsq its sums
// ([n_partials][M]); rows are multiplied by rsqrt(sum / K + eps) before bias and activation.
extern "C" int lmsf_gemv_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
                                int M, int N, int K, int act, const float* sumsq, int n_partials, float eps,
                                hipStream_t stream) {
  if (int rc = gemv_check("gemv_scaled", x, ldx, W, ldw, M, N, K)) return rc;
  LMSF_CHECK(y != nullptr && ldy >= N && sumsq && n_partials > 0, "gemv_scaled: bad output or sums");
  LMSF_CHECK(act == 1 || act == 2, "gemv_scaled: activation %d (1 silu, 2 gelu)", act);
  if (M == 0) return 0;
  GemvNorm nm = GemvNorm();
  nm.sumsq_in = sumsq; nm.n_partials = n_partials; nm.eps = eps;
  int r;
#define GV(NX_)                                                                                                          \
  r = act == 1 ? launch_gemv<NX_, 1, bf16_t, true>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream, RopeCacheArgs(), nm) \
               : launch_gemv<NX_, 2, bf16_t, true>(x, ldx, W, ldw, bias, y, ldy, N, K, N, stream, RopeCacheArgs(), nm)
  if (M == 1) GV(1); else GV(2);
#undef GV
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemv_scaled");
  return 0;
}

// lmsf_gemv_qkv_rope_cache after a norm: x and sumsq as in lmsf_gemv_scaled.
extern "C" int lmsf_gemv_scaled_qkv_rope_cache(const void* x, long ldx, const void* W, long ldw, const void* bias,
                                               void* y, long ldy, int M, int K, const int* positions,
                                               const float* table, int max_pos, const int* slots, void* k_pages,
                                               void* v_pages, long num_pages, int nh, int nkv, int d, int ps,
                                               const float* sumsq, int n_partials, float eps, hipStream_t stream) {
  LMSF_CHECK(y && positions && table && slots && k_pages && v_pages, "gemv_scaled_qkv_rope_cache: null pointer");
  LMSF_CHECK(nh > 0 && nkv > 0 && d >= 2 && d % 2 == 0, "gemv_scaled_qkv_rope_cache: head size %d must be even", d);
  const long N = (long)(nh + 2 * nkv) * d;
  if (int rc = gemv_check("gemv_scaled_qkv_rope_cache", x, ldx, W, ldw, M, N, K)) return rc;
  LMSF_CHECK(ldy >= N, "gemv_scaled_qkv_rope_cache: row stride of y below %ld", N);
  LMSF_CHECK(ps > 0 && num_pages > 0 && max_pos > 0, "gemv_scaled_qkv_rope_cache: bad page geometry or empty table");
  LMSF_CHECK(sumsq && n_partials > 0, "gemv_scaled_qkv_rope_cache: no sums of squares");
  if (M == 0) return 0;
  RopeCacheArgs rc;
  rc.positions = positions; rc.table = table; rc.slots = slots;
  rc.k_pages = (bf16_t*)k_pages; rc.v_pages = (bf16_t*)v_pages;
  rc.nh = nh; rc.nkv = nkv; rc.d = d; rc.ps = ps;
  GemvNorm nm = GemvNorm();
  nm.sumsq_in = sumsq; nm.n_partials = n_partials; nm.eps = eps;
  const int n_units = (int)(N / 2);
  int r = M == 1 ? launch_gemv<1, 3, bf16_t, true>(x, ldx, W, ldw, bias, y, ldy, (int)N, K, n_units, stream, rc, nm)
                 : launch_gemv<2, 3, bf16_t, true>(x, ldx, W, ldw, bias, y, ldy, (int)N, K, n_units, stream, rc, nm);
  if (r) return r;
  LMSF_LAUNCH_CHECK("gemv_scaled_qkv_rope_cache");
  return 0;
}
