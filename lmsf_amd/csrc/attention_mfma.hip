// Paged attention on the matrix cores, bfloat16 storage, float32 softmax and accumulation.
//
// Two kernels over the same cache (K pages [page, kv_head, offset, d], V pages transposed
// [page, kv_head, d, offset]):
//   - "prefill": tiles of consecutive query tokens of one request, any number of tokens per tile;
//   - "decode": one query token per workgroup and split of its keys, followed by a reduction over
//     the splits.
// Both compute, per query head h with kv head h / (nh / nkv),
//   s_j = scale * <q, k_j>,  p = softmax_j(s) over lo <= j <= pos,  out = sum_j p_j v_j
// (core/src/model_executor/layers/attention.rs:91-103, :139-155;
// vllm/kernels/attention/attention_kernels.cu:82-414). The reference's decode kernel rounds p to
// the model's dtype before the product with v (:337-351); so does the matrix-core product here.
//
// Layout of the products (v_mfma_f32_16x16x32_bf16: A is 16 rows x 32 k, lane l holds row l % 16 and
// k = (l / 16) * 8 .. + 7; B is 32 k x 16 columns with the same lane pattern; D[row][col]: lane l holds
// column l % 16 and rows (l / 16) * 4 .. + 3).
//   S^T[key][row] = K[key][:] . Q[row][:]       A = 16 keys of K, B = 16 query rows, k runs over d.
//   O^T[dv][row]  = V^T[dv][key] . P^T[key][row] A = 16 output dims of V^T, B = P^T, k runs over 32 keys.
// A lane that holds column ``row`` of S^T for the keys 4g .. 4g+3 of two 16-key blocks holds exactly
// the eight k-values of P^T that the second product wants from it, if the product's k index is read as
// (block, 4g + i); V^T is fetched with the same reading. So the probabilities never leave the lane
// that computed them, and both K and V^T come straight from global memory in operand layout: K rows
// are contiguous in d, V^T rows are contiguous in the key offset.
//
// The query rows of a workgroup are (token, head of the kv group) pairs, so that the heads that
// share a kv head share its keys in registers.
#include "common.h"

#include <limits.h>
#include <math.h>

#include <type_traits>

typedef unsigned int attn_u32x2_t __attribute__((ext_vector_type(2)));
union Frag8 {
  bf16x8_t v;
  uint4 q;
  uint2 h[2];
  uint32_t w[4];
};

// Maximum over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the lanes that hold one query row's scores), with
// gfx950's row and half-wave swaps: two VALU instructions each instead of two trips through LDS.
// v_permlane16_swap exchanges the odd rows of 16 lanes of its first operand with the even rows of its
// second, v_permlane32_swap the upper half of the first with the lower half of the second; with the same
// value in both operands, the two results hold the two partners side by side.
__device__ __forceinline__ float max_over_lane_groups(float x) {
  unsigned u = __float_as_uint(x);
  auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  x = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  u = __float_as_uint(x);
  auto b = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}

__device__ __forceinline__ int wave_max_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_min_i(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}

struct KvView {
  const bf16_t* k;
  const bf16_t* v;
  const int* bt;   // block table row of the request
  int btw;         // its width
  int nkv, d, ps, kvh;
};

// Element offset of key ``key``'s row in the K pages.
__device__ __forceinline__ long k_row_offset(const KvView& G, int key) {
  int blk = key / G.ps;
  if (blk > G.btw - 1) blk = G.btw - 1;   // keys beyond the table are masked by the caller; stay inside it
  const int page = G.bt[blk];
  return ((long)(page * G.nkv + G.kvh) * G.ps + (key - (key / G.ps) * G.ps)) * G.d;
}
// Element offset of (dv = 0, key) in the transposed V pages; add dv * ps.
__device__ __forceinline__ long v_col_offset(const KvView& G, int key) {
  int blk = key / G.ps;
  if (blk > G.btw - 1) blk = G.btw - 1;
  const int page = G.bt[blk];
  return (long)(page * G.nkv + G.kvh) * G.d * G.ps + (key - (key / G.ps) * G.ps);
}

// ---------------------------------------------------------------- prefill

// One workgroup of 4 waves per (tile, kv head, block of HB heads of its group). Wave w owns the rows
// (w * NQB + j) * 16 + c, j < NQB, c = lane % 16; row r is token r / HB of the tile and head r % HB of
// the block. tiles[2 i], tiles[2 i + 1]: first flat token and number of tokens of tile i.
template <int DPAD, int NQB>
__global__ __launch_bounds__(256) void attn_prefill_mfma_kernel(
    const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long out_stride,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages, const int* __restrict__ block_tables,
    int btw, const int* __restrict__ tiles, const int* __restrict__ seg, const int* __restrict__ pos, int nh, int nkv,
    int d, int ps, float scale_log2, int window, int HB, int n_hb) {
  constexpr int DS = DPAD / 32, DV = DPAD / 16;
  const int tile = blockIdx.x;
  const int kvh = blockIdx.y / n_hb, hb = blockIdx.y - kvh * n_hb;
  const int n_rep = nh / nkv;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, c = l & 15, g = l >> 4;
  const int t0 = tiles[2 * tile], ntok = tiles[2 * tile + 1];
  KvView G;
  G.k = k_pages; G.v = v_pages; G.btw = btw; G.nkv = nkv; G.d = d; G.ps = ps; G.kvh = kvh;
  G.bt = block_tables + (long)seg[t0] * btw;

  int rpos[NQB], rlo[NQB];
  long qoff[NQB], ooff[NQB];
  int wmax = -1, wlo = INT_MAX;
#pragma unroll
  for (int j = 0; j < NQB; ++j) {
    const int row = (w * NQB + j) * 16 + c;
    const int t = row / HB, hin = hb * HB + (row - t * HB);
    const bool valid = t < ntok && hin < n_rep;
    const int tok = t0 + (valid ? t : 0);
    const int p = valid ? pos[tok] : -1;
    rpos[j] = p;
    rlo[j] = (window > 0 && p >= 0) ? max(0, p - window + 1) : 0;
    const int head = kvh * n_rep + (valid ? hin : 0);
    qoff[j] = (long)tok * q_stride + (long)head * d;
    ooff[j] = (long)tok * out_stride + (long)head * d;
    wmax = max(wmax, p);
    if (valid) wlo = min(wlo, rlo[j]);
  }
  wmax = wave_max_i(wmax);
  wlo = wave_min_i(wlo);
  if (wmax < 0) return;   // no row of this wave is in use (waves share nothing, so it may leave)

  Frag8 qf[NQB][DS];
#pragma unroll
  for (int j = 0; j < NQB; ++j)
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int d0 = s * 32 + g * 8;
      if (rpos[j] >= 0 && d0 < d)
        qf[j][s].q = *reinterpret_cast<const uint4*>(q + qoff[j] + d0);
      else
        qf[j][s].q = make_uint4(0, 0, 0, 0);
    }

  f32x4_t acc[DV][NQB];
  float m[NQB], lsum[NQB];
#pragma unroll
  for (int j = 0; j < NQB; ++j) {
    m[j] = -INFINITY;
    lsum[j] = 0.f;
#pragma unroll
    for (int v = 0; v < DV; ++v) acc[v][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }

  for (int kbase = (wlo / 32) * 32; kbase <= wmax; kbase += 32) {
    // S^T for two blocks of 16 keys
    f32x4_t st[2][NQB];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const long kr = k_row_offset(G, kbase + b * 16 + c);
      Frag8 kf[DS];
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const int d0 = s * 32 + g * 8;
        if (d0 < d)
          kf[s].q = *reinterpret_cast<const uint4*>(k_pages + kr + d0);
        else
          kf[s].q = make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int j = 0; j < NQB; ++j) {
        f32x4_t a = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < DS; ++s) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[s].v, qf[j][s].v, a, 0, 0, 0);
        st[b][j] = a;
      }
    }
    // V^T addresses of this lane's two groups of four keys (issued early, used after the softmax)
    const long vo0 = v_col_offset(G, kbase + 4 * g), vo1 = v_col_offset(G, kbase + 16 + 4 * g);
    // mask, online softmax, probabilities as the B operand of the second product
    Frag8 pf[NQB];
#pragma unroll
    for (int j = 0; j < NQB; ++j) {
      float sv[8];
      float mx = -INFINITY;
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kbase + b * 16 + g * 4 + i;
          const bool ok = key <= rpos[j] && key >= rlo[j];
          const float x = ok ? st[b][j][i] * scale_log2 : -INFINITY;
          sv[b * 4 + i] = x;
          mx = fmaxf(mx, x);
        }
      mx = max_over_lane_groups(mx);
      const float m_new = fmaxf(m[j], mx);
      const bool dead = m_new == -INFINITY;           // nothing seen yet by this row
      const float corr = (m[j] == -INFINITY) ? (dead ? 1.f : 0.f) : exp2f(m[j] - m_new);
      float ps_ = 0.f;
      float pv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        pv[e] = dead ? 0.f : exp2f(sv[e] - m_new);
        ps_ += pv[e];
      }
      lsum[j] = lsum[j] * corr + ps_;
      m[j] = m_new;
#pragma unroll
      for (int v = 0; v < DV; ++v) acc[v][j] *= corr;
      pf[j].w[0] = pack2_bf16(pv[0], pv[1]);
      pf[j].w[1] = pack2_bf16(pv[2], pv[3]);
      pf[j].w[2] = pack2_bf16(pv[4], pv[5]);
      pf[j].w[3] = pack2_bf16(pv[6], pv[7]);
    }
    // O^T += V^T P^T
#pragma unroll
    for (int v = 0; v < DV; ++v) {
      if (v * 16 < d) {
        const long dvo = (long)(v * 16 + c) * ps;
        Frag8 vf;
        vf.h[0] = *reinterpret_cast<const uint2*>(v_pages + vo0 + dvo);
        vf.h[1] = *reinterpret_cast<const uint2*>(v_pages + vo1 + dvo);
#pragma unroll
        for (int j = 0; j < NQB; ++j) acc[v][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf[j].v, acc[v][j], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int j = 0; j < NQB; ++j) {
    float ls = lsum[j];
    ls += __shfl_xor(ls, 16, 64);
    ls += __shfl_xor(ls, 32, 64);
    if (rpos[j] < 0) continue;
    const float inv = 1.0f / ls;
#pragma unroll
    for (int v = 0; v < DV; ++v) {
      const int dv = v * 16 + g * 4;
      if (dv < d) {
        uint2 o;
        o.x = pack2_bf16(acc[v][j][0] * inv, acc[v][j][1] * inv);
        o.y = pack2_bf16(acc[v][j][2] * inv, acc[v][j][3] * inv);
        *reinterpret_cast<uint2*>(out + ooff[j] + dv) = o;
      }
    }
  }
}

// The same with the keys and values staged in LDS by the workgroup and read from there by its waves (NW: eight
// of 16 rows where the transfers divide evenly among them, else four of 32 rows);
// the kernel above has every wave fetch them from global memory for itself and spends its time waiting.
// Here tiles of 32 keys travel from global memory straight into LDS (global_load_lds_dwordx4: lane i of a
// wave writes its 16 bytes at the wave's LDS base + 16 i, whatever global address it reads), STAGES - 1
// steps ahead of the one being multiplied, so that the memory latency is covered by several steps of work
// and no registers are held by data in flight. One barrier per step.
//
// A stage holds the K tile [32 keys][DPAD] and the V^T tile [DPAD][32 keys], both without padding (the
// transfer writes lane after lane). In the product K Q^T the 16 rows of block b are the keys
// 8 (r / 4) + 4 b + r % 4 and not 16 b + r: a lane's eight scores (four of each block) are then eight keys in
// a row, 8 g .. 8 g + 7, which is the order the second product wants, and a V^T fragment is one 16-byte read.
// Bank conflicts of the operand reads are avoided by choosing which piece each lane fetches: eight lanes in
// a row are served together and must differ in address bits 4 to 6. 16-byte piece ``col`` of K row ``row``
// lies in slot col xor row_lane(row) of its row, row_lane being the lane that reads the row, where a row has
// a power of two of pieces (measured: full rate; the rotation (col - row_lane) mod PR, used for the other head
// sizes, loses 40 % of the rate when two workgroups share a compute unit), piece ``p`` of V^T row ``dv`` in
// slot (p + dv / 2) mod 4. The request's block table is copied to LDS first,
// so that no address waits for a lookup in global memory. Needs pages of 8, 16, 32, ... tokens.
//
// The transfer instruction is written as inline assembly: through the compiler's builtin every LDS read
// that follows would first wait for all transfers in flight (the compiler cannot tell that they write other
// stages), which undoes the pipelining. The waits are therefore explicit: s_waitcnt vmcnt(n) before the
// barrier of each step.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"   // m0 is named as clobbered on purpose
__device__ __forceinline__ void global_to_lds_16(const void* src, unsigned lds_base_uniform) {
  // lane i's 16 bytes go to LDS address m0 + 16 i
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base_uniform)
               : "memory", "m0");
}
#pragma clang diagnostic pop
// c = lane % 16 of the lane that reads K row ``row`` (0 .. 31) of a stage; both blocks of 16 rows give 0 .. 15
__device__ __forceinline__ int row_lane(int row) { return ((row >> 3) << 2) | (row & 3); }
__device__ __forceinline__ unsigned lds_address(const void* p) {
  return (unsigned)(size_t)(__attribute__((address_space(3))) const unsigned char*)p;
}

// A step of 32 keys costs a wave 32 matrix-core instructions (512 cycles); everything else has to stay below
// that, so whatever does not change from step to step (which piece a lane moves, where it reads its
// operands in a stage) is worked out before the loop, pages are powers of two (shifts, no divisions), the
// mask is only applied in steps that touch the diagonal or the window's edge, and the accumulators are
// only rescaled when a row's maximum has moved.
// How far (in powers of two) a row's scores may rise above the reference of its exponentials before the
// accumulators are rescaled: 2^24 times a few thousand keys times the values stays far inside float32.
//
// What bounds it (measured with timestamps inside the kernel, with parts of the step taken out, and with
// counters): the matrix pipe is busy 39 percent of the time, the vector issue port 56 percent, both at once 15
// percent; a step's 32 matrix instructions a SIMD need 250 ns, the step takes 490 ns where two workgroups share a
// compute unit (8,192 tokens: 0.94 PFLOP/s) and 800 ns where one is alone. Around the matrix instructions stand,
// per 16 rows and 32 keys, 67 vector instructions (scale, exponential, sum, conversion, largest score, the
// transfers' addresses), the waits for LDS and the barrier; a v_exp_f32 never runs beside a matrix instruction (a
// fused multiply-add does: measured apart), and a wave issues one instruction at a time, so what hides these is
// other waves: eight waves of 16 rows (four on a SIMD, two of them the workgroup's own) against four waves of 32
// rows (two on a SIMD) took 13 percent off at 2,048 tokens, where the longest tile's workgroup is alone on its
// compute unit for most of its 64 steps and the kernel takes as long as that workgroup (4.4 us of set-up, 64
// steps). Tried, measured, not kept: the next step's scores multiplied beside the current step's exponentials,
// in the order fixed with scheduling groups (four waves of 32 rows: the same times within 3 percent).
// Also not kept: two groups of eight waves in a workgroup of 16, each with half of a tile's keys, put together
// through LDS at the end (the longest tile would take half the steps): 66.6 against 63.9 us at 2,048 tokens,
// 727 against 626 at 8,192; a barrier over 16 waves and one workgroup a compute unit cost more than the balance gives.
#define PREFILL_LAZY_LOG2 24.0f
// Entries of a block table that the LDS-staged kernel keeps beside its stages at a time, and how many copies of the
// table's last entry follow them there. PREFILL_BT_CAP_SMALL: a window for tests, which moves at short contexts.
#define PREFILL_BT_CAP 2048
#define PREFILL_BT_CAP_SMALL 64
#define PREFILL_BT_PAD 8
template <int DPAD, int NQB, int STAGES, int NW>
__global__ __launch_bounds__(NW * 64, (NW == 8 ? 4 : 1)) void attn_prefill_dma_kernel(
    const bf16_t* __restrict__ q, long q_stride, bf16_t* __restrict__ out, long out_stride,
    const bf16_t* __restrict__ k_pages, const bf16_t* __restrict__ v_pages, const int* __restrict__ block_tables,
    int btw, const int* __restrict__ tiles, const int* __restrict__ seg, const int* __restrict__ pos, int nh, int nkv,
    int d, int ps_log2, float scale_log2, int window, int HB, int n_hb, int bt_cap, int n_cus) {
  constexpr int DS = DPAD / 32, DV = DPAD / 16;
  constexpr int PR = DPAD / 8;                   // 16-byte pieces per K row
  constexpr bool PR_POW2 = (PR & (PR - 1)) == 0;
  constexpr int KTILE = 32 * DPAD * 2;           // bytes; the V^T tile has the same size
  constexpr int STAGE = 2 * KTILE;
  constexpr int LPW = DPAD / (8 * NW);           // transfers per wave and stage (DPAD / 8 in all)
  static_assert(LPW * 8 * NW == DPAD && NW * NQB == 8, "the waves share the transfers evenly and hold 128 rows");
  extern __shared__ __align__(16) unsigned char lds_raw[];   // [STAGES][STAGE], then the block table
  int* lds_bt = reinterpret_cast<int*>(lds_raw + STAGES * STAGE);
  // Which (tile, kv head, block of heads) this workgroup takes. The caller lists the tiles with the most keys
  // first, and workgroups start in the order of their index, so long tiles start first and short ones fill the
  // gaps. When all workgroups fit on the chip at once, two to a compute unit, what counts is which two share
  // one: workgroup n and workgroup n + n_cus do when the workgroups are placed in order, so the second n_cus take
  // the items from the light end, and the longest tile is paired with the shortest. Items of one tile differ in
  // the kv head, so that neighbours in the order (which go to different dies) read different keys and values,
  // and each die keeps to few kv heads.
  const int n_y = nkv * n_hb, n_items = gridDim.x;
  int item = blockIdx.x;
  if (n_items <= 2 * n_cus && item >= n_cus) item = n_items - 1 - (item - n_cus);
  const int tile = item / n_y, y = item - tile * n_y;
  const int kvh = y / n_hb, hb = y - kvh * n_hb;
  const int n_rep = nh / nkv;
  const int tid = threadIdx.x, w = __builtin_amdgcn_readfirstlane(tid >> 6), l = tid & 63, c = l & 15, g = l >> 4;
  const int t0 = tiles[2 * tile], ntok = tiles[2 * tile + 1];
  const int* bt = block_tables + (long)seg[t0] * btw;
  const int ps = 1 << ps_log2, pm = ps - 1;

  // the workgroup's range of keys: positions of a tile are consecutive
  const int p_first = pos[t0], p_last = p_first + ntok - 1;
  const int k_begin = window > 0 ? (max(0, p_first - window + 1) / 32) * 32 : 0;
  const int n_steps = (p_last - k_begin) / 32 + 1;
  const int blk0 = k_begin >> ps_log2;                                   // first block of the table that is needed
  const int n_blk = min(btw, (p_last >> ps_log2) + 1) - blk0;             // blocks of the table that are needed
  // LDS holds bt_cap of them at a time, from block wbase on (counted from blk0), and PREFILL_BT_PAD more: entries
  // after the table's last one repeat it, so the lookups of the steps ahead need no bound. A tile with more blocks
  // than that (a prompt's portion after tens of thousands of tokens) moves the window on as it walks the keys.
  int wbase = 0;
  for (int i = tid; i < min(n_blk, bt_cap) + PREFILL_BT_PAD; i += NW * 64) lds_bt[i] = bt[blk0 + min(i, n_blk - 1)];

  int rpos[NQB], rlo[NQB];
  long qoff[NQB], ooff[NQB];
  int wmax = -1, wlo = INT_MAX, wminpos = INT_MAX, wmaxlo = 0;
#pragma unroll
  for (int j = 0; j < NQB; ++j) {
    const int row = (w * NQB + j) * 16 + c;
    const int t = row / HB, hin = hb * HB + (row - t * HB);
    const bool valid = t < ntok && hin < n_rep;
    const int tok = t0 + (valid ? t : 0);
    const int p = valid ? p_first + t : -1;
    rpos[j] = p;
    rlo[j] = (window > 0 && p >= 0) ? max(0, p - window + 1) : 0;
    const int head = kvh * n_rep + (valid ? hin : 0);
    qoff[j] = (long)tok * q_stride + (long)head * d;
    ooff[j] = (long)tok * out_stride + (long)head * d;
    wmax = max(wmax, p);
    if (valid) {
      wlo = min(wlo, rlo[j]);
      wminpos = min(wminpos, p);
      wmaxlo = max(wmaxlo, rlo[j]);
    }
  }
  wmax = __builtin_amdgcn_readfirstlane(wave_max_i(wmax));
  wlo = __builtin_amdgcn_readfirstlane(wave_min_i(wlo));
  wminpos = __builtin_amdgcn_readfirstlane(wave_min_i(wminpos));   // a step whose keys all lie in [wmaxlo, wminpos] needs no mask
  wmaxlo = __builtin_amdgcn_readfirstlane(wave_max_i(wmaxlo));

  Frag8 qf[NQB][DS];
#pragma unroll
  for (int j = 0; j < NQB; ++j)
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int d0 = s * 32 + g * 8;
      if (rpos[j] >= 0 && d0 < d)
        qf[j][s].q = *reinterpret_cast<const uint4*>(q + qoff[j] + d0);
      else
        qf[j][s].q = make_uint4(0, 0, 0, 0);
    }

  f32x4_t acc[DV][NQB];
  // (neg_m: what is added to a scaled score before the exponential; a row that has seen nothing yet has only
  // masked keys: exp2(-inf) = 0 whatever is added)
  float m[NQB], neg_m[NQB], lsum[NQB];
#pragma unroll
  for (int j = 0; j < NQB; ++j) {
    m[j] = -INFINITY;
    neg_m[j] = 0.f;
    lsum[j] = 0.f;
#pragma unroll
    for (int v = 0; v < DV; ++v) acc[v][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  }

  // what this lane moves in every step: transfer i of the wave covers pieces j * 64 .. j * 64 + 63 of a stage,
  // j = w + NW i; the first DPAD / 16 transfers are the K tile, the others the V^T tile. A step starts at a
  // multiple of 32 keys and pages are powers of two, so a key's block and its place in the page are each a
  // part that is the same for the whole wave (from the step) plus a part that never changes (from the lane).
  const unsigned page_stride = (unsigned)(nkv * d) << ps_log2;   // elements per page, K and V alike
  int t_blk[LPW];              // the lane's part of the block index
  int t_mul[LPW];              // elements per key within a page: d for K, 1 for V^T (the same for the wave)
  const bf16_t* t_base[LPW];   // the pages plus everything of the offset that never changes
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int j = w + NW * i;
    if (j < DPAD / 16) {
      const int P = j * 64 + l;
      const int row = P / PR, slot = P - row * PR;
      const int rz = PR == 4 ? (row_lane(row) >> 1) & 3 : row_lane(row);
      int col;
      if (PR_POW2) {
        col = slot ^ (rz & (PR - 1));
      } else {
        col = slot + rz % PR;
        if (col >= PR) col -= PR;
      }
      if (col * 8 >= d) col = 0;                   // beyond the head: any finite data, the query is zero there
      t_blk[i] = row >> ps_log2;
      t_mul[i] = d;
      t_base[i] = k_pages + (((long)kvh * d << ps_log2) + col * 8 + (long)(row & pm) * d);
    } else {
      const int P = (j - DPAD / 16) * 64 + l;
      int dv = P >> 2;
      const int slot = P & 3;
      const int piece = (slot - (dv >> 1)) & 3;
      if (dv >= d) dv = 0;                         // rows beyond the head: any finite data, their results are dropped
      t_blk[i] = (piece * 8) >> ps_log2;
      t_mul[i] = 1;
      t_base[i] = v_pages + (((long)(kvh * d + dv) << ps_log2) + ((piece * 8) & pm));
    }
  }
  // where this lane reads its operands in a stage (bytes)
  int koff[2][DS];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int s = 0; s < DS; ++s) {
      const int row = (c >> 2) * 8 + b * 4 + (c & 3);   // row_lane(row) == c
      const int rz = PR == 4 ? (c >> 1) & 3 : c;
      int slot;
      if (PR_POW2) {
        slot = (s * 4 + g) ^ (rz & (PR - 1));
      } else {
        slot = s * 4 + g - rz % PR;
        if (slot < 0) slot += PR;
      }
      koff[b][s] = (row * PR + slot) * 16;
    }
  const int voff = KTILE + c * 64 + ((g + (c >> 1)) & 3) * 16;   // piece g of V^T row 16 v + c

  // The query fragments are pinned here, so that the compiler waits for their loads now and not, with a
  // wait for everything in flight, inside the loop.
#pragma unroll
  for (int j = 0; j < NQB; ++j)
#pragma unroll
    for (int s = 0; s < DS; ++s) asm volatile("" : "+v"(qf[j][s].v));
  __syncthreads();   // the block table is in LDS

  // The pages of this lane's transfers are looked up one step before the transfers are issued, so that the
  // way to LDS and back is over by then (looked up where they are needed, the four lookups of a step cost a
  // wave that runs alone on its SIMD a tenth of the step).
  int page_of[LPW];
  auto lookup = [&](int kb) {
    const int blk_step = min((kb >> ps_log2) - blk0, n_blk) - wbase;   // the step's part, the same for the wave
#pragma unroll
    for (int i = 0; i < LPW; ++i)
      page_of[i] = lds_bt[blk_step + t_blk[i]];               // keys beyond the last block are masked: any valid page
  };
  // this wave's transfers of the step that starts at key kb, into the stage at byte ``stage_byte``
  auto issue = [&](int kb, int stage_byte) {
    const int in_page = kb & pm;
#pragma unroll
    for (int i = 0; i < LPW; ++i) {
      const unsigned long long off = (unsigned long long)(unsigned)page_of[i] * page_stride + (unsigned)(in_page * t_mul[i]);
      global_to_lds_16(t_base[i] + off, __builtin_amdgcn_readfirstlane(lds_address(lds_raw) + stage_byte +
                                                                       (w + NW * i) * 1024));
    }
  };

#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < n_steps) {
      lookup(k_begin + s * 32);
      issue(k_begin + s * 32, s * STAGE);
    }
  lookup(k_begin + (STAGES - 1) * 32);

  // One step; SI: which stage holds it (a constant, so that the places of the operands in LDS are constants in
  // the instructions and cost no additions).
  auto step = [&](auto SI, int it) {
    constexpr int consume = decltype(SI)::value * STAGE;                                  // the stage read now
    constexpr int produce = ((decltype(SI)::value + STAGES - 1) % STAGES) * STAGE;       // the stage filled now
    const int kbase = k_begin + it * 32;
    // step ``it`` has arrived when at most the transfers of the later steps are outstanding
    if (it + STAGES - 2 < n_steps)
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * LPW) : "memory");
    else
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();   // everybody's part of step ``it`` is there, and everybody is done with step ``it - 1``
    if (it + STAGES - 1 < n_steps) {
      issue(kbase + (STAGES - 1) * 32, produce);
      // The window of the table moves on when the next lookup would leave it (the same for the whole workgroup).
      // Nobody reads the table between this step's barrier and the one below: the lookups of the step before
      // are done, this step's follow.
      const int next_blk = min(((kbase + STAGES * 32) >> ps_log2) - blk0, n_blk);
      if (next_blk - wbase >= bt_cap) {
        wbase = next_blk;
        for (int i = tid; i < bt_cap + PREFILL_BT_PAD; i += NW * 64) lds_bt[i] = bt[blk0 + min(wbase + i, n_blk - 1)];
        __syncthreads();
      }
      lookup(kbase + STAGES * 32);
    }
    if (kbase <= wmax && kbase + 31 >= wlo) {
      const unsigned char* st_base = lds_raw + consume;
      // 2 * NQB sums that do not depend on each other, one matrix instruction of each in turn: none waits for
      // the one before it
      f32x4_t st[2][NQB];
      Frag8 kf[2][DS];
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int s = 0; s < DS; ++s) kf[b][s].q = *reinterpret_cast<const uint4*>(st_base + koff[b][s]);
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int j = 0; j < NQB; ++j) st[b][j] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DS; ++s)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int j = 0; j < NQB; ++j)
            st[b][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b][s].v, qf[j][s].v, st[b][j], 0, 0, 0);
      // the V^T fragments are asked for now and used after the softmax, which covers their way from LDS
      Frag8 vf[DV];
#pragma unroll
      for (int v = 0; v < DV; ++v) {
        vf[v].q = *reinterpret_cast<const uint4*>(st_base + voff + v * 1024);
      }
      const bool need_mask = kbase + 31 > wminpos || kbase < wmaxlo;   // the same for the whole wave
      Frag8 pf[NQB];
#pragma unroll
      for (int j = 0; j < NQB; ++j) {
        float r[8];
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int i = 0; i < 4; ++i) r[b * 4 + i] = st[b][j][i];
        if (need_mask) {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int key = kbase + g * 8 + e;
            if (key > rpos[j] || key < rlo[j]) r[e] = -INFINITY;
          }
        }
        const float mx = fmaxf(fmaxf(fmaxf(r[0], r[1]), fmaxf(r[2], r[3])), fmaxf(fmaxf(r[4], r[5]), fmaxf(r[6], r[7])));
        // m is the reference the exponentials are taken against, not the running maximum: any reference gives
        // the same softmax as long as nothing overflows, and bfloat16 probabilities and float32 sums have room
        // for 2^LAZY above it. So the accumulators (which the matrix cores hold where other instructions cannot
        // reach them without copies) are rescaled only when a row's scores rise that far above its reference,
        // which after a row's first step happens almost never. The four lanes that hold a row's scores need
        // the same reference, so the row's largest score is taken over them, but only where one of them has
        // found a score that far up.
        if (__builtin_expect(__any(mx * scale_log2 > m[j] + PREFILL_LAZY_LOG2), 0)) {   // the scale is positive
          const float cand = max_over_lane_groups(mx) * scale_log2;
          const float m_new = cand > m[j] + PREFILL_LAZY_LOG2 ? cand : m[j];
          const float corr = (m[j] == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m[j] - m_new);   // nothing summed yet: keep
          lsum[j] *= corr;
#pragma unroll
          for (int v = 0; v < DV; ++v) acc[v][j] *= corr;
          m[j] = m_new;
          neg_m[j] = (m_new == -INFINITY) ? 0.f : -m_new;
        }
        float pv[8], ps_ = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          pv[e] = __builtin_amdgcn_exp2f(fmaf(r[e], scale_log2, neg_m[j]));
          ps_ += pv[e];
        }
        lsum[j] += ps_;
        pf[j].w[0] = pack2_bf16(pv[0], pv[1]);
        pf[j].w[1] = pack2_bf16(pv[2], pv[3]);
        pf[j].w[2] = pack2_bf16(pv[4], pv[5]);
        pf[j].w[3] = pack2_bf16(pv[6], pv[7]);
      }
#pragma unroll
      for (int v = 0; v < DV; ++v)
#pragma unroll
        for (int j = 0; j < NQB; ++j) acc[v][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[v].v, pf[j].v, acc[v][j], 0, 0, 0);
    }
  };
  for (int it = 0; it < n_steps; it += STAGES) {
    step(std::integral_constant<int, 0>(), it);
    if (it + 1 < n_steps) step(std::integral_constant<int, 1>(), it + 1);
    if (it + 2 < n_steps) step(std::integral_constant<int, 2>(), it + 2);
    if constexpr (STAGES == 4)
      if (it + 3 < n_steps) step(std::integral_constant<int, 3>(), it + 3);
  }

#pragma unroll
  for (int j = 0; j < NQB; ++j) {
    float ls = lsum[j];
    ls += __shfl_xor(ls, 16, 64);
    ls += __shfl_xor(ls, 32, 64);
    if (rpos[j] < 0) continue;
    const float inv = 1.0f / ls;
#pragma unroll
    for (int v = 0; v < DV; ++v) {
      const int dv = v * 16 + g * 4;
      if (dv < d) {
        uint2 o;
        o.x = pack2_bf16(acc[v][j][0] * inv, acc[v][j][1] * inv);
        o.y = pack2_bf16(acc[v][j][2] * inv, acc[v][j][3] * inv);
        *reinterpret_cast<uint2*>(out + ooff[j] + dv) = o;
      }
    }
  }
}


template <int DPAD>
static int launch_prefill_dma(dim3 grid, hipStream_t stream, const bf16_t* q, long q_stride, bf16_t* out,
                              long out_stride, const bf16_t* k_pages, const bf16_t* v_pages, const int* block_tables,
                              int btw, const int* tiles, const int* seg, const int* pos, int nh, int nkv, int d, int ps,
                              float scale_log2, int window, int HB, int n_hb, int bt_cap) {
  int ps_log2 = 0;
  while ((1 << ps_log2) < ps) ++ps_log2;
  // four stages of a head size of 128 and the table are 72 KB: two workgroups share a compute unit's LDS,
  // and one's softmax runs beside the other's matrix products
  constexpr int STAGES = DPAD <= 128 ? 4 : 3;
  // Eight waves of 16 rows each where the transfers divide evenly among them (head sizes of 64 and 128), else
  // four waves of 32 rows: the workgroup of a long tile that is alone on its compute unit then still has two
  // waves on every SIMD, which hide each other's waits.
  constexpr int NW = (DPAD == 64 || DPAD == 128) ? 8 : 4;
  const size_t smem = (size_t)STAGES * 4 * 32 * DPAD + (PREFILL_BT_CAP + PREFILL_BT_PAD) * sizeof(int);
  auto kernel = attn_prefill_dma_kernel<DPAD, 8 / NW, STAGES, NW>;
  static bool configured = false;   // per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("paged_attention_prefill: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  hipLaunchKernelGGL(kernel, dim3(grid.x * grid.y), dim3(NW * 64), smem, stream, q, q_stride, out, out_stride, k_pages,
                     v_pages, block_tables, btw, tiles, seg, pos, nh, nkv, d, ps_log2, scale_log2, window, HB, n_hb,
                     bt_cap, lmsf_compute_units());
  return 0;
}

// ---------------------------------------------------------------- decode

// One workgroup of 4 waves per (query token, kv head and block of up to 16 heads of its group, split).
// Split s covers the keys [s * chunk, (s + 1) * chunk); wave w takes the 32-key steps w, w + 4, ... of it.
// The waves' results are merged through LDS and written as a partial result
//   part_o[((i * nh + head) * n_splits + s) * d + dv]  (not normalised),
//   part_ml[((i * nh + head) * n_splits + s) * 2 + {0, 1}] = (running maximum in log2 units, sum),
// i being the index of the token in this launch. A split without keys writes nothing; the reduction
// knows from the position which splits have keys. With n_splits == 1 there is nothing to reduce and the
// workgroup writes out[tok, head, :] itself.
// (Tried instead of the reduction kernel: the workgroup that finishes last, found by a counter per (token, kv
// head), adds the partial results up. With release and acquire fences at device scope a launch took 25 us
// longer: each fence writes back or drops what the die's L2 holds. With stores and loads at device scope and a
// wait for the stores' acknowledgement instead of the fences, the three trips to memory in a row (results,
// counter, results) cost what the second kernel's start costs: 10.8 against 9.9 us at 8 tokens of 585 keys, 12.5
// against 13.8 at 1,024 keys, 18 against 23 at one token of 8,000 keys in 16 splits. Not kept. Nor were
// workgroups of 16 waves that take a context's keys unsplit and need no second kernel: 26.8 against 12.6 us at 8
// tokens of 585 keys, with keys and values that come from memory; one compute unit pulls a context's 300 KB far
// slower than eight do. Nor a dealing of a step's 32 keys that makes a lane's eight scores eight keys in a row, as
// the prefill kernel has it, so that their values are one 16-byte load from one page instead of two of 8 bytes
// from two: 35.5 against 37 us at 64 tokens of 585 keys, but 68 against 63.7 at 128 and 222 against 217 at 64
// tokens of 1,150 keys with 32 kv heads. Nor two sets of fragments a wave, the next step's keys and values asked for
// before this step is multiplied (the table's entries for the step after asked for first, since loads come back in
// the order they were asked for): the same times at 64 and 128 tokens and at 8,000 keys, so it is not a wave's
// waiting for its own loads that bounds the kernel at 4.4 to 4.9 TB/s there. Nor a form for steps of single tokens
// that takes the unrotated QKV product (finished, or as the partial sums of a product that splits K), rotates its
// queries itself and has the one wave whose keys include the token's own make, store and use that key and value
// from its registers, so that no rotation kernel runs between product and attention: the same bits, but at 64
// tokens of 585 keys 38.6 us from partial sums and 33.4 from a finished product against 27.2 + 5.4 for the two
// kernels, at 128 tokens 77 and 66 against 51.6 + 6.3. With the chip's queues full of keys and values a trip to
// memory takes about 5 us, and the trips that position -> table and product -> rotation add before the first
// score, and slot -> key and value for the owning wave, cost more than the launch they save: 4 us for the queries
// alone, 7 for the token's own key and value, nothing for the stores.)
// FULL: the head size is DPAD itself (a multiple of 32); the loads and products of a step then run without a test
// each for the part of DPAD beyond the head size (8 tokens of 585 keys: 12.3 -> 11.6 us with the reduction).
// ROW8: a step's 32 keys are dealt so that a lane's eight scores are eight keys in a row (row c of score block b is
// key 8 (c / 4) + 4 b + c % 4, as in the prefill kernel), and their values are one 16-byte load. For pages of 32
// tokens and more, where the two 8-byte loads of the other dealing each take half of what a row of the transposed
// V page holds and every line is asked for twice: continuous batching at 32 kv heads with pages of 32 tokens 3,580 ->
// 3,710 generated tokens/s (pages of 16: 3,830), with pages of 64 3,030 -> 3,290; 8 tokens of 8,000 keys at 8 kv heads
// with pages of 64 1,520 -> 1,770 tokens/s. Pages of 8 and 16 tokens stay with the other dealing (measured above).
template <int DPAD, bool FULL, bool ROW8>
__global__ __launch_bounds__(256) void attn_decode_mfma_kernel(
    const bf16_t* __restrict__ q, long q_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ v_pages, const int* __restrict__ block_tables, int btw,
    const int* __restrict__ tok_idx, const int* __restrict__ seg, const int* __restrict__ pos, int nh, int nkv, int d,
    int ps, float scale_log2, int window, int HB, int n_hb, int chunk, int n_splits, float* __restrict__ part_o,
    float* __restrict__ part_ml, bf16_t* __restrict__ out, long out_stride, int heads_first) {
  constexpr int DS = DPAD / 32, DV = DPAD / 16;
  extern __shared__ float lds_f[];
  // (heads_first: the heads of a token are started together, the tokens in the order of tok_idx, so that a
  // caller that lists the longest contexts first has the workgroups with the most steps start first; otherwise
  // the tokens of a head are started together, which is a little faster where all workgroups fit on the chip)
  const int i_tok = heads_first ? blockIdx.y : blockIdx.x;
  const int by = heads_first ? blockIdx.x : blockIdx.y;
  const int tok = tok_idx ? tok_idx[i_tok] : i_tok;
  const int kvh = by / n_hb, hb = by - kvh * n_hb;
  const int split = blockIdx.z;
  const int n_rep = nh / nkv;
  const int tid = threadIdx.x, w = tid >> 6, l = tid & 63, c = l & 15, g = l >> 4;
  const int p = pos[tok];
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int c0 = max(split * chunk, (lo / 32) * 32), c1 = min((split + 1) * chunk, p + 1);   // keys [c0, c1)
  if (c0 >= c1) return;
  KvView G;
  G.k = k_pages; G.v = v_pages; G.btw = btw; G.nkv = nkv; G.d = d; G.ps = ps; G.kvh = kvh;
  G.bt = block_tables + (long)(seg ? seg[tok] : tok) * btw;   // (no seg: token i is request i, one trip to memory fewer)

  const int hin = hb * HB + c;
  const bool valid = c < HB && hin < n_rep;
  const int head = kvh * n_rep + (valid ? hin : 0);
  Frag8 qf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    const int d0 = s * 32 + g * 8;
    if (valid && d0 < d)
      qf[s].q = *reinterpret_cast<const uint4*>(q + (long)tok * q_stride + (long)head * d + d0);
    else
      qf[s].q = make_uint4(0, 0, 0, 0);
  }
  f32x4_t acc[DV];
#pragma unroll
  for (int v = 0; v < DV; ++v) acc[v] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, lsum = 0.f;

  // The pages of a step's keys are looked up one step ahead (four entries of the block table a lane: the two
  // blocks of 16 keys whose rows it fetches, the two groups of four keys whose values it fetches), so that the
  // keys' addresses do not wait for a trip to the table.
  const int klast = c1 - 1;
  auto page_of = [&](int key) {
    // keys beyond the range are masked below; their addresses stay inside the pages that the range has
    return G.bt[min(key, klast) / G.ps];
  };
  auto k_at = [&](int page, int key) { return ((long)(page * G.nkv + G.kvh) * G.ps + (key - (key / G.ps) * G.ps)) * G.d; };
  auto v_at = [&](int page, int key) { return (long)(page * G.nkv + G.kvh) * G.d * G.ps + (key - (key / G.ps) * G.ps); };
  auto lookup = [&](int kb, int* out) {
    if (ROW8) {
      // a group of eight keys lies in one page (pages of a multiple of 8 tokens): one entry for both blocks' rows,
      // one for the values
      out[0] = out[1] = page_of(kb + 8 * (c >> 2) + (c & 3));
      out[2] = out[3] = page_of(kb + 8 * g);
    } else {
      out[0] = page_of(kb + c); out[1] = page_of(kb + 16 + c); out[2] = page_of(kb + 4 * g); out[3] = page_of(kb + 16 + 4 * g);
    }
  };
  // the keys and values of one step of 32 keys, as the matrix instructions take them
  auto fetch = [&](Frag8 (&kf)[2][DS], Frag8 (&vf)[DV], const int* pg, int kbase) {
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const long kr = k_at(pg[b], ROW8 ? kbase + 8 * (c >> 2) + 4 * b + (c & 3) : kbase + b * 16 + c);
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        const int d0 = s * 32 + g * 8;
        if (FULL || d0 < d)
          kf[b][s].v = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(k_pages + kr + d0));
        else
          kf[b][s].q = make_uint4(0, 0, 0, 0);
      }
    }
    const long vo0 = v_at(pg[2], ROW8 ? kbase + 8 * g : kbase + 4 * g), vo1 = v_at(pg[3], kbase + 16 + 4 * g);
#pragma unroll
    for (int v = 0; v < DV; ++v) {
      if (FULL || v * 16 < d) {
        const long dvo = (long)(v * 16 + c) * ps;
        if (ROW8) {
          vf[v].v = __builtin_nontemporal_load(reinterpret_cast<const bf16x8_t*>(v_pages + vo0 + dvo));
          continue;
        }
        // (a step's keys and values are read once by the launch: marked non-temporal)
        const attn_u32x2_t lo2 = __builtin_nontemporal_load(reinterpret_cast<const attn_u32x2_t*>(v_pages + vo0 + dvo));
        const attn_u32x2_t hi2 = __builtin_nontemporal_load(reinterpret_cast<const attn_u32x2_t*>(v_pages + vo1 + dvo));
        vf[v].w[0] = lo2.x; vf[v].w[1] = lo2.y; vf[v].w[2] = hi2.x; vf[v].w[3] = hi2.y;
      }
    }
  };
  auto compute = [&](Frag8 (&kf)[2][DS], Frag8 (&vf)[DV], int kbase) {
    float sv[8];
    float mx = -INFINITY;
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      f32x4_t a = (f32x4_t){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DS; ++s) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[b][s].v, qf[s].v, a, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = ROW8 ? kbase + 8 * g + 4 * b + i : kbase + b * 16 + g * 4 + i;
        const bool ok = valid && key <= p && key >= lo && key < c1;
        const float x = ok ? a[i] * scale_log2 : -INFINITY;
        sv[b * 4 + i] = x;
        mx = fmaxf(mx, x);
      }
    }
    mx = max_over_lane_groups(mx);
    const float m_new = fmaxf(m, mx);
    const bool dead = m_new == -INFINITY;
    const float corr = (m == -INFINITY) ? (dead ? 1.f : 0.f) : exp2f(m - m_new);
    float pv[8], ps_ = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      pv[e] = dead ? 0.f : exp2f(sv[e] - m_new);
      ps_ += pv[e];
    }
    lsum = lsum * corr + ps_;
    m = m_new;
    Frag8 pf;
    pf.w[0] = pack2_bf16(pv[0], pv[1]);
    pf.w[1] = pack2_bf16(pv[2], pv[3]);
    pf.w[2] = pack2_bf16(pv[4], pv[5]);
    pf.w[3] = pack2_bf16(pv[6], pv[7]);
#pragma unroll
    for (int v = 0; v < DV; ++v) {
      if (FULL || v * 16 < d) {
        acc[v] *= corr;
        acc[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[v].v, pf.v, acc[v], 0, 0, 0);
      }
    }
  };
  int pg[4];
  lookup(c0 + w * 32, pg);
  for (int kbase = c0 + w * 32; kbase < c1; kbase += 128) {
    int pg_next[4] = {pg[0], pg[1], pg[2], pg[3]};
    if (kbase + 128 < c1) lookup(kbase + 128, pg_next);
    Frag8 kf[2][DS], vf[DV];
    fetch(kf, vf, pg, kbase);
    compute(kf, vf, kbase);
#pragma unroll
    for (int i = 0; i < 4; ++i) pg[i] = pg_next[i];
  }
  lsum += __shfl_xor(lsum, 16, 64);
  lsum += __shfl_xor(lsum, 32, 64);

  // merge the four waves: lds_o[w][row c][dv], lds_m[w][c], lds_l[w][c]
  float* lds_o = lds_f;                       // 4 * 16 * (DPAD + 4)
  float* lds_m = lds_o + 4 * 16 * (DPAD + 4);
  float* lds_l = lds_m + 64;
#pragma unroll
  for (int v = 0; v < DV; ++v)
    *reinterpret_cast<f32x4_t*>(lds_o + (w * 16 + c) * (DPAD + 4) + v * 16 + g * 4) = acc[v];
  if (g == 0) {
    lds_m[w * 16 + c] = m;
    lds_l[w * 16 + c] = lsum;
  }
  __syncthreads();
  const int rows = min(HB, n_rep - hb * HB);
  for (int e = tid; e < rows * d; e += 256) {
    const int r = e / d, dv = e - r * d;
    float M = lds_m[r];
#pragma unroll
    for (int ww = 1; ww < 4; ++ww) M = fmaxf(M, lds_m[ww * 16 + r]);
    float o = 0.f, ls = 0.f;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) {
      const float mw = lds_m[ww * 16 + r];
      const float f = (mw == -INFINITY) ? 0.f : exp2f(mw - M);
      o += f * lds_o[(ww * 16 + r) * (DPAD + 4) + dv];
      ls += f * lds_l[ww * 16 + r];
    }
    const int hd = kvh * n_rep + hb * HB + r;
    if (n_splits == 1) {
      out[(long)tok * out_stride + (long)hd * d + dv] = f32_to_bf16(o / ls);
      continue;
    }
    const long slot = ((long)i_tok * nh + hd) * n_splits + split;
    part_o[slot * d + dv] = o;
    if (dv == 0) {
      part_ml[slot * 2] = M;
      part_ml[slot * 2 + 1] = ls;
    }
  }
}

// out[tok, head, :] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s over the splits that have keys.
// One workgroup of 256 threads per (token, head): d / 4 lanes hold four output elements each, and the
// 256 / (d / 4) groups of such lanes take every G-th split, so that the loads of many splits are in flight at
// once (with 64 splits a single loop over them costs more than the attention itself); the groups' sums are
// added in a fixed order.
#define REDUCE_THREADS 256
#define REDUCE_SERIAL_SPLITS 16   // up to this many splits a thread per output element that loops over them is faster
__global__ __launch_bounds__(256) void attn_decode_reduce_serial_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, bf16_t* __restrict__ out, long out_stride,
    const int* __restrict__ tok_idx, const int* __restrict__ pos, int nh, int d, int window, int chunk, int n_splits) {
  // One thread per output element (the block has at least d threads). Everything a thread needs is asked for at
  // once, the position beside the partial results of all splits (those of splits without keys hold whatever the
  // memory held and are dropped unread): one trip to memory before the sums instead of three in a row.
  const int i_tok = blockIdx.x, head = blockIdx.y, dv = threadIdx.x;
  const int tok = tok_idx ? tok_idx[i_tok] : i_tok;
  const int p = pos[tok];
  const long base = ((long)i_tok * nh + head) * n_splits;
  float pm[REDUCE_SERIAL_SPLITS], pl[REDUCE_SERIAL_SPLITS], po[REDUCE_SERIAL_SPLITS];
#pragma unroll
  for (int s = 0; s < REDUCE_SERIAL_SPLITS; ++s) {
    if (s < n_splits) {
      const float2 ml = *reinterpret_cast<const float2*>(part_ml + (base + s) * 2);
      pm[s] = ml.x;
      pl[s] = ml.y;
      po[s] = dv < d ? part_o[(base + s) * d + dv] : 0.f;
    }
  }
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int s0 = ((lo / 32) * 32) / chunk, s1 = min(n_splits - 1, p / chunk);   // splits s0 .. s1 have keys
  float M = -INFINITY;
#pragma unroll
  for (int s = 0; s < REDUCE_SERIAL_SPLITS; ++s)
    if (s >= s0 && s <= s1) M = fmaxf(M, pm[s]);
  float ls = 0.f, o = 0.f;
#pragma unroll
  for (int s = 0; s < REDUCE_SERIAL_SPLITS; ++s) {
    if (s >= s0 && s <= s1) {
      const float f = exp2f(pm[s] - M);
      ls += f * pl[s];
      o += f * po[s];
    }
  }
  if (dv < d) out[(long)tok * out_stride + (long)head * d + dv] = f32_to_bf16(o * (1.0f / ls));
}

__global__ __launch_bounds__(REDUCE_THREADS) void attn_decode_reduce_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, bf16_t* __restrict__ out, long out_stride,
    const int* __restrict__ tok_idx, const int* __restrict__ pos, int nh, int d, int window, int chunk, int n_splits) {
  __shared__ float red_max[REDUCE_THREADS / 64];
  __shared__ __align__(16) float red_o[REDUCE_THREADS * 4];   // [G][d], G * d <= 1024
  __shared__ float red_l[REDUCE_THREADS];
  const int i_tok = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int tok = tok_idx ? tok_idx[i_tok] : i_tok;
  const int p = pos[tok];
  const int lo = window > 0 ? max(0, p - window + 1) : 0;
  const int s0 = ((lo / 32) * 32) / chunk, s1 = min(n_splits - 1, p / chunk);   // splits s0 .. s1 have keys
  const long base = ((long)i_tok * nh + head) * n_splits;
  float M = -INFINITY;
  for (int s = s0 + tid; s <= s1; s += REDUCE_THREADS) M = fmaxf(M, part_ml[(base + s) * 2]);
  M = wave_max(M);
  if ((tid & 63) == 0) red_max[tid >> 6] = M;
  __syncthreads();
  M = fmaxf(fmaxf(red_max[0], red_max[1]), fmaxf(red_max[2], red_max[3]));
  const int L = d / 4, G = REDUCE_THREADS / L;   // d is a multiple of 16, at most 256: G >= 4
  const int g = tid / L, lane = tid - g * L;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  float ls = 0.f;
  if (g < G) {
#pragma unroll 4
    for (int s = s0 + g; s <= s1; s += G) {
      const float2 ml = *reinterpret_cast<const float2*>(part_ml + (base + s) * 2);
      const float4 o = *reinterpret_cast<const float4*>(part_o + (base + s) * d + lane * 4);
      const float w = exp2f(ml.x - M);
      ls += w * ml.y;
      acc.x += w * o.x; acc.y += w * o.y; acc.z += w * o.z; acc.w += w * o.w;
    }
    *reinterpret_cast<float4*>(red_o + (g * d + lane * 4)) = acc;
    if (lane == 0) red_l[g] = ls;
  }
  __syncthreads();
  if (g == 0) {
    for (int gg = 1; gg < G; ++gg) {
      const float4 o = *reinterpret_cast<const float4*>(red_o + (gg * d + lane * 4));
      acc.x += o.x; acc.y += o.y; acc.z += o.z; acc.w += o.w;
      ls += red_l[gg];
    }
    const float inv = 1.0f / ls;
    uint2 packed;
    packed.x = pack2_bf16(acc.x * inv, acc.y * inv);
    packed.y = pack2_bf16(acc.z * inv, acc.w * inv);
    *reinterpret_cast<uint2*>(out + (long)tok * out_stride + (long)head * d + lane * 4) = packed;
  }
}

// ---------------------------------------------------------------- entry points

static int check_common(const char* who, const void* q, const void* out, const void* k_pages, const void* v_pages,
                        const int* block_tables, const int* seg, const int* pos, long q_stride, long out_stride,
                        long num_pages, int btw, int nh, int nkv, int d, int ps, int window) {
  LMSF_CHECK(q && out && k_pages && v_pages && block_tables && seg && pos, "%s: null pointer", who);
  LMSF_CHECK(nh > 0 && nkv > 0 && nh % nkv == 0, "%s: heads %d not a multiple of kv heads %d", who, nh, nkv);
  LMSF_CHECK(d >= 16 && d % 16 == 0 && d <= 256, "%s: head size %d not supported (multiples of 16 up to 256)", who, d);
  LMSF_CHECK(ps > 0 && ps % 4 == 0, "%s: page size %d not supported (multiples of 4)", who, ps);
  LMSF_CHECK(btw > 0 && num_pages > 0, "%s: bad page geometry", who);
  LMSF_CHECK(num_pages * nkv * (long)ps * d < 2147483647L * 64, "%s: cache too large", who);
  LMSF_CHECK(num_pages * nkv < 2147483647L / 2, "%s: too many pages for 32-bit page arithmetic", who);
  LMSF_CHECK(q_stride >= (long)nh * d && out_stride >= (long)nh * d && q_stride % 8 == 0 && out_stride % 4 == 0,
             "%s: row strides must cover nh*d and keep 16-byte (q) and 8-byte (out) alignment", who);
  LMSF_CHECK(lmsf_aligned16(q) && lmsf_aligned16(k_pages) && lmsf_aligned16(v_pages) && lmsf_aligned16(out),
             "%s: operands must be 16-byte aligned", who);
  LMSF_CHECK(window >= 0, "%s: negative window", who);
  return 0;
}

static inline int heads_per_block(int n_rep) { return n_rep < 16 ? n_rep : 16; }

// Rows of query (token, head) pairs a prefill workgroup holds; a tile may have at most
// lmsf_attention_tile_tokens(nh, nkv) tokens.
#define PREFILL_NQB 2
#define PREFILL_ROWS (4 * PREFILL_NQB * 16)

extern "C" int lmsf_attention_tile_tokens(int nh, int nkv) {
  if (nh <= 0 || nkv <= 0 || nh % nkv) return 0;
  return PREFILL_ROWS / heads_per_block(nh / nkv);
}

// tiles: int32 [n_tiles, 2] = (first flat token, number of tokens <= lmsf_attention_tile_tokens); all tokens
// of a tile belong to one request and stand at consecutive positions. variant 0: keys and values staged in
// LDS where the page size allows it (the default); 1: every wave fetches them itself; 2: as 0 with a window of 64
// entries of the block table in LDS instead of 2,048, so that it moves at contexts that a test can afford.
extern "C" int lmsf_paged_attention_prefill_mfma(const void* q, long q_stride, void* out, long out_stride,
                                                 const void* k_pages, const void* v_pages, long num_pages,
                                                 const int* block_tables, int btw, const int* tiles, int n_tiles,
                                                 const int* seg, const int* pos, int nh, int nkv, int d, int ps,
                                                 float scale, int window, int variant, hipStream_t stream) {
  if (int rc = check_common("paged_attention_prefill", q, out, k_pages, v_pages, block_tables, seg, pos, q_stride,
                            out_stride, num_pages, btw, nh, nkv, d, ps, window))
    return rc;
  LMSF_CHECK(tiles != nullptr && n_tiles >= 0, "paged_attention_prefill: bad tile list");
  LMSF_CHECK(scale > 0.f, "paged_attention_prefill: the scale must be positive, got %g", (double)scale);
  if (n_tiles == 0) return 0;
  const int n_rep = nh / nkv, HB = heads_per_block(n_rep), n_hb = (n_rep + HB - 1) / HB;
  LMSF_CHECK((long)nkv * n_hb <= 65535, "paged_attention_prefill: too many kv heads");
  const float scale_log2 = scale * 1.44269504088896340736f;
  dim3 grid(n_tiles, nkv * n_hb), block(256);
  const int dpad = (d + 31) / 32 * 32;
  if ((variant == 0 || variant == 2) && ps >= 8 && (ps & (ps - 1)) == 0) {
    // tiles staged in LDS
    const int bt_cap = variant == 2 ? PREFILL_BT_CAP_SMALL : PREFILL_BT_CAP;
    int rc = 0;
#define LAUNCH_LDS(DP)                                                                                           \
  rc = launch_prefill_dma<DP>(grid, stream, (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride,                \
                              (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_tables, btw, tiles, seg, pos, \
                              nh, nkv, d, ps, scale_log2, window, HB, n_hb, bt_cap)
    switch (dpad) {
      case 32: LAUNCH_LDS(32); break;
      case 64: LAUNCH_LDS(64); break;
      case 96: LAUNCH_LDS(96); break;
      case 128: LAUNCH_LDS(128); break;
      case 160: LAUNCH_LDS(160); break;
      case 192: LAUNCH_LDS(192); break;
      case 224: LAUNCH_LDS(224); break;
      default: LAUNCH_LDS(256); break;
    }
#undef LAUNCH_LDS
    if (rc) return rc;
    LMSF_LAUNCH_CHECK("paged_attention_prefill");
    return 0;
  }
#define LAUNCH(DP)                                                                                                  \
  hipLaunchKernelGGL((attn_prefill_mfma_kernel<DP, PREFILL_NQB>), grid, block, 0, stream, (const bf16_t*)q, q_stride, \
                     (bf16_t*)out, out_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_tables, btw,   \
                     tiles, seg, pos, nh, nkv, d, ps, scale_log2, window, HB, n_hb)
  switch (dpad) {
    case 32: LAUNCH(32); break;
    case 64: LAUNCH(64); break;
    case 96: LAUNCH(96); break;
    case 128: LAUNCH(128); break;
    case 160: LAUNCH(160); break;
    case 192: LAUNCH(192); break;
    case 224: LAUNCH(224); break;
    default: LAUNCH(256); break;
  }
#undef LAUNCH
  LMSF_LAUNCH_CHECK("paged_attention_prefill");
  return 0;
}

template <int DPAD, bool FULL, bool ROW8>
static int launch_decode(dim3 grid, hipStream_t stream, const bf16_t* q, long q_stride, const bf16_t* k_pages,
                         const bf16_t* v_pages, const int* block_tables, int btw, const int* tok_idx, const int* seg,
                         const int* pos, int nh, int nkv, int d, int ps, float scale_log2, int window, int HB, int n_hb,
                         int chunk, int n_splits, float* part_o, float* part_ml, bf16_t* out, long out_stride,
                         int heads_first) {
  const size_t smem = (size_t)(4 * 16 * (DPAD + 4) + 128) * sizeof(float);
  auto kernel = attn_decode_mfma_kernel<DPAD, FULL, ROW8>;
  static bool configured = false;   // per instantiation
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess) {
      lmsf_set_error("paged_attention_decode: cannot reserve %zu bytes of LDS: %s", smem, hipGetErrorString(e));
      return 2;
    }
    configured = true;
  }
  hipLaunchKernelGGL(kernel, grid, dim3(256), smem, stream, q, q_stride, k_pages, v_pages, block_tables, btw, tok_idx,
                     seg, pos, nh, nkv, d, ps, scale_log2, window, HB, n_hb, chunk, n_splits, part_o, part_ml, out,
                     out_stride, heads_first);
  return 0;
}

// Floats that part_o and part_ml must hold for a decode launch of n tokens.
extern "C" long lmsf_attention_decode_scratch_floats(int n, int nh, int d, int n_splits) {
  return (long)n * nh * n_splits * (d + 2);
}

// One query token per entry of tok_idx (null: tokens 0 .. n - 1), at most 65535; the tokens' workgroups start
// in this order from 16 tokens on (order 0; 1 and 2 force one of the two arrangements), so the longest contexts
// should come first where they differ. chunk: keys per split, a multiple of 128;
// n_splits * chunk must cover the longest context. scratch: lmsf_attention_decode_scratch_floats floats
// (not touched with n_splits == 1). seg null: token i is the only token of request i (row i of the block tables),
// as in a step of single tokens.
extern "C" int lmsf_paged_attention_decode_mfma(const void* q, long q_stride, void* out, long out_stride,
                                                const void* k_pages, const void* v_pages, long num_pages,
                                                const int* block_tables, int btw, const int* tok_idx, int n,
                                                const int* seg, const int* pos, int nh, int nkv, int d, int ps,
                                                float scale, int window, int chunk, int n_splits, float* scratch,
                                                int order, hipStream_t stream) {
  if (int rc = check_common("paged_attention_decode", q, out, k_pages, v_pages, block_tables, seg ? seg : pos, pos,
                            q_stride, out_stride, num_pages, btw, nh, nkv, d, ps, window))
    return rc;
  LMSF_CHECK(n >= 0 && scratch != nullptr && lmsf_aligned16(scratch), "paged_attention_decode: bad arguments (scratch must be 16-byte aligned)");
  LMSF_CHECK(chunk > 0 && chunk % 128 == 0 && n_splits > 0 && n_splits <= 65535,
             "paged_attention_decode: chunk %d must be a positive multiple of 128 and splits %d in [1, 65535]", chunk,
             n_splits);
  if (n == 0) return 0;
  const int n_rep = nh / nkv, HB = heads_per_block(n_rep), n_hb = (n_rep + HB - 1) / HB;
  LMSF_CHECK(nh <= 65535 && (long)nkv * n_hb <= 65535, "paged_attention_decode: too many heads");
  LMSF_CHECK(n <= 65535, "paged_attention_decode: %d tokens in one launch (at most 65535)", n);
  // order 0: chosen here; 1: the tokens of a head start together; 2: the heads of a token. Measured at 8 kv
  // heads and 64 tokens with contexts of 192 to 2,112 keys: 75 us against 64 us with the heads of a token
  // together and the longest contexts first (32 kv heads: 214 against 176); equal contexts: the same from 16
  // tokens on, and 1 us in 12 the other way round at 8 tokens.
  const int heads_first = order == 2 || (order == 0 && n >= 16);
  const float scale_log2 = scale * 1.44269504088896340736f;
  const int dpad = (d + 31) / 32 * 32;
  float* part_o = scratch;
  float* part_ml = scratch + (long)n * nh * n_splits * d;
  dim3 grid(heads_first ? nkv * n_hb : n, heads_first ? n : nkv * n_hb, n_splits);
  int rc = 0;
#define DECODE_ARGS                                                                                                 \
  grid, stream, (const bf16_t*)q, q_stride, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_tables, btw, tok_idx, \
      seg, pos, nh, nkv, d, ps, scale_log2, window, HB, n_hb, chunk, n_splits, part_o, part_ml, (bf16_t*)out,       \
      out_stride, heads_first
  const bool row8 = ps % 32 == 0;   // (needs pages of a multiple of 8 tokens; chosen from 32 on)
#define LAUNCH(DP)                                                                                      \
  rc = d == DP ? (row8 ? launch_decode<DP, true, true>(DECODE_ARGS) : launch_decode<DP, true, false>(DECODE_ARGS)) \
               : (row8 ? launch_decode<DP, false, true>(DECODE_ARGS) : launch_decode<DP, false, false>(DECODE_ARGS))
  switch (dpad) {
    case 32: LAUNCH(32); break;
    case 64: LAUNCH(64); break;
    case 96: LAUNCH(96); break;
    case 128: LAUNCH(128); break;
    case 160: LAUNCH(160); break;
    case 192: LAUNCH(192); break;
    case 224: LAUNCH(224); break;
    default: LAUNCH(256); break;
  }
#undef LAUNCH
#undef DECODE_ARGS
  if (rc) return rc;
  LMSF_LAUNCH_CHECK("paged_attention_decode");
  if (n_splits == 1) return 0;
  if (n_splits <= REDUCE_SERIAL_SPLITS)
    hipLaunchKernelGGL(attn_decode_reduce_serial_kernel, dim3(n, nh), dim3((d + 63) / 64 * 64), 0, stream, part_o,
                       part_ml, (bf16_t*)out, out_stride, tok_idx, pos, nh, d, window, chunk, n_splits);
  else
    hipLaunchKernelGGL(attn_decode_reduce_kernel, dim3(n, nh), dim3(REDUCE_THREADS), 0, stream, part_o, part_ml, (bf16_t*)out,
                     out_stride, tok_idx, pos, nh, d, window, chunk, n_splits);
  LMSF_LAUNCH_CHECK("paged_attention_decode_reduce");
  return 0;
}
