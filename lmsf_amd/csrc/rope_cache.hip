// Rotary position embedding fused with the write of K and V into the paged cache.
//
// Rotation (vllm/kernels/pos_encoding_kernels.cu:12-77): for every head of q and k and every
// pair index i < rot/2,  x' = x cos - y sin,  y' = y cos + x sin, with (x, y) = elements
// (i, i + rot/2) in NeoX style or (2i, 2i+1) in GPT-J style, and cos/sin read from the row of the
// table that the token's position selects. The reference computes in the model's dtype from a
// table in that dtype; here the table is float32 [max_pos, rot] = [cos(rot/2) | sin(rot/2)] and the
// arithmetic is float32, rounded once at the store.
//
// Cache write (vllm/kernels/cache_kernels.cu:190-232): the token's rotated k and its v go to slot
// s = page * page_size + offset; a negative slot is skipped. Page layout here is
// [page, kv_head, offset, d] for K and [page, kv_head, d, offset] for V, which the attention kernels read
// as matrix-core operands without a transposition (the reference uses [page, head, d/x, offset, x] and,
// like here, [page, head, d, offset]).
//
// q, k, v point at the first column of their parts inside one row-strided buffer (the fused QKV
// output); row_stride is in elements. Either half may be switched off: table == null leaves q and
// k unrotated, slots == null writes no cache.
#include "common.h"

// One wave per (token, head): heads 0 .. nh-1 are q heads, then nkv k heads, then nkv v heads (a decode step
// has few tokens, so the parallelism has to come from the heads); a workgroup holds the waves of
// blockDim.y consecutive tokens of one head.
// PART: the values come from the partial sums of the fused QKV product (column (head index) * d + i of row
// t) and q, k, v are only written: the reduction, the rotation and the cache write in one kernel.
template <typename T, bool PART>
__global__ __launch_bounds__(256) void rope_cache_write_kernel(
    T* __restrict__ q, T* __restrict__ k, T* __restrict__ v, long row_stride, const int* __restrict__ positions,
    const float* __restrict__ table, int rot, int neox, const int* __restrict__ slots, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int nh, int nkv, int d, int ps, int n_tokens, LmsfPartialSum partial) {
  const long t = (long)blockIdx.x * blockDim.y + threadIdx.y;
  if (t >= n_tokens) return;
  const int hy = blockIdx.y;
  const int half = rot / 2;
  const int col0 = hy * d;
  auto rd = [&](const T* x, int i) -> float {
    return PART ? partial_sum_value(partial, (int)t, col0 + i) : to_f32<T>(x[i]);
  };
  const float* cs = table ? table + (long)positions[t] * rot : nullptr;
  int slot = -1;
  if (slots) slot = slots[t];
  if (hy < nh) {
    if (!q || (!cs && !PART)) return;
    T* x = q + t * row_stride + (long)hy * d;
    if (cs) {
      for (int i = threadIdx.x; i < half; i += 64) {
        const int xi = neox ? i : 2 * i, yi = neox ? i + half : 2 * i + 1;
        const float c = cs[i], s = cs[half + i];
        float xr, yr;
        rope_rotate(rd(x, xi), rd(x, yi), c, s, &xr, &yr);
        x[xi] = from_f32<T>(xr);
        x[yi] = from_f32<T>(yr);
      }
    }
    if (PART)
      for (int i = (cs ? rot : 0) + threadIdx.x; i < d; i += 64) x[i] = from_f32<T>(rd(x, i));
  } else if (hy < nh + nkv) {
    if (!k) return;
    const int h = hy - nh;
    T* x = k + t * row_stride + (long)h * d;
    // element offset of (page, head h, offset, 0) in the K pages
    T* dst = slot >= 0 ? k_pages + (((long)(slot / ps) * nkv + h) * ps + (slot % ps)) * d : nullptr;
    if (cs) {
      for (int i = threadIdx.x; i < half; i += 64) {
        const int xi = neox ? i : 2 * i, yi = neox ? i + half : 2 * i + 1;
        const float c = cs[i], s = cs[half + i];
        float xf, yf;
        rope_rotate(rd(x, xi), rd(x, yi), c, s, &xf, &yf);
        const T xr = from_f32<T>(xf), yr = from_f32<T>(yf);
        x[xi] = xr;
        x[yi] = yr;
        if (dst) {
          dst[xi] = xr;
          dst[yi] = yr;
        }
      }
    }
    if (dst || PART) {
      // the part of k that the rotation did not touch (all of it without a table)
      for (int i = (cs ? rot : 0) + threadIdx.x; i < d; i += 64) {
        const T val = PART ? from_f32<T>(rd(x, i)) : x[i];
        if (PART) x[i] = val;
        if (dst) dst[i] = val;
      }
    }
  } else {
    if (!v || (slot < 0 && !PART)) return;
    const int h = hy - nh - nkv;
    T* x = v + t * row_stride + (long)h * d;
    // element offset of (page, head h, 0, offset) in the transposed V pages
    T* dst = slot >= 0 ? v_pages + ((long)(slot / ps) * nkv + h) * ps * d + (slot % ps) : nullptr;
    for (int i = threadIdx.x; i < d; i += 64) {
      const T val = PART ? from_f32<T>(rd(x, i)) : x[i];
      if (PART) x[i] = val;
      if (dst) dst[(long)i * ps] = val;
    }
  }
}

// The same work for steps of many tokens (prompts): a workgroup takes 16 consecutive tokens of one head and
// moves 16-byte pieces, so q, k and the K cache are read and written in whole pieces, and the transposed V
// cache, whose rows run along the tokens of a page, is written through an LDS tile with the 16 tokens of a
// value next to each other: where their slots are consecutive, 16 lanes write 16 neighbouring elements. Needs
// d, rot (GPT-J pairing) or rot / 2 (NeoX pairing) to be multiples of the piece (8 bfloat16, 4 float32) and
// rows that start on 16-byte boundaries; the kernel above serves the rest and the steps of few tokens.
template <typename T>
__global__ __launch_bounds__(256) void rope_cache_tile_kernel(
    T* __restrict__ q, T* __restrict__ k, T* __restrict__ v, long row_stride, const int* __restrict__ positions,
    const float* __restrict__ table, int rot, int neox, const int* __restrict__ slots, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int nh, int nkv, int d, int ps, int n_tokens) {
  constexpr int VEC = 16 / (int)sizeof(T);
  constexpr int TOK = 16;
  extern __shared__ __align__(16) unsigned char tile_raw[];
  const int t0 = blockIdx.x * TOK, hy = blockIdx.y, tid = threadIdx.x;
  const int ntok = min(TOK, n_tokens - t0);
  const int half = rot / 2;
  if (hy < nh + nkv) {
    const bool is_k = hy >= nh;
    const int h = hy - nh;
    T* base = is_k ? k + (long)h * d : q + (long)hy * d;
    const bool to_cache = is_k && slots != nullptr;
    if (!base || (!table && !to_cache)) return;
    auto cache_row = [&](int t) -> T* {
      const int slot = to_cache ? slots[t] : -1;
      return slot >= 0 ? k_pages + (((long)(slot / ps) * nkv + h) * ps + (slot % ps)) * d : nullptr;
    };
    if (table) {
      if (neox) {
        const int pieces = half / VEC;
        for (int item = tid; item < ntok * pieces; item += 256) {
          const int tt = item / pieces, pc = item - tt * pieces, t = t0 + tt;
          T* x = base + (long)t * row_stride;
          const float* cs = table + (long)positions[t] * rot + pc * VEC;
          Vec16<T> lo, hi;
          lo.load(x + pc * VEC);
          hi.load(x + half + pc * VEC);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            float xr, yr;
            rope_rotate(lo.get(e), hi.get(e), cs[e], cs[half + e], &xr, &yr);
            lo.set(e, xr);
            hi.set(e, yr);
          }
          lo.store(x + pc * VEC);
          hi.store(x + half + pc * VEC);
          if (T* dst = cache_row(t)) {
            lo.store(dst + pc * VEC);
            hi.store(dst + half + pc * VEC);
          }
        }
      } else {
        const int pieces = rot / VEC;
        for (int item = tid; item < ntok * pieces; item += 256) {
          const int tt = item / pieces, pc = item - tt * pieces, t = t0 + tt;
          T* x = base + (long)t * row_stride;
          const float* cs = table + (long)positions[t] * rot + pc * (VEC / 2);
          Vec16<T> a;
          a.load(x + pc * VEC);
#pragma unroll
          for (int e = 0; e < VEC / 2; ++e) {
            float xr, yr;
            rope_rotate(a.get(2 * e), a.get(2 * e + 1), cs[e], cs[half + e], &xr, &yr);
            a.set(2 * e, xr);
            a.set(2 * e + 1, yr);
          }
          a.store(x + pc * VEC);
          if (T* dst = cache_row(t)) a.store(dst + pc * VEC);
        }
      }
    }
    if (to_cache) {
      // the part of k that the rotation did not touch (all of it without a table)
      const int start = table ? rot : 0, pieces = (d - start) / VEC;
      for (int item = tid; item < ntok * pieces; item += 256) {
        const int tt = item / pieces, pc = item - tt * pieces, t = t0 + tt;
        if (T* dst = cache_row(t)) {
          Vec16<T> a;
          a.load(base + (long)t * row_stride + start + pc * VEC);
          a.store(dst + start + pc * VEC);
        }
      }
    }
  } else {
    if (!v || !slots) return;
    const int h = hy - nh - nkv;
    T* tile = reinterpret_cast<T*>(tile_raw);
    const int ld = d + (sizeof(T) == 2 ? 2 : 1);   // rows an odd number of 4-byte words apart: no bank conflicts
    const int pieces = d / VEC;
    for (int item = tid; item < ntok * pieces; item += 256) {
      const int tt = item / pieces, pc = item - tt * pieces;
      Vec16<T> a;
      a.load(v + (long)(t0 + tt) * row_stride + (long)h * d + pc * VEC);
#pragma unroll
      for (int e = 0; e < VEC; ++e) tile[tt * ld + pc * VEC + e] = a.raw(e);
    }
    __syncthreads();
    for (int e = tid; e < ntok * d; e += 256) {
      const int dv = e / ntok, tt = e - dv * ntok;
      const int slot = slots[t0 + tt];
      if (slot >= 0) v_pages[(((long)(slot / ps) * nkv + h) * d + dv) * ps + (slot % ps)] = tile[tt * ld + dv];
    }
  }
}

static int rope_cache_check(const char* who, const void* k, const void* v, int n_tokens, long row_stride,
                            const int* positions, const float* table, int rot, int max_pos, const int* slots,
                            const void* k_pages, const void* v_pages, long num_pages, int nh, int nkv, int d, int ps) {
  LMSF_CHECK(n_tokens >= 0 && nh >= 0 && nkv >= 0 && d > 0, "%s: bad sizes", who);
  LMSF_CHECK(row_stride >= 0, "%s: bad row stride", who);
  if (table) {
    LMSF_CHECK(positions != nullptr, "%s: rotation needs positions", who);
    LMSF_CHECK(rot > 0 && rot % 2 == 0 && rot <= d, "%s: rotary_dim %d must be even and <= head_dim %d", who, rot, d);
    LMSF_CHECK(max_pos > 0, "%s: empty table", who);
  }
  if (slots) {
    LMSF_CHECK(k && v && k_pages && v_pages, "%s: cache write needs k, v and both page tensors", who);
    LMSF_CHECK(ps > 0 && num_pages > 0, "%s: bad page geometry", who);
  }
  const int heads = nh + 2 * nkv;
  LMSF_CHECK(heads > 0 && heads <= 65535, "%s: %d heads do not fit the grid", who, heads);
  return 0;
}

extern "C" int lmsf_rope_cache_write(void* q, void* k, void* v, int dtype, int n_tokens, long row_stride,
                                     const int* positions, const float* table, int rot, int neox, int max_pos,
                                     const int* slots, void* k_pages, void* v_pages, long num_pages, int nh, int nkv,
                                     int d, int ps, hipStream_t stream) {
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "rope_cache_write: unknown dtype code %d", dtype);
  if (int rc = rope_cache_check("rope_cache_write", k, v, n_tokens, row_stride, positions, table, rot, max_pos, slots,
                                k_pages, v_pages, num_pages, nh, nkv, d, ps))
    return rc;
  if (n_tokens == 0) return 0;
  const int heads = nh + 2 * nkv;
  const LmsfPartialSum none = {nullptr, nullptr, 0, 0, 0};
  // steps of many tokens go in tiles of 16 tokens with 16-byte accesses where the sizes allow it
  const int vec = dtype == LMSF_F32 ? 4 : 8;
  const bool rot_ok = !table || (neox ? (rot / 2) % vec == 0 : rot % vec == 0);
  const auto al16 = [](const void* p) { return p == nullptr || lmsf_aligned16(p); };
  if (n_tokens >= 64 && d % vec == 0 && rot_ok && row_stride % vec == 0 && al16(q) && al16(k) && al16(v) &&
      al16(k_pages) && al16(table)) {
    dim3 tgrid((n_tokens + 15) / 16, heads);
    const size_t smem = (size_t)16 * (d + 4) * (dtype == LMSF_F32 ? 4 : 2);
    if (dtype == LMSF_F32)
      hipLaunchKernelGGL((rope_cache_tile_kernel<float>), tgrid, dim3(256), smem, stream, (float*)q, (float*)k, (float*)v,
                         row_stride, positions, table, rot, neox, slots, (float*)k_pages, (float*)v_pages, nh, nkv, d,
                         ps, n_tokens);
    else
      hipLaunchKernelGGL((rope_cache_tile_kernel<bf16_t>), tgrid, dim3(256), smem, stream, (bf16_t*)q, (bf16_t*)k,
                         (bf16_t*)v, row_stride, positions, table, rot, neox, slots, (bf16_t*)k_pages, (bf16_t*)v_pages,
                         nh, nkv, d, ps, n_tokens);
    LMSF_LAUNCH_CHECK("rope_cache_write (tiles)");
    return 0;
  }
  const int per_block = n_tokens >= 64 ? 4 : 1;   // tokens per workgroup: many small workgroups cost a long prompt time
  dim3 grid((n_tokens + per_block - 1) / per_block, heads), block(64, per_block);
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((rope_cache_write_kernel<float, false>), grid, block, 0, stream, (float*)q, (float*)k,
                       (float*)v, row_stride, positions, table, rot, neox, slots, (float*)k_pages,
                       (float*)v_pages, nh, nkv, d, ps, n_tokens, none);
  else
    hipLaunchKernelGGL((rope_cache_write_kernel<bf16_t, false>), grid, block, 0, stream, (bf16_t*)q,
                       (bf16_t*)k, (bf16_t*)v, row_stride, positions, table, rot, neox, slots, (bf16_t*)k_pages,
                       (bf16_t*)v_pages, nh, nkv, d, ps, n_tokens, none);
  LMSF_LAUNCH_CHECK("rope_cache_write");
  return 0;
}

// The same for a fused QKV product that was left as partial sums (lmsf_gemm_mid_partial with
// N = (nh + 2 nkv) * d): part float32 [n_split, n_tokens, N], bias bfloat16 [N] or null. y [n_tokens, N]
// bfloat16 (row stride ldy) receives the rotated q and k and v; the cache receives k and v.
extern "C" int lmsf_rope_cache_write_partial(const float* part, const void* bias, int n_split, void* y, long ldy,
                                             int n_tokens, const int* positions, const float* table, int rot,
                                             int neox, int max_pos, const int* slots, void* k_pages, void* v_pages,
                                             long num_pages, int nh, int nkv, int d, int ps, hipStream_t stream) {
  LMSF_CHECK(part != nullptr && y != nullptr && n_split >= 1, "rope_cache_write_partial: bad arguments");
  const long N = (long)(nh + 2 * nkv) * d;
  LMSF_CHECK(ldy >= N && N <= 2147483647L, "rope_cache_write_partial: row stride %ld below %ld columns", ldy, N);
  if (int rc = rope_cache_check("rope_cache_write_partial", y, y, n_tokens, ldy, positions, table, rot, max_pos, slots,
                                k_pages, v_pages, num_pages, nh, nkv, d, ps))
    return rc;
  if (n_tokens == 0) return 0;
  const LmsfPartialSum ps_ = {part, (const bf16_t*)bias, n_split, n_tokens, (int)N};
  bf16_t* yb = (bf16_t*)y;
  const int per_block = n_tokens >= 64 ? 4 : 1;
  dim3 grid((n_tokens + per_block - 1) / per_block, nh + 2 * nkv), block(64, per_block);
  hipLaunchKernelGGL((rope_cache_write_kernel<bf16_t, true>), grid, block, 0, stream, yb, yb + (long)nh * d,
                     yb + (long)(nh + nkv) * d, ldy, positions, table, rot, neox, slots, (bf16_t*)k_pages,
                     (bf16_t*)v_pages, nh, nkv, d, ps, n_tokens, ps_);
  LMSF_LAUNCH_CHECK("rope_cache_write_partial");
  return 0;
}
