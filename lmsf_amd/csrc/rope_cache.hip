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
template <typename T>
__global__ __launch_bounds__(256) void rope_cache_write_kernel(
    T* __restrict__ q, T* __restrict__ k, const T* __restrict__ v, long row_stride, const int* __restrict__ positions,
    const float* __restrict__ table, int rot, int neox, const int* __restrict__ slots, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int nh, int nkv, int d, int ps, int n_tokens) {
  const long t = (long)blockIdx.x * blockDim.y + threadIdx.y;
  if (t >= n_tokens) return;
  const int hy = blockIdx.y;
  const int half = rot / 2;
  const float* cs = table ? table + (long)positions[t] * rot : nullptr;
  int slot = -1;
  if (slots) slot = slots[t];
  if (hy < nh) {
    if (!cs || !q) return;
    T* x = q + t * row_stride + (long)hy * d;
    for (int i = threadIdx.x; i < half; i += 64) {
      const int xi = neox ? i : 2 * i, yi = neox ? i + half : 2 * i + 1;
      const float c = cs[i], s = cs[half + i];
      float xr, yr;
      rope_rotate(to_f32<T>(x[xi]), to_f32<T>(x[yi]), c, s, &xr, &yr);
      x[xi] = from_f32<T>(xr);
      x[yi] = from_f32<T>(yr);
    }
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
        rope_rotate(to_f32<T>(x[xi]), to_f32<T>(x[yi]), c, s, &xf, &yf);
        const T xr = from_f32<T>(xf), yr = from_f32<T>(yf);
        x[xi] = xr;
        x[yi] = yr;
        if (dst) {
          dst[xi] = xr;
          dst[yi] = yr;
        }
      }
    }
    if (dst) {
      // the part of k that the rotation did not touch (all of it without a table)
      for (int i = (cs ? rot : 0) + threadIdx.x; i < d; i += 64) dst[i] = x[i];
    }
  } else {
    if (!v || slot < 0) return;
    const int h = hy - nh - nkv;
    const T* x = v + t * row_stride + (long)h * d;
    // element offset of (page, head h, 0, offset) in the transposed V pages
    T* dst = v_pages + ((long)(slot / ps) * nkv + h) * ps * d + (slot % ps);
    for (int i = threadIdx.x; i < d; i += 64) dst[(long)i * ps] = x[i];
  }
}

extern "C" int lmsf_rope_cache_write(void* q, void* k, const void* v, int dtype, int n_tokens, long row_stride,
                                     const int* positions, const float* table, int rot, int neox, int max_pos,
                                     const int* slots, void* k_pages, void* v_pages, long num_pages, int nh, int nkv,
                                     int d, int ps, hipStream_t stream) {
  LMSF_CHECK(dtype == LMSF_F32 || dtype == LMSF_BF16, "rope_cache_write: unknown dtype code %d", dtype);
  LMSF_CHECK(n_tokens >= 0 && nh >= 0 && nkv >= 0 && d > 0, "rope_cache_write: bad sizes");
  LMSF_CHECK(row_stride >= 0, "rope_cache_write: bad row stride");
  if (table) {
    LMSF_CHECK(positions != nullptr, "rope_cache_write: rotation needs positions");
    LMSF_CHECK(rot > 0 && rot % 2 == 0 && rot <= d, "rope_cache_write: rotary_dim %d must be even and <= head_dim %d",
               rot, d);
    LMSF_CHECK(max_pos > 0, "rope_cache_write: empty table");
  }
  if (slots) {
    LMSF_CHECK(k && v && k_pages && v_pages, "rope_cache_write: cache write needs k, v and both page tensors");
    LMSF_CHECK(ps > 0 && num_pages > 0, "rope_cache_write: bad page geometry");
  }
  if (n_tokens == 0) return 0;
  const int heads = nh + 2 * nkv;
  LMSF_CHECK(heads > 0 && heads <= 65535, "rope_cache_write: %d heads do not fit the grid", heads);
  const int per_block = n_tokens >= 64 ? 4 : 1;   // tokens per workgroup: many small workgroups cost a long prompt time
  dim3 grid((n_tokens + per_block - 1) / per_block, heads), block(64, per_block);
  if (dtype == LMSF_F32)
    hipLaunchKernelGGL((rope_cache_write_kernel<float>), grid, block, 0, stream, (float*)q, (float*)k,
                       (const float*)v, row_stride, positions, table, rot, neox, slots, (float*)k_pages,
                       (float*)v_pages, nh, nkv, d, ps, n_tokens);
  else
    hipLaunchKernelGGL((rope_cache_write_kernel<bf16_t>), grid, block, 0, stream, (bf16_t*)q,
                       (bf16_t*)k, (const bf16_t*)v, row_stride, positions, table, rot, neox, slots, (bf16_t*)k_pages,
                       (bf16_t*)v_pages, nh, nkv, d, ps, n_tokens);
  LMSF_LAUNCH_CHECK("rope_cache_write");
  return 0;
}
