// The switch points between the kernels (dispatch.h): host code only.
#include "dispatch.h"

#include "common.h"
#include "entry_points.h"

#include <algorithm>

namespace {

inline bool both_bf16(const LmsfProductShape& s) { return s.x_dtype == LMSF_BF16 && s.w_dtype == LMSF_BF16; }
// what the few-rows and the one-row kernels ask of their operands
inline bool skinny_ok(const LmsfProductShape& s) {
  return s.K % 8 == 0 && s.ldx % 8 == 0 && s.ldw % 8 == 0 && s.x_ok16 && s.w_ok16;
}
// what the 17-and-more-rows and the many-rows kernels ask
inline bool mid_ok(const LmsfProductShape& s) {
  return s.K % 64 == 0 && s.N % 8 == 0 && s.ldx % 8 == 0 && s.ldw % 8 == 0 && s.x_ok16 && s.w_ok16;
}
// the one-or-two-rows kernel keeps x in LDS
inline bool gemv_ok(int M, int K) { return (long)M * K * 2 <= 128 * 1024; }

inline LmsfRoute route(int r) {
  LmsfRoute o;
  o.route = r;
  o.splits = 1;
  o.plan = 0;
  o.pending = 0;
  o.chunk_rows = 0;
  return o;
}

}  // namespace

extern "C" void lmsf_route_linear(const LmsfTunables* t, const LmsfProductShape* sp, int pending_ok, LmsfRoute* out) {
  const LmsfProductShape& s = *sp;
  const int M = s.M, N = s.N, K = s.K;
  const bool bf = both_bf16(s), out_bf = s.out_dtype == LMSF_BF16;
  const bool m_ok = mid_ok(s), s_ok = skinny_ok(s);
  // deep: K at least three times N; such products go to the many-rows kernel from fewer rows on and stay with it longer
  const bool deep = (long)K >= 3L * N && out_bf;
  if (bf && t->skinny_max_rows < M && M <= t->mid_max_rows && m_ok &&
      (M <= 64 || N <= t->mid_wide_max_cols || !out_bf) && !(deep && M > t->large_deep_min_rows)) {
    *out = route(LMSF_ROUTE_MID);
    out->splits = lmsf_gemm_mid_splits(M, N, K, 0);
    out->pending = pending_ok && out_bf && out->splits > 1;
    return;
  }
  if (bf && out_bf && m_ok &&
      ((t->mid_max_rows < M && M <= t->large_max_rows) ||
       (deep && t->large_deep_min_rows < M && M <= t->large_deep_max_rows))) {
    *out = route(LMSF_ROUTE_LARGE);
    out->plan = lmsf_gemm_large_plan(M, N, K, 0);
    out->splits = out->plan % 16;
    out->pending = pending_ok && out->splits > 1;
    return;
  }
  if (pending_ok && bf && out_bf && s_ok && M > 0 &&
      ((M <= std::min(t->fuse_stream_rows, t->gemv_max_rows) && gemv_ok(M, K)) ||
       M <= std::min(std::min(t->fuse_norm_rows, t->skinny_max_rows), 16))) {
    *out = route(LMSF_ROUTE_DEFERRED);
    return;
  }
  // one row: a pure stream of W (with two rows only the fused forms gain; the LM head's matrix is large enough for
  // the few-rows kernel to reach the same rate, so it stays there)
  if (bf && 0 < M && M <= std::min(1, t->gemv_max_rows) && s_ok && gemv_ok(M, K) && (long)N * K <= (1L << 28)) {
    *out = route(LMSF_ROUTE_GEMV);
    return;
  }
  // float32 output (logits) for many rows, which the library does not offer
  if (bf && !out_bf && M > t->mid_max_rows && m_ok && t->mid_max_rows > 0) {
    *out = route(LMSF_ROUTE_CHUNKS);
    out->chunk_rows = t->mid_max_rows;
    return;
  }
  // few rows: the weight-streaming kernel; it also serves float32 output where the kernels above do not take the
  // operands, for any number of rows
  if (bf && s_ok && (M <= (out_bf ? t->skinny_max_rows : 64) || !out_bf)) {
    *out = route(LMSF_ROUTE_SKINNY);
    return;
  }
  // (float32 output that no kernel above takes, a K that is no multiple of 8, goes to the plain kernel: the library
  // would round it to bfloat16 first)
  if (t->use_library_gemm && bf && M > t->skinny_max_rows && out_bf) {
    *out = route(LMSF_ROUTE_BLAS);
    return;
  }
  *out = route(LMSF_ROUTE_PLAIN);
}

extern "C" void lmsf_route_linear_gated(const LmsfTunables* t, const LmsfProductShape* sp, int scaled_rows_per_tile,
                                        int scaled_tiles, LmsfRoute* out) {
  const LmsfProductShape& s = *sp;
  const int M = s.M, I = s.N / 2, K = s.K;
  if (scaled_rows_per_tile != 0) {
    if (!(s.w_dtype == LMSF_BF16 && skinny_ok(s) && (scaled_rows_per_tile == 16 || gemv_ok(M, K)))) {
      *out = route(LMSF_ROUTE_MATERIALIZE);
    } else if (scaled_rows_per_tile == 16 && M <= t->mid_scaled_rows && mid_ok(s) &&
               lmsf_gemm_mid_scaled_fits(M, I, K, scaled_tiles)) {
      *out = route(LMSF_ROUTE_MID_SCALED);
    } else if (scaled_rows_per_tile != 16) {
      *out = route(LMSF_ROUTE_GEMV_SCALED);
    } else {
      *out = route(LMSF_ROUTE_SKINNY_SCALED);
    }
    return;
  }
  const bool bf = both_bf16(s);
  if (bf && 0 < M && M <= t->skinny_max_rows && skinny_ok(s)) {
    *out = route(M <= t->gemv_max_rows && gemv_ok(M, K) ? LMSF_ROUTE_GEMV : LMSF_ROUTE_SKINNY);
    return;
  }
  if (bf && t->skinny_max_rows < M && M <= 64 && mid_ok(s)) {
    *out = route(LMSF_ROUTE_MID);
    out->splits = lmsf_gemm_mid_splits(M, I, K, 1);
    return;
  }
  // (the many-rows kernel writes its outputs eight at a time)
  if (bf && 64 < M && M <= t->large_max_rows && mid_ok(s) && I % 8 == 0) {
    *out = route(LMSF_ROUTE_LARGE);
    out->plan = lmsf_gemm_large_plan(M, I, K, 1);
    out->splits = out->plan % 16;
    return;
  }
  *out = route(LMSF_ROUTE_SEPARATE);
}

extern "C" void lmsf_route_qkv(const LmsfTunables* t, const LmsfProductShape* sp, int fused_shape,
                               int scaled_rows_per_tile, LmsfRoute* out) {
  const LmsfProductShape& s = *sp;
  const int M = s.M, K = s.K;
  if (scaled_rows_per_tile != 0) {
    if (fused_shape && skinny_ok(s) && (scaled_rows_per_tile == 16 || gemv_ok(M, K)))
      *out = route(scaled_rows_per_tile != 16 ? LMSF_ROUTE_GEMV_SCALED : LMSF_ROUTE_SKINNY_SCALED);
    else
      *out = route(LMSF_ROUTE_MATERIALIZE);
    return;
  }
  if (fused_shape && s.x_dtype == LMSF_BF16 && 0 < M && M <= std::min(64, std::max(t->skinny_max_rows, t->qkv_fused_max_rows)) &&
      skinny_ok(s)) {
    *out = route(M <= t->gemv_max_rows && gemv_ok(M, K) ? LMSF_ROUTE_GEMV : LMSF_ROUTE_SKINNY);
    return;
  }
  // the plain product, unfinished where it splits K (the rotation and the cache write then add up the partial sums),
  // but never as a product not yet started
  *out = route(LMSF_ROUTE_SEPARATE);
  out->pending = M > std::max(std::max(t->fuse_stream_rows, t->fuse_norm_rows), t->skinny_max_rows);
}

extern "C" void lmsf_route_deferred_norm(const LmsfTunables* t, int M, int N, int K, int fits, int prepares,
                                         LmsfRoute* out) {
  const bool one_or_two = fits && M <= std::min(t->fuse_stream_rows, t->gemv_max_rows) && gemv_ok(M, K);
  if (prepares && one_or_two && gemv_ok(M, N))
    *out = route(LMSF_ROUTE_GEMV_ADD_NORM);
  else if (prepares && M <= std::min(std::min(t->fuse_norm_rows, t->skinny_max_rows), 16) && !one_or_two)
    *out = route(LMSF_ROUTE_SKINNY_ADD_NORM);
  else if (one_or_two)
    *out = route(LMSF_ROUTE_GEMV_ADD);
  else
    *out = route(LMSF_ROUTE_MATERIALIZE);
}

// Measured: about 512 workgroups fill the chip; beyond that a split only adds partial results, and with two short
// halves the reduction kernel costs more than the second half saves. With contexts of tens of thousands of keys
// twice as many do better (8 tokens of 100,000 keys: a step of 21.2 -> 19.2 ms, 16 of 50,000: 21.6 -> 18.9), from
// 49,152 keys and 16 pairs of token and kv head on four times as many (2 tokens of 100,000 keys: 8.28 -> 7.33 ms).
extern "C" void lmsf_route_decode_attention(const LmsfTunables* t, int n_single, int nh, int nkv, int max_context,
                                            int* chunk, int* n_splits) {
  const int n_hb = ((nh / nkv) + 15) / 16;
  const int most = std::max(1, (max_context + 127) / 128);
  const int pairs = std::max(1, n_single * nkv * n_hb);
  const int fill = max_context >= 49152 && pairs >= 16 ? 2048 : max_context >= 32768 && pairs >= 32 ? 1024 : 512;
  int want = std::max(1, std::min(most, fill / pairs));
  if (want == 2 && max_context <= 512) want = 1;
  if (t->decode_attention_splits) want = std::min(most, t->decode_attention_splits);
  const int c = std::max(128, (((max_context + want - 1) / want) + 127) / 128 * 128);
  *chunk = c;
  *n_splits = std::max(1, (max_context + c - 1) / c);
}
