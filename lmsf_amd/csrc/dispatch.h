// Which kernel runs an operation: the one table of switch points of this library.
//
// The matrix products change kernels with the number of rows (one row: a pure stream of W; up to 16: the
// few-rows kernel with its fused epilogues; 17 to 128: the 17-and-more-rows kernel; up to 256, or 1,024 for deep
// products: the many-rows kernel; beyond: the BLAS library), and so do the forms in which a norm, a rotation or
// a gated activation is folded into them. Both callers of the kernels, the step program (program.hip) and the
// Python face (ops/hip_ops.py), ask the functions below and launch what they are told; neither decides anything
// from a number of rows itself. The reference has one product for all sizes and leaves the choice to cuBLASLt's
// profiled tactics (tops/src/cublas.rs:121-223).
#pragma once

#ifdef __cplusplus
extern "C" {
#endif

// The numbers of rows at which the kernels change (attributes of the same names of ops.HipOps).
typedef struct {
  int fuse_norm_rows;             // up to this many rows (beyond fuse_stream_rows) the products around a norm do its work (0: never)
  int fuse_stream_rows;           // up to this many rows the residual addition and the norm run inside the products (0: never)
  int gemv_max_rows;              // products of up to this many rows stream W without the matrix cores (0: never)
  int skinny_variant;             // tiling of the few-rows kernel (0: default; others for tuning)
  int mid_wide_max_cols;          // beyond 64 rows the 17-and-more-rows kernel takes products of up to this many columns
  int mid_max_rows;               // rows up to which the 17-and-more-rows kernel runs (64 with the gated activation)
  int skinny_max_rows;            // rows up to which the few-rows kernel runs
  int prefill_attention_variant;  // 0: keys and values staged in LDS; 1: fetched by every wave; 2: as 0, short table window
  int decode_attention_order;     // 0: chosen from the number of workgroups; 1: tokens of a head together; 2: heads of a token
  int decode_attention_splits;    // 0: chosen from batch and context; n: at most n splits of the keys
  int use_library_gemm;           // bfloat16 products of many rows go to the BLAS library (0: to the plain kernel)
  int large_max_rows;             // rows up to which the many-rows kernel runs (0: never)
  int large_deep_min_rows;        // products with K >= 3 N go to the many-rows kernel from beyond this many rows
  int mid_scaled_rows;            // rows up to which the gated product after a norm runs in the 17-and-more-rows kernel (0: never)
  int large_deep_max_rows;        // rows up to which products with K >= 3 N stay with the many-rows kernel
  int qkv_fused_max_rows;         // rows up to which the QKV product with rotation and cache write runs in the few-rows kernel
} LmsfTunables;

enum {
  // plain products
  LMSF_ROUTE_PLAIN = 0,       // the float32 multiply-add kernel (any shape)
  LMSF_ROUTE_MID,             // 17-and-more-rows kernel; ``splits`` parts of K; ``pending``: partial sums stay
  LMSF_ROUTE_LARGE,           // many-rows kernel with ``plan``; ``splits``, ``pending`` likewise
  LMSF_ROUTE_DEFERRED,        // not started: the norm that follows runs it
  LMSF_ROUTE_GEMV,            // one row
  LMSF_ROUTE_CHUNKS,          // ``chunk_rows`` rows at a time, each chunk routed again (float32 output of many rows)
  LMSF_ROUTE_SKINNY,          // few-rows kernel, 64 rows a launch
  LMSF_ROUTE_BLAS,            // the BLAS library
  // gated products and QKV products with rotation and cache write
  LMSF_ROUTE_MATERIALIZE,     // finish the operand first, then ask again with a tensor
  LMSF_ROUTE_MID_SCALED,      // operand with its norm factor missing, 17-and-more-rows kernel
  LMSF_ROUTE_GEMV_SCALED,     // the same, one-or-two-rows kernel
  LMSF_ROUTE_SKINNY_SCALED,   // the same, few-rows kernel
  LMSF_ROUTE_SEPARATE,        // the plain product (``pending`` allowed as said), then the elementwise kernel
  // a product that a norm finds unstarted
  LMSF_ROUTE_GEMV_ADD_NORM,   // adds into the stream, leaves stream * w and sums of squares (one or two rows)
  LMSF_ROUTE_SKINNY_ADD_NORM, // the same from the few-rows kernel
  LMSF_ROUTE_GEMV_ADD         // adds into the stream; the norm kernel follows
};

typedef struct {
  int route, splits, plan, pending, chunk_rows;
} LmsfRoute;

// What a product's operands look like to the kernels. ``x_ok16`` / ``w_ok16``: the base address is 16-byte aligned.
typedef struct {
  int M, N, K;             // rows of x, rows of W (for a gated product: both halves, 2 I), columns of both
  int x_dtype, w_dtype, out_dtype;
  long ldx, ldw;
  int x_ok16, w_ok16;
} LmsfProductShape;

// y = x W^T (+ bias). ``pending_ok``: the caller takes an unfinished product.
void lmsf_route_linear(const LmsfTunables* t, const LmsfProductShape* s, int pending_ok, LmsfRoute* out);
// act(x Wg^T) * (x Wu^T). ``scaled_rows_per_tile`` 0: x is a tensor; else x lacks its norm factor, with sums of
// squares in ``scaled_tiles`` tiles of that many rows.
void lmsf_route_linear_gated(const LmsfTunables* t, const LmsfProductShape* s, int scaled_rows_per_tile,
                             int scaled_tiles, LmsfRoute* out);
// The QKV product with rotation and cache write. ``fused_shape``: the epilogue forms apply (a table and slots
// are given, NeoX pairing over the whole head, a head size that is a multiple of 32, bfloat16 weight and pages,
// the weight has (nh + 2 nkv) d rows of K columns).
void lmsf_route_qkv(const LmsfTunables* t, const LmsfProductShape* s, int fused_shape, int scaled_rows_per_tile,
                    LmsfRoute* out);
// A norm whose branch is a product not yet started (M rows, N columns over K). ``fits``: the product has the
// stream's shape and no rows are selected; ``prepares``: moreover the caller takes rows without their factor and
// the norm's output and weight are bfloat16.
void lmsf_route_deferred_norm(const LmsfTunables* t, int M, int N, int K, int fits, int prepares, LmsfRoute* out);
// How the decode attention kernel splits the keys of a step of ``n_single`` single tokens whose longest context
// is ``max_context``: keys a split (a multiple of 128) and the number of splits.
void lmsf_route_decode_attention(const LmsfTunables* t, int n_single, int nh, int nkv, int max_context, int* chunk,
                                 int* n_splits);

#ifdef __cplusplus
}
#endif
