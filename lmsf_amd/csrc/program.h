// The step program's C interface (program.hip): operations are added one by one, the program is sealed, and
// every step is one call of lmsf_program_run. The structures are mirrored with ctypes in ops/program.py.
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LMSF_MAX_GROUPS 8

// return values of lmsf_program_run beside 0 and errors
#define LMSF_PROGRAM_NOT_NATIVE 3   // the step needs a product that only the BLAS library has; nothing was launched
#define LMSF_PROGRAM_NO_ROOM 4      // the workspace is too small for the step; nothing was launched

enum {
  LMSF_OP_EMBEDDING = 1,
  LMSF_OP_ADD_RMS_NORM,
  LMSF_OP_QKV_ROPE_CACHE,
  LMSF_OP_ATTENTION,
  LMSF_OP_LINEAR,
  LMSF_OP_LINEAR_GATED,
  LMSF_OP_MATERIALIZE,
  LMSF_OP_COUNT
};

// which of the step's device arrays an operation reads
enum {
  LMSF_CTX_NONE = 0,
  LMSF_CTX_TOKEN_IDS = 1,
  LMSF_CTX_POSITIONS = 2,
  LMSF_CTX_SEG_OF = 3,
  LMSF_CTX_LOGIT_ROWS = 4,
  LMSF_CTX_SLOTS = 16,    // + cache group
  LMSF_CTX_TABLES = 32    // + cache group
};

// The numbers of rows at which the products change kernels (the attributes of the same names of ops.HipOps).
typedef struct {
  int fuse_norm_rows, fuse_stream_rows, gemv_max_rows, skinny_variant, mid_wide_max_cols, mid_max_rows,
      skinny_max_rows, prefill_attention_variant, decode_attention_order, decode_attention_splits, use_library_gemm,
      large_max_rows, large_deep_min_rows, mid_scaled_rows;
} LmsfTunables;

// One operation. Registers (in0, in1, out) are numbered in the order they are first written; -1: none.
//   embedding:       out = rows of w [vocab, N] (wdtype) at the ids ctx0, times scale, float32
//   add_rms_norm:    out = norm(in0 + in1) * (w + weight_offset); in1 is the float32 stream [*, N], updated in
//                    place; rows_ctx: only these rows; defer_ok: the reader of out takes rows whose factor is missing
//   qkv_rope_cache:  out = in0 w^T + bias, w [N, K]; q and k heads rotated by table [max_pos, rot] at the positions
//                    ctx0; k and v stored in the pages at the slots ctx1 (none: not stored)
//   attention:       out = attention of the first nh * d columns of in0 over the pages, block tables ctx0
//   linear:          out = in0 w^T + bias in out_dtype; pending_ok: the reader of out takes an unfinished product;
//                    is_head: the result goes to the step's logits buffer
//   linear_gated:    out = act(in0 wg^T) * (in0 wu^T), w = [wg; wu] of N = 2 I rows; act 1: SiLU, 2: GELU
//   materialize:     out = in0 as a finished tensor
typedef struct {
  int kind, in0, in1, out;
  int ctx0, ctx1, rows_ctx;
  const void* w;
  const void* bias;
  const void* table;
  void* k_pages;
  void* v_pages;
  int wdtype, out_dtype, cache_dtype;
  int N, K;
  long ldw;
  int nh, nkv, d, rot, neox, ps, window, max_pos, act, defer_ok, pending_ok, is_head, vocab;
  long num_pages;
  float eps, weight_offset, scale;
} LmsfOpDesc;

// One step: its sizes, its device arrays (engine.batch.StepContext), the workspace and where the logits go.
typedef struct {
  int n_tokens, n_segments, n_logit_rows, max_context, all_single, n_groups;
  const int* token_ids;
  const int* positions;
  const int* seg_of;
  const int* logit_rows;
  const int* longest_first;           // a step of single tokens: its tokens, the longest context first
  const int* slots[LMSF_MAX_GROUPS];
  const int* tables[LMSF_MAX_GROUPS];
  int widths[LMSF_MAX_GROUPS];
  const int* plan;                    // device copy of what lmsf_program_plan wrote (null for single tokens)
  void* workspace;
  long workspace_bytes;
  float* logits;                      // [n_logit_rows, vocabulary]
  int* bad_flag;                      // set by the embedding when an id lies outside the vocabulary
} LmsfStepDesc;

void* lmsf_program_create(const LmsfTunables* tunables);
void lmsf_program_destroy(void* program);
int lmsf_program_add(void* program, const LmsfOpDesc* op);
int lmsf_program_seal(void* program);
long lmsf_program_plan(void* program, int S, const int* seg_lens, const int* seg_first_pos, int* out, long capacity);
long lmsf_program_plan_capacity(void* program, int N);
int lmsf_program_run(void* program, const LmsfStepDesc* step, int check_only, hipStream_t stream);

#ifdef __cplusplus
}
#endif
