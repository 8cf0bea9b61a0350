// The step program's C interface (program.hip): operations are added one by one, the program is sealed, and
// every step is one call of lmsf_program_run. The structures are mirrored with ctypes in ops/program.py.
#pragma once

#include <hip/hip_runtime.h>

#include "dispatch.h"

#ifdef __cplusplus
extern "C" {
#endif

#define LMSF_MAX_GROUPS 8
#define LMSF_MAX_PLANS 4

// return value of lmsf_program_run beside 0 and errors
#define LMSF_PROGRAM_NO_ROOM 4      // the workspace is too small for the step; nothing was launched

enum {
  LMSF_OP_EMBEDDING = 1,
  LMSF_OP_ADD_RMS_NORM,
  LMSF_OP_QKV_ROPE_CACHE,
  LMSF_OP_ATTENTION,
  LMSF_OP_LINEAR,
  LMSF_OP_LINEAR_GATED,
  LMSF_OP_MATERIALIZE,
  LMSF_OP_ROPE_CACHE_WRITE,
  LMSF_OP_GATED_ACT,
  LMSF_OP_CALLBACK,
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

// One operation. Registers (in0, in1, out) are numbered in the order they are first written; -1: none.
//   embedding:        out = rows of w [vocab, N] (wdtype) at the ids ctx0, times scale, float32
//   add_rms_norm:     out = norm(in0 + in1) * (w + weight_offset); in1 is the float32 stream [*, N], updated in
//                     place; rows_ctx: only these rows; defer_ok: the reader of out takes rows whose factor is missing
//   qkv_rope_cache:   out = in0 w^T + bias, w [N, K]; q and k heads rotated by table [max_pos, rot] at the positions
//                     ctx0; k and v stored in the pages at the slots ctx1 (none: not stored)
//   attention:        out = attention of the first nh * d columns of in0 over the pages, block tables ctx0
//   linear:           out = in0 w^T + bias in out_dtype; pending_ok: the reader of out takes an unfinished product;
//                     is_head: the result goes to the step's logits buffer
//   linear_gated:     out = act(in0 wg^T) * (in0 wu^T), w = [wg; wu] of N = 2 I rows; act 1: SiLU, 2: GELU
//   materialize:      out = in0 as a finished tensor
//   rope_cache_write: in0 [*, (nh + 2 nkv) d] rotated in place and stored, as the second half of qkv_rope_cache
//   gated_act:        out = act(in0[:, :I]) * in0[:, I:], N = 2 I; act as above
//   callback:         the caller's function (lmsf_program_set_callback) is called with ``callback_id`` and where
//                     in0, in1 and out lie; out has N columns of out_dtype and as many rows as in0 (as the step has
//                     wanted rows with rows_ctx, as the step has tokens without in0); out -1: the callback works on
//                     in0 in place; is_head: out is the step's logits buffer
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
  int callback_id;
} LmsfOpDesc;

// Where the attention plan of a step that is not all single tokens lies (lmsf_program_plan fills it): per tile
// size of the program's attention operations, the pairs (first flat index, tokens) of the tiles and the flat
// indices of the single tokens, as offsets in ints into the plan's array.
typedef struct {
  int n_plans;
  int tq[LMSF_MAX_PLANS], n_tiles[LMSF_MAX_PLANS], n_single[LMSF_MAX_PLANS];
  long tiles_at[LMSF_MAX_PLANS], single_at[LMSF_MAX_PLANS];
} LmsfPlanInfo;

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
  LmsfPlanInfo plan_info;             // and where its parts lie
  void* workspace;
  long workspace_bytes;
  float* logits;                      // [n_logit_rows, vocabulary]
  int* bad_flag;                      // set by the embedding when an id lies outside the vocabulary
} LmsfStepDesc;

// A tensor handed to a callback: bytes from the workspace's start (-1: none, -2: the logits buffer).
typedef struct {
  long offset;
  int rows, cols, dtype;
} LmsfTensorRef;
typedef struct {
  int callback_id;
  LmsfTensorRef in0, in1, out;
} LmsfCallbackArgs;
// Returns 0, or non-zero to stop the step with an error. Called on the thread that runs the step, between the
// launches before it and after it; whatever it launches belongs on the step's stream.
typedef int (*LmsfCallbackFn)(const LmsfCallbackArgs* args);

// What the last step that ran launched, by kind (lmsf_program_stats): the routes of dispatch.h for the products
// (plain, gated and QKV alike), then the kernels that take an unfinished product, then attention and callbacks.
enum {
  LMSF_STAT_NORM_OVER_PARTIALS = 16,
  LMSF_STAT_ROPE_OVER_PARTIALS,
  LMSF_STAT_REDUCE_PARTIALS,
  LMSF_STAT_PREFILL_ATTENTION,
  LMSF_STAT_DECODE_ATTENTION,
  LMSF_STAT_GENERIC_ATTENTION,
  LMSF_STAT_CALLBACK,
  LMSF_STAT_COUNT
};

void* lmsf_program_create(const LmsfTunables* tunables);
void lmsf_program_destroy(void* program);
int lmsf_program_add(void* program, const LmsfOpDesc* op);
int lmsf_program_seal(void* program);
void lmsf_program_set_callback(void* program, LmsfCallbackFn fn);
long lmsf_program_plan(void* program, int S, const int* seg_lens, const int* seg_first_pos, int* out, long capacity,
                       LmsfPlanInfo* info);
long lmsf_program_plan_capacity(void* program, int N);
int lmsf_program_run(void* program, const LmsfStepDesc* step, int check_only, hipStream_t stream);
int lmsf_program_stats(void* program, long* out, int capacity);

#ifdef __cplusplus
}
#endif
