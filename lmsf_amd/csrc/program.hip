// The step program: a model's kernel calls, recorded once from the parts, run for every step from C++.
//
// The reference's step is native code from the worker down (core/src/worker/model_worker.rs:213-264 calls
// core/src/model_executor/models/llama/llama.rs:397-476, which calls the kernels). Here the model is put
// together from parts in Python; what a step costs the host there is one interpreter call per kernel. So the
// parts' calls are recorded once (ops/program.py runs the model's forward over a recorder that stands in for
// the kernels) as a list of operations over value registers, and this file runs that list: it chooses the
// kernel for each operation from the step's number of rows exactly as ops/hip_ops.py does, takes every
// temporary from one workspace the caller owns, and launches. A step is one call, whatever it holds.
//
// A value is a tensor or one of three unfinished forms that the kernels hand to each other (see
// ops/handles.py): a product left as partial sums, a product not yet started, rows whose norm factor is still
// to come. Temporaries live in a ring: a register's memory is free again after the last operation that reads
// it; the few registers that live long (the residual stream) are taken from the other end of the workspace.
// Before anything is launched the whole step is walked once without launching, so a step that does not fit
// the workspace is refused with nothing done. Which kernel an operation runs in is not decided here: the
// functions of dispatch.h say, as they do for the Python face of the kernels. Products that go to the BLAS
// library are called through blas.hip, so a step of any number of tokens is one call. A part that the
// recorder could not follow (it computes on its activations itself) is a callback operation: the program
// hands the caller's function the places of its operands in the workspace and goes on after it returns.
#include "program.h"

#include "common.h"
#include "entry_points.h"

#include <algorithm>
#include <deque>
#include <utility>
#include <vector>

namespace {

enum { V_NONE = 0, V_TENSOR, V_PENDING, V_DEFERRED, V_SCALED };

struct Value {
  int kind = V_NONE;
  // tensor [M, N] of dtype, row stride ld (also the xw of scaled rows)
  void* p = nullptr;
  int dtype = LMSF_BF16, M = 0, N = 0;
  long ld = 0;
  // pending: float32 partial sums [n_split, M, N]; pending and deferred: the bias still to add
  float* partials = nullptr;
  int n_split = 0;
  const void* bias = nullptr;
  // deferred: x [M, K] and W [N, K]
  const void* x = nullptr;
  long ldx = 0;
  int K = 0;
  const void* W = nullptr;
  long ldw = 0;
  // scaled rows: sums of squares [tiles][rows_per_tile] and what the norm kernel would need instead
  float* sumsq = nullptr;
  int tiles = 0, rows_per_tile = 0;
  float eps = 0.f, weight_offset = 0.f;
  const void* norm_weight = nullptr;
  int norm_wdtype = LMSF_BF16;
  float* stream = nullptr;
};

struct Block {
  int reg;
  size_t begin, end;
};

struct Program {
  std::vector<LmsfOpDesc> ops;
  std::vector<int> last_use;        // per register: index of the last operation that reads it
  std::vector<int> first_def;
  std::vector<char> long_lived;
  int n_regs = 0;
  bool sealed = false;
  LmsfTunables tun;
  std::vector<int> tile_sizes;      // the distinct tile sizes of the attention operations
  LmsfCallbackFn callback = nullptr;
  mutable long stats[LMSF_STAT_COUNT] = {0};   // what the last step that ran launched
};

const int kLongLife = 12;   // a register read this many operations after it was written lives at the far end

struct Run {
  const Program* prog;
  const LmsfStepDesc* st;
  hipStream_t stream;
  bool dry;
  std::vector<Value> regs;
  std::deque<Block> ring;
  size_t tail = 0, limit = 0, far_at = 0;
  int op_index = 0, cur_reg = -1;
  bool cur_long = false;

  char* base() const { return (char*)st->workspace; }
  void count(int what) const {
    if (!dry && what >= 0 && what < LMSF_STAT_COUNT) ++prog->stats[what];
  }

  void release_dead() {
    while (!ring.empty() && (ring.front().reg < 0 || prog->last_use[ring.front().reg] < op_index)) ring.pop_front();
    if (ring.empty()) tail = 0;
  }

  // memory for the register that the current operation writes; null (error set) if the workspace is too small
  void* take(size_t bytes) {
    bytes = (bytes + 255) & ~(size_t)255;
    if (bytes == 0) bytes = 256;
    if (cur_long) {
      if (far_at < bytes || far_at - bytes < ring_high()) {
        lmsf_set_error("program: workspace of %ld bytes is too small", st->workspace_bytes);
        return nullptr;
      }
      far_at -= bytes;
      limit = far_at;
      return base() + far_at;
    }
    size_t at;
    if (ring.empty()) {
      at = 0;
    } else if (ring.back().begin >= ring.front().begin) {      // not wrapped
      at = tail;
      if (at + bytes > limit) {
        at = 0;                                                 // wrap
        if (bytes > ring.front().begin) at = (size_t)-1;
      }
    } else {
      at = tail;
      if (at + bytes > ring.front().begin) at = (size_t)-1;
    }
    if (at == (size_t)-1 || at + bytes > limit) {
      lmsf_set_error("program: workspace of %ld bytes is too small", st->workspace_bytes);
      return nullptr;
    }
    ring.push_back(Block{cur_reg, at, at + bytes});
    tail = at + bytes;
    return base() + at;
  }
  size_t ring_high() const {
    size_t h = 0;
    for (const Block& b : ring) h = std::max(h, b.end);
    return h;
  }
};

#define RC(call)              \
  do {                        \
    const int rc_ = (call);   \
    if (rc_ != 0) return rc_; \
  } while (0)
#define LAUNCH(call)                \
  do {                              \
    if (!r.dry) {                   \
      const int rc_ = (call);       \
      if (rc_ != 0) return rc_;     \
    }                               \
  } while (0)
#define TAKE(var, type, bytes)                     \
  type var = (type)r.take((size_t)(bytes));        \
  if (var == nullptr) return LMSF_PROGRAM_NO_ROOM

inline int esize(int dtype) { return dtype == LMSF_F32 ? 4 : 2; }

// what the functions of dispatch.h want to know of a product x W^T, W of ``w_rows`` rows
LmsfProductShape shape_of(const void* x, int x_dtype, long ldx, int M, int K, const void* W, int wdtype, long ldw,
                          int w_rows, int out_dtype) {
  LmsfProductShape s;
  s.M = M;
  s.N = w_rows;
  s.K = K;
  s.x_dtype = x_dtype;
  s.w_dtype = wdtype;
  s.out_dtype = out_dtype;
  s.ldx = ldx;
  s.ldw = ldw;
  s.x_ok16 = lmsf_aligned16(x);
  s.w_ok16 = lmsf_aligned16(W);
  return s;
}

Value tensor(void* p, int dtype, int M, int N) {
  Value v;
  v.kind = V_TENSOR;
  v.p = p;
  v.dtype = dtype;
  v.M = M;
  v.N = N;
  v.ld = N;
  return v;
}

int op_linear(Run& r, const Value& x, const void* W, int wdtype, long ldw, int N, const void* bias, int out_dtype,
              bool pending_ok, void* out, Value* res);

Value pending(float* partials, int splits, const void* bias, int dtype, int M, int N) {
  Value v;
  v.kind = V_PENDING;
  v.partials = partials;
  v.n_split = splits;
  v.bias = bias;
  v.dtype = dtype;
  v.M = M;
  v.N = N;
  return v;
}

// the 17-and-more-rows kernel; act 0: plain, else the gated activation over W's two halves
int linear_mid(Run& r, const Value& x, const void* W, long ldw, int w_rows, const void* bias, int act, int out_dtype,
               const LmsfRoute& rt, void* out, Value* res) {
  const int M = x.M, K = x.N;
  const int N = act ? w_rows / 2 : w_rows;
  if (rt.pending) {
    TAKE(partials, float*, (size_t)rt.splits * M * N * 4);
    LAUNCH(lmsf_gemm_mid_partial(x.p, x.ld, W, ldw, M, N, K, rt.splits, partials, r.stream));
    *res = pending(partials, rt.splits, bias, out_dtype, M, N);
    return 0;
  }
  const long floats = lmsf_gemm_mid_scratch_floats(M, N, rt.splits, act);
  float* scratch = nullptr;
  if (floats > 0) {
    TAKE(s, float*, (size_t)floats * 4);
    scratch = s;
  }
  void* y = out;
  if (y == nullptr) {
    TAKE(yy, void*, (size_t)M * N * esize(out_dtype));
    y = yy;
  }
  LAUNCH(lmsf_gemm_mid(x.p, x.ld, W, ldw, bias, y, out_dtype, N, M, N, K, act, rt.splits, scratch, r.stream));
  *res = tensor(y, out_dtype, M, N);
  return 0;
}

// the many-rows kernel
int linear_large(Run& r, const Value& x, const void* W, long ldw, int w_rows, const void* bias, int act,
                 const LmsfRoute& rt, void* out, Value* res) {
  const int M = x.M, K = x.N;
  const int N = act ? w_rows / 2 : w_rows;
  float* scratch = nullptr;
  if (rt.splits > 1) {
    TAKE(s, float*, (size_t)rt.splits * M * N * 4);
    scratch = s;
    if (rt.pending) {
      LAUNCH(lmsf_gemm_large(x.p, x.ld, W, ldw, nullptr, nullptr, 0, M, N, K, 0, rt.plan, scratch, 0, r.stream));
      *res = pending(scratch, rt.splits, bias, LMSF_BF16, M, N);
      return 0;
    }
  }
  void* y = out;
  if (y == nullptr) {
    TAKE(yy, void*, (size_t)M * N * 2);
    y = yy;
  }
  LAUNCH(lmsf_gemm_large(x.p, x.ld, W, ldw, bias, y, N, M, N, K, act, rt.plan, scratch, 1, r.stream));
  *res = tensor(y, LMSF_BF16, M, N);
  return 0;
}

// y = x W^T + bias (HipOps.linear launches the same kernels for the same routes)
int op_linear(Run& r, const Value& x, const void* W, int wdtype, long ldw, int N, const void* bias, int out_dtype,
              bool pending_ok, void* out, Value* res) {
  const LmsfTunables& t = r.prog->tun;
  if (x.kind != V_TENSOR) {
    lmsf_set_error("program: a product's operand is not a tensor");
    return 1;
  }
  const int M = x.M, K = x.N;
  const LmsfProductShape shape = shape_of(x.p, x.dtype, x.ld, M, K, W, wdtype, ldw, N, out_dtype);
  LmsfRoute rt;
  lmsf_route_linear(&t, &shape, pending_ok ? 1 : 0, &rt);
  if (rt.route != LMSF_ROUTE_CHUNKS) r.count(rt.route);
  if (rt.route == LMSF_ROUTE_MID) return linear_mid(r, x, W, ldw, N, bias, 0, out_dtype, rt, out, res);
  if (rt.route == LMSF_ROUTE_LARGE) return linear_large(r, x, W, ldw, N, bias, 0, rt, out, res);
  if (rt.route == LMSF_ROUTE_DEFERRED) {
    Value v;
    v.kind = V_DEFERRED;
    v.x = x.p;
    v.ldx = x.ld;
    v.K = K;
    v.W = W;
    v.ldw = ldw;
    v.bias = bias;
    v.dtype = out_dtype;
    v.M = M;
    v.N = N;
    *res = v;
    return 0;
  }
  void* y = out;
  if (y == nullptr) {
    TAKE(yy, void*, (size_t)M * N * esize(out_dtype));
    y = yy;
  }
  *res = tensor(y, out_dtype, M, N);
  switch (rt.route) {
    case LMSF_ROUTE_GEMV:
      LAUNCH(lmsf_gemv(x.p, x.ld, W, ldw, bias, y, out_dtype, N, M, N, K, 0, r.stream));
      return 0;
    case LMSF_ROUTE_CHUNKS:
      for (int r0 = 0; r0 < M; r0 += rt.chunk_rows) {
        Value xs = x;
        xs.p = (char*)x.p + (size_t)r0 * x.ld * esize(x.dtype);
        xs.M = std::min(rt.chunk_rows, M - r0);
        Value part;
        RC(op_linear(r, xs, W, wdtype, ldw, N, bias, out_dtype, false, (char*)y + (size_t)r0 * N * esize(out_dtype),
                     &part));
      }
      return 0;
    case LMSF_ROUTE_SKINNY:
      for (int r0 = 0; r0 < M; r0 += 64)
        LAUNCH(lmsf_gemm_skinny((const char*)x.p + (size_t)r0 * x.ld * 2, x.ld, W, ldw, bias,
                                (char*)y + (size_t)r0 * N * esize(out_dtype), out_dtype, N, std::min(64, M - r0), N, K,
                                t.skinny_variant, 0, r.stream));
      return 0;
    case LMSF_ROUTE_BLAS:
      LAUNCH(lmsf_blas_linear(x.p, x.ld, W, ldw, bias, y, N, M, N, K, r.stream));
      return 0;
    default:
      LAUNCH(lmsf_gemm_plain(x.p, x.dtype, x.ld, W, wdtype, ldw, bias, y, out_dtype, N, M, N, K, r.stream));
      return 0;
  }
}

int op_add_rms_norm(Run& r, const Value& branch, float* residual, int M, int H, const void* weight, int wdtype,
                    float eps, float weight_offset, int out_dtype, const int* rows, int n_rows, bool defer_ok,
                    Value* res);

// HipOps.materialize
int materialize(Run& r, const Value& v, Value* res) {
  if (v.kind == V_TENSOR) {
    *res = v;
    return 0;
  }
  if (v.kind == V_DEFERRED) {
    const Value x = tensor(const_cast<void*>(v.x), LMSF_BF16, v.M, v.K);
    Value xs = x;
    xs.ld = v.ldx;
    return op_linear(r, xs, v.W, LMSF_BF16, v.ldw, v.N, v.bias, v.dtype, false, nullptr, res);
  }
  if (v.kind == V_SCALED) {
    Value none;
    return op_add_rms_norm(r, none, v.stream, v.M, v.N, v.norm_weight, v.norm_wdtype, v.eps, v.weight_offset, v.dtype,
                           nullptr, 0, false, res);
  }
  if (v.kind == V_PENDING) {
    TAKE(y, void*, (size_t)v.M * v.N * esize(v.dtype));
    r.count(LMSF_STAT_REDUCE_PARTIALS);
    LAUNCH(lmsf_gemm_mid_reduce(v.partials, v.bias, y, v.dtype, v.N, v.M, v.N, v.n_split, r.stream));
    *res = tensor(y, v.dtype, v.M, v.N);
    return 0;
  }
  lmsf_set_error("program: an operation reads a register that holds nothing");
  return 1;
}

// HipOps.add_rms_norm, with _run_deferred and _add_rms_norm_pending. M: rows of the operands; rows/n_rows select
// input rows (n_rows outputs); residual may be null (norm of the branch alone).
int op_add_rms_norm(Run& r, const Value& branch_in, float* residual, int M, int H, const void* weight, int wdtype,
                    float eps, float weight_offset, int out_dtype, const int* rows, int n_rows, bool defer_ok,
                    Value* res) {
  const LmsfTunables& t = r.prog->tun;
  Value branch = branch_in;
  const int n_out = rows ? n_rows : M;
  if (branch.kind == V_PENDING) {
    const bool fits = H % 4 == 0 && H <= 16384 && lmsf_aligned16(weight) && (residual == nullptr || lmsf_aligned16(residual));
    if (fits && branch.N == H) {
      TAKE(out, void*, (size_t)n_out * H * esize(out_dtype));
      r.count(LMSF_STAT_NORM_OVER_PARTIALS);
      LAUNCH(lmsf_add_rms_norm_partial(branch.partials, branch.bias, branch.n_split, branch.M, residual, weight, wdtype,
                                       out, out_dtype, rows, n_out, H, eps, weight_offset, r.stream));
      *res = tensor(out, out_dtype, n_out, H);
      return 0;
    }
    Value m;
    RC(materialize(r, branch, &m));
    branch = m;
  }
  if (branch.kind == V_DEFERRED) {
    const int Mb = branch.M, N = branch.N, K = branch.K;
    const bool fits = rows == nullptr && residual != nullptr && Mb == M && N == H;
    const bool prepares = fits && defer_ok && out_dtype == LMSF_BF16 && wdtype == LMSF_BF16;
    LmsfRoute rt;
    lmsf_route_deferred_norm(&t, Mb, N, K, fits ? 1 : 0, prepares ? 1 : 0, &rt);
    if (rt.route != LMSF_ROUTE_MATERIALIZE) r.count(rt.route);
    if (rt.route == LMSF_ROUTE_GEMV_ADD_NORM || rt.route == LMSF_ROUTE_SKINNY_ADD_NORM) {
      const bool one_or_two = rt.route == LMSF_ROUTE_GEMV_ADD_NORM;
      const int tiles = one_or_two ? lmsf_gemv_partials(N) : (N + 15) / 16;
      const int rows_per_tile = one_or_two ? Mb : 16;
      TAKE(xw, void*, (size_t)Mb * N * 2 + 256 + (size_t)tiles * rows_per_tile * 4);
      float* sumsq = (float*)((char*)xw + (((size_t)Mb * N * 2 + 255) & ~(size_t)255));
      if (one_or_two)
        LAUNCH(lmsf_gemv_add_norm(branch.x, branch.ldx, branch.W, branch.ldw, branch.bias, residual, H, weight,
                                  weight_offset, xw, N, sumsq, Mb, N, K, r.stream));
      else
        LAUNCH(lmsf_gemm_skinny_add_norm(branch.x, branch.ldx, branch.W, branch.ldw, branch.bias, residual, H, weight,
                                         weight_offset, xw, N, sumsq, Mb, N, K, t.skinny_variant, r.stream));
      Value v = tensor(xw, LMSF_BF16, Mb, N);
      v.kind = V_SCALED;
      v.sumsq = sumsq;
      v.tiles = tiles;
      v.rows_per_tile = rows_per_tile;
      v.eps = eps;
      v.weight_offset = weight_offset;
      v.norm_weight = weight;
      v.norm_wdtype = wdtype;
      v.stream = residual;
      *res = v;
      return 0;
    }
    if (rt.route == LMSF_ROUTE_GEMV_ADD) {
      LAUNCH(lmsf_gemv_add(branch.x, branch.ldx, branch.W, branch.ldw, branch.bias, residual, H, Mb, N, K, r.stream));
      branch = Value();
    } else {
      Value m;
      RC(materialize(r, branch, &m));
      branch = m;
    }
  }
  if (branch.kind == V_SCALED) {
    Value m;
    RC(materialize(r, branch, &m));
    branch = m;
  }
  if (branch.kind == V_NONE && residual == nullptr) {
    lmsf_set_error("program: a norm without operands");
    return 1;
  }
  if (branch.kind == V_TENSOR && (branch.N != H || branch.ld != H || branch.M != M)) {
    lmsf_set_error("program: a norm's branch [%d, %d] does not fit its stream [%d, %d]", branch.M, branch.N, M, H);
    return 1;
  }
  TAKE(out, void*, (size_t)n_out * H * esize(out_dtype));
  LAUNCH(lmsf_add_rms_norm(branch.kind == V_TENSOR ? branch.p : nullptr, branch.kind == V_TENSOR ? branch.dtype : LMSF_F32,
                           residual, weight, wdtype, out, out_dtype, rows, n_out, H, eps, weight_offset, r.stream));
  *res = tensor(out, out_dtype, n_out, H);
  return 0;
}

// act(x Wg^T) * (x Wu^T); kind 1: SiLU, 2: GELU (HipOps.linear_gated launches the same kernels for the same routes)
int op_linear_gated(Run& r, const Value& x_in, const void* W, int wdtype, long ldw, int w_rows, const void* bias,
                    int kind, Value* res) {
  const LmsfTunables& t = r.prog->tun;
  Value x = x_in;
  const int I = w_rows / 2;
  LmsfRoute rt;
  if (x.kind == V_SCALED) {
    const LmsfProductShape shape = shape_of(x.p, x.dtype, x.ld, x.M, x.N, W, wdtype, ldw, w_rows, LMSF_BF16);
    lmsf_route_linear_gated(&t, &shape, x.rows_per_tile, x.tiles, &rt);
    if (rt.route != LMSF_ROUTE_MATERIALIZE) {
      r.count(rt.route);
      const int M = x.M, K = x.N;
      TAKE(y, void*, (size_t)M * I * 2);
      if (rt.route == LMSF_ROUTE_MID_SCALED)
        LAUNCH(lmsf_gemm_mid_scaled(x.p, x.ld, W, ldw, bias, y, I, M, I, K, kind, x.sumsq, x.tiles, x.eps, r.stream));
      else if (rt.route == LMSF_ROUTE_GEMV_SCALED)
        LAUNCH(lmsf_gemv_scaled(x.p, x.ld, W, ldw, bias, y, I, M, I, K, kind, x.sumsq, x.tiles, x.eps, r.stream));
      else
        LAUNCH(lmsf_gemm_skinny_scaled(x.p, x.ld, W, ldw, bias, y, I, M, I, K, kind, x.sumsq, x.tiles, x.eps,
                                       t.skinny_variant, r.stream));
      *res = tensor(y, LMSF_BF16, M, I);
      return 0;
    }
  }
  if (x.kind != V_TENSOR) {
    Value m;
    RC(materialize(r, x, &m));
    x = m;
  }
  const int M = x.M, K = x.N;
  const LmsfProductShape shape = shape_of(x.p, x.dtype, x.ld, M, K, W, wdtype, ldw, w_rows, x.dtype);
  lmsf_route_linear_gated(&t, &shape, 0, 0, &rt);
  if (rt.route != LMSF_ROUTE_SEPARATE) r.count(rt.route);
  if (rt.route == LMSF_ROUTE_GEMV || rt.route == LMSF_ROUTE_SKINNY) {
    TAKE(y, void*, (size_t)M * I * 2);
    if (rt.route == LMSF_ROUTE_GEMV)
      LAUNCH(lmsf_gemv(x.p, x.ld, W, ldw, bias, y, LMSF_BF16, I, M, I, K, kind, r.stream));
    else
      LAUNCH(lmsf_gemm_skinny(x.p, x.ld, W, ldw, bias, y, LMSF_BF16, I, M, I, K, t.skinny_variant, kind, r.stream));
    *res = tensor(y, LMSF_BF16, M, I);
    return 0;
  }
  if (rt.route == LMSF_ROUTE_MID) return linear_mid(r, x, W, ldw, w_rows, bias, kind, LMSF_BF16, rt, nullptr, res);
  if (rt.route == LMSF_ROUTE_LARGE) return linear_large(r, x, W, ldw, w_rows, bias, kind, rt, nullptr, res);
  Value gu;
  RC(op_linear(r, x, W, wdtype, ldw, w_rows, bias, x.dtype, false, nullptr, &gu));
  TAKE(y, void*, (size_t)M * I * esize(gu.dtype));
  LAUNCH(lmsf_gated_act(gu.p, y, gu.dtype, M, I, gu.ld, kind - 1, r.stream));
  *res = tensor(y, gu.dtype, M, I);
  return 0;
}

int rope_cache_write(Run& r, const Value& qkv, const LmsfOpDesc& op, const int* positions, const int* slots) {
  const int es = esize(qkv.dtype);
  char* b = (char*)qkv.p;
  const bool rot = op.table != nullptr;
  LAUNCH(lmsf_rope_cache_write(b, b + (size_t)op.nh * op.d * es, b + (size_t)(op.nh + op.nkv) * op.d * es, qkv.dtype,
                               qkv.M, qkv.ld, rot ? positions : nullptr, (const float*)op.table, rot ? op.rot : 0,
                               op.neox, rot ? op.max_pos : 0, slots, slots ? op.k_pages : nullptr,
                               slots ? op.v_pages : nullptr, slots ? op.num_pages : 0, op.nh, op.nkv, op.d,
                               slots ? op.ps : 1, r.stream));
  return 0;
}

// The QKV product with rotation and cache write (HipOps.qkv_rope_cache launches the same kernels for the same routes)
int op_qkv_rope_cache(Run& r, const Value& x_in, const LmsfOpDesc& op, const int* positions, const int* slots,
                      Value* res) {
  const LmsfTunables& t = r.prog->tun;
  Value x = x_in;
  const int N = (op.nh + 2 * op.nkv) * op.d;
  const float* table = (const float*)op.table;
  const auto fused_shape = [&](int K) {
    return table != nullptr && slots != nullptr && op.neox && op.rot == op.d && op.d % 32 == 0 &&
           op.wdtype == LMSF_BF16 && op.N == N && op.K == K && op.k_pages != nullptr && op.cache_dtype == LMSF_BF16;
  };
  LmsfRoute rt;
  if (x.kind == V_SCALED) {
    const int M = x.M, K = x.N;
    const LmsfProductShape shape = shape_of(x.p, x.dtype, x.ld, M, K, op.w, op.wdtype, op.ldw, op.N, LMSF_BF16);
    lmsf_route_qkv(&t, &shape, fused_shape(K) ? 1 : 0, x.rows_per_tile, &rt);
    if (rt.route != LMSF_ROUTE_MATERIALIZE) {
      r.count(rt.route);
      TAKE(y, void*, (size_t)M * N * 2);
      if (rt.route == LMSF_ROUTE_GEMV_SCALED)
        LAUNCH(lmsf_gemv_scaled_qkv_rope_cache(x.p, x.ld, op.w, op.ldw, op.bias, y, N, M, K, positions, table,
                                               op.max_pos, slots, op.k_pages, op.v_pages, op.num_pages, op.nh, op.nkv,
                                               op.d, op.ps, x.sumsq, x.tiles, x.eps, r.stream));
      else
        LAUNCH(lmsf_gemm_qkv_rope_cache_scaled(x.p, x.ld, op.w, op.ldw, op.bias, y, N, M, K, positions, table,
                                               op.max_pos, slots, op.k_pages, op.v_pages, op.num_pages, op.nh, op.nkv,
                                               op.d, op.ps, x.sumsq, x.tiles, x.eps, r.stream));
      *res = tensor(y, LMSF_BF16, M, N);
      return 0;
    }
  }
  if (x.kind != V_TENSOR) {
    Value m;
    RC(materialize(r, x, &m));
    x = m;
  }
  const int M = x.M, K = x.N;
  const LmsfProductShape shape = shape_of(x.p, x.dtype, x.ld, M, K, op.w, op.wdtype, op.ldw, op.N, x.dtype);
  lmsf_route_qkv(&t, &shape, fused_shape(K) ? 1 : 0, 0, &rt);
  if (rt.route != LMSF_ROUTE_SEPARATE) r.count(rt.route);
  if (rt.route == LMSF_ROUTE_GEMV || rt.route == LMSF_ROUTE_SKINNY) {
    TAKE(y, void*, (size_t)M * N * 2);
    if (rt.route == LMSF_ROUTE_GEMV)
      LAUNCH(lmsf_gemv_qkv_rope_cache(x.p, x.ld, op.w, op.ldw, op.bias, y, N, M, K, positions, table, op.max_pos, slots,
                                      op.k_pages, op.v_pages, op.num_pages, op.nh, op.nkv, op.d, op.ps, r.stream));
    else
      LAUNCH(lmsf_gemm_qkv_rope_cache(x.p, x.ld, op.w, op.ldw, op.bias, y, N, M, K, positions, table, op.max_pos, slots,
                                      op.k_pages, op.v_pages, op.num_pages, op.nh, op.nkv, op.d, op.ps,
                                      t.skinny_variant, r.stream));
    *res = tensor(y, LMSF_BF16, M, N);
    return 0;
  }
  Value y;
  RC(op_linear(r, x, op.w, op.wdtype, op.ldw, op.N, op.bias, x.dtype, rt.pending != 0, nullptr, &y));
  if (y.kind == V_PENDING) {
    if ((table == nullptr && slots == nullptr) || op.N != N) {
      Value m;
      RC(materialize(r, y, &m));
      *res = m;
      return 0;
    }
    if (slots != nullptr && op.cache_dtype != LMSF_BF16) {
      lmsf_set_error("program: a bfloat16 projection writes a cache of another type");
      return 1;
    }
    TAKE(out, void*, (size_t)M * N * 2);
    const bool rot = table != nullptr;
    r.count(LMSF_STAT_ROPE_OVER_PARTIALS);
    LAUNCH(lmsf_rope_cache_write_partial(y.partials, y.bias, y.n_split, out, N, M, rot ? positions : nullptr, table,
                                         rot ? op.rot : 0, op.neox, rot ? op.max_pos : 0, slots,
                                         slots ? op.k_pages : nullptr, slots ? op.v_pages : nullptr,
                                         slots ? op.num_pages : 0, op.nh, op.nkv, op.d, slots ? op.ps : 1, r.stream));
    *res = tensor(out, LMSF_BF16, M, N);
    return 0;
  }
  if (y.kind != V_TENSOR) {
    Value m;
    RC(materialize(r, y, &m));
    y = m;
  }
  if (table != nullptr || slots != nullptr) {
    if (op.N != N) {
      lmsf_set_error("program: the projection has %d columns, its heads ask for %d", op.N, N);
      return 1;
    }
    if (slots != nullptr && op.cache_dtype != y.dtype) {
      lmsf_set_error("program: the projection and its cache differ in type");
      return 1;
    }
    RC(rope_cache_write(r, y, op, positions, slots));
  }
  *res = y;
  return 0;
}

// Attention over the pages (HipOps.paged_attention launches the same kernels)
int op_attention(Run& r, const Value& q, const LmsfOpDesc& op, const int* tables, int width, Value* res) {
  const LmsfStepDesc& st = *r.st;
  const LmsfTunables& t = r.prog->tun;
  if (q.kind != V_TENSOR || q.N < op.nh * op.d) {
    lmsf_set_error("program: attention needs a tensor of at least %d columns", op.nh * op.d);
    return 1;
  }
  if (op.cache_dtype != q.dtype) {
    lmsf_set_error("program: queries and cache differ in type");
    return 1;
  }
  const int N = q.M, nh = op.nh, nkv = op.nkv, d = op.d, ps = op.ps;
  TAKE(out, void*, (size_t)N * nh * d * esize(q.dtype));
  *res = tensor(out, q.dtype, N, nh * d);
  if (N == 0) return 0;
  const bool fast_ok = q.dtype == LMSF_BF16 && d % 16 == 0 && 16 <= d && d <= 256 && ps % 4 == 0 && q.ld % 8 == 0 &&
                       lmsf_aligned16(q.p) && op.scale > 0.f;
  if (!fast_ok) {
    r.count(LMSF_STAT_GENERIC_ATTENTION);
    LAUNCH(lmsf_paged_attention_generic(q.p, q.ld, out, (long)nh * d, op.k_pages, op.v_pages, op.num_pages, tables, width,
                                        st.seg_of, st.positions, N, nh, nkv, d, ps, op.scale, op.window, q.dtype,
                                        r.stream));
    return 0;
  }
  const int* tiles = nullptr;
  const int* single = nullptr;
  int n_tiles = 0, n_single = 0;
  const int max_context = st.max_context;
  if (st.all_single) {
    // the order matters from 16 tokens on (the kernel starts the longest contexts first); below that the tokens
    // are taken as they come, which saves the kernel the trip to the list
    single = N >= 16 ? st.longest_first : nullptr;
    n_single = N;
  } else {
    const int tq = lmsf_attention_tile_tokens(nh, nkv);
    const LmsfPlanInfo& info = st.plan_info;
    int at = -1;
    for (int i = 0; i < info.n_plans && i < LMSF_MAX_PLANS; ++i)
      if (info.tq[i] == tq) at = i;
    if (at < 0 || st.plan == nullptr || info.n_tiles[at] + info.n_single[at] <= 0) {
      lmsf_set_error("program: the step carries no attention plan for tiles of %d tokens", tq);
      return 1;
    }
    n_tiles = info.n_tiles[at];
    n_single = info.n_single[at];
    tiles = n_tiles ? st.plan + info.tiles_at[at] : nullptr;
    single = n_single ? st.plan + info.single_at[at] : nullptr;
  }
  if (n_tiles) r.count(LMSF_STAT_PREFILL_ATTENTION);
  if (n_single) r.count(LMSF_STAT_DECODE_ATTENTION);
  if (n_tiles)
    LAUNCH(lmsf_paged_attention_prefill_mfma(q.p, q.ld, out, (long)nh * d, op.k_pages, op.v_pages, op.num_pages, tables,
                                             width, tiles, n_tiles, st.seg_of, st.positions, nh, nkv, d, ps, op.scale,
                                             op.window, t.prefill_attention_variant, r.stream));
  if (n_single) {
    int chunk = 0, n_splits = 0;
    lmsf_route_decode_attention(&t, n_single, nh, nkv, max_context, &chunk, &n_splits);
    const long floats = n_splits > 1 ? lmsf_attention_decode_scratch_floats(n_single, nh, d, n_splits) : 1;
    TAKE(scratch, float*, (size_t)floats * 4);
    LAUNCH(lmsf_paged_attention_decode_mfma(q.p, q.ld, out, (long)nh * d, op.k_pages, op.v_pages, op.num_pages, tables,
                                            width, single, n_single, st.all_single ? nullptr : st.seg_of, st.positions, nh, nkv,
                                            d, ps, op.scale, op.window, chunk, n_splits, scratch, t.decode_attention_order,
                                            r.stream));
  }
  return 0;
}

const int* step_array(const LmsfStepDesc& st, int code, int* width) {
  if (width) *width = 0;
  switch (code) {
    case LMSF_CTX_TOKEN_IDS: return st.token_ids;
    case LMSF_CTX_POSITIONS: return st.positions;
    case LMSF_CTX_SEG_OF: return st.seg_of;
    case LMSF_CTX_LOGIT_ROWS: return st.logit_rows;
    default: break;
  }
  if (code >= LMSF_CTX_SLOTS && code < LMSF_CTX_SLOTS + LMSF_MAX_GROUPS) return st.slots[code - LMSF_CTX_SLOTS];
  if (code >= LMSF_CTX_TABLES && code < LMSF_CTX_TABLES + LMSF_MAX_GROUPS) {
    if (width) *width = st.widths[code - LMSF_CTX_TABLES];
    return st.tables[code - LMSF_CTX_TABLES];
  }
  return nullptr;
}

int run_pass(const Program& prog, const LmsfStepDesc& st, hipStream_t stream, bool dry) {
  Run r;
  r.prog = &prog;
  r.st = &st;
  r.stream = stream;
  r.dry = dry;
  r.regs.assign(prog.n_regs, Value());
  r.far_at = r.limit = (size_t)st.workspace_bytes & ~(size_t)255;   // (everything handed out is 256-byte aligned)
  const int N = st.n_tokens, R = st.n_logit_rows;
  for (size_t i = 0; i < prog.ops.size(); ++i) {
    const LmsfOpDesc& op = prog.ops[i];
    r.op_index = (int)i;
    r.release_dead();
    r.cur_reg = op.out;
    r.cur_long = op.out >= 0 && prog.long_lived[op.out];
    if (op.rows_ctx != LMSF_CTX_NONE && R == 0) break;   // nothing is wanted: the step ends before the head
    Value none, res;
    const Value& in0 = op.in0 >= 0 ? r.regs[op.in0] : none;
    switch (op.kind) {
      case LMSF_OP_EMBEDDING: {
        TAKE(out, float*, (size_t)N * op.N * 4);
        LAUNCH(lmsf_embedding(step_array(st, op.ctx0, nullptr), op.w, op.wdtype, out, N, op.N, op.vocab, op.scale,
                              st.bad_flag, stream));
        res = tensor(out, LMSF_F32, N, op.N);
        break;
      }
      case LMSF_OP_ADD_RMS_NORM: {
        float* residual = nullptr;
        int M = N;
        if (op.in1 >= 0) {
          const Value& s = r.regs[op.in1];
          if (s.kind != V_TENSOR || s.dtype != LMSF_F32 || s.N != op.N || s.ld != op.N) {
            lmsf_set_error("program: a norm's stream is not a float32 tensor of %d columns", op.N);
            return 1;
          }
          residual = (float*)s.p;
          M = s.M;
        } else if (in0.kind != V_NONE) {
          M = in0.M;
        }
        const int* rows = op.rows_ctx != LMSF_CTX_NONE ? step_array(st, op.rows_ctx, nullptr) : nullptr;
        RC(op_add_rms_norm(r, in0, residual, M, op.N, op.w, op.wdtype, op.eps, op.weight_offset, op.out_dtype, rows, R,
                           op.defer_ok != 0, &res));
        break;
      }
      case LMSF_OP_QKV_ROPE_CACHE:
        RC(op_qkv_rope_cache(r, in0, op, step_array(st, op.ctx0, nullptr),
                             op.ctx1 != LMSF_CTX_NONE ? step_array(st, op.ctx1, nullptr) : nullptr, &res));
        break;
      case LMSF_OP_ATTENTION: {
        int width = 0;
        const int* tables = step_array(st, op.ctx0, &width);
        RC(op_attention(r, in0, op, tables, width, &res));
        break;
      }
      case LMSF_OP_LINEAR: {
        Value x = in0;
        if (x.kind != V_TENSOR) {
          Value m;
          RC(materialize(r, in0, &m));
          x = m;
        }
        void* out = nullptr;
        if (op.is_head) {
          if (st.logits == nullptr) {
            lmsf_set_error("program: the step has no buffer for its logits");
            return 1;
          }
          out = st.logits;
        }
        RC(op_linear(r, x, op.w, op.wdtype, op.ldw, op.N, op.bias, op.out_dtype, op.pending_ok != 0 && !op.is_head, out,
                     &res));
        break;
      }
      case LMSF_OP_LINEAR_GATED:
        RC(op_linear_gated(r, in0, op.w, op.wdtype, op.ldw, op.N, op.bias, op.act, &res));
        break;
      case LMSF_OP_MATERIALIZE:
        RC(materialize(r, in0, &res));
        break;
      case LMSF_OP_ROPE_CACHE_WRITE: {
        if (in0.kind != V_TENSOR || in0.N != (op.nh + 2 * op.nkv) * op.d) {
          lmsf_set_error("program: rotation and cache write need a tensor of %d columns", (op.nh + 2 * op.nkv) * op.d);
          return 1;
        }
        const int* slots = op.ctx1 != LMSF_CTX_NONE ? step_array(st, op.ctx1, nullptr) : nullptr;
        if (slots != nullptr && op.cache_dtype != in0.dtype) {
          lmsf_set_error("program: the projection and its cache differ in type");
          return 1;
        }
        RC(rope_cache_write(r, in0, op, op.ctx0 != LMSF_CTX_NONE ? step_array(st, op.ctx0, nullptr) : nullptr, slots));
        break;
      }
      case LMSF_OP_GATED_ACT: {
        if (in0.kind != V_TENSOR || in0.N != op.N || op.N % 2 != 0) {
          lmsf_set_error("program: a gated activation needs a tensor of %d columns", op.N);
          return 1;
        }
        TAKE(y, void*, (size_t)in0.M * (op.N / 2) * esize(in0.dtype));
        LAUNCH(lmsf_gated_act(in0.p, y, in0.dtype, in0.M, op.N / 2, in0.ld, op.act - 1, stream));
        res = tensor(y, in0.dtype, in0.M, op.N / 2);
        break;
      }
      case LMSF_OP_CALLBACK: {
        const Value& in1 = op.in1 >= 0 ? r.regs[op.in1] : none;
        for (const Value* v : {&in0, &in1})
          if (v->kind != V_NONE && (v->kind != V_TENSOR || v->ld != v->N)) {
            lmsf_set_error("program: a callback's operand is not a finished tensor");
            return 1;
          }
        if (prog.callback == nullptr) {
          lmsf_set_error("program: a callback operation, and no function to call");
          return 1;
        }
        const auto ref = [&](const Value& v) {
          LmsfTensorRef t;
          t.offset = v.kind == V_NONE ? -1 : v.p == (void*)st.logits ? -2 : (long)((char*)v.p - r.base());
          t.rows = v.M;
          t.cols = v.N;
          t.dtype = v.dtype;
          return t;
        };
        LmsfCallbackArgs args;
        args.callback_id = op.callback_id;
        args.in0 = ref(in0);
        args.in1 = ref(in1);
        if (op.out >= 0) {
          const int rows = op.rows_ctx != LMSF_CTX_NONE ? R : in0.kind != V_NONE ? in0.M : N;
          void* y = nullptr;
          if (op.is_head) {
            if (st.logits == nullptr) {
              lmsf_set_error("program: the step has no buffer for its logits");
              return 1;
            }
            y = st.logits;
          } else {
            TAKE(yy, void*, (size_t)rows * op.N * esize(op.out_dtype));
            y = yy;
          }
          res = tensor(y, op.out_dtype, rows, op.N);
        }
        args.out = ref(res);
        r.count(LMSF_STAT_CALLBACK);
        if (!r.dry && prog.callback(&args) != 0) {
          lmsf_set_error("program: callback %d failed", op.callback_id);
          return 1;
        }
        break;
      }
      default:
        lmsf_set_error("program: unknown operation %d", op.kind);
        return 1;
    }
    if (op.out >= 0) r.regs[op.out] = res;
  }
  return 0;
}

}  // namespace

extern "C" void* lmsf_program_create(const LmsfTunables* tunables) {
  Program* p = new Program();
  p->tun = *tunables;
  return p;
}

extern "C" void lmsf_program_destroy(void* program) { delete static_cast<Program*>(program); }

extern "C" int lmsf_program_add(void* program, const LmsfOpDesc* op) {
  Program* p = static_cast<Program*>(program);
  LMSF_CHECK(p && op, "program_add: null pointer");
  LMSF_CHECK(!p->sealed, "program_add: the program is sealed");
  LMSF_CHECK(op->kind > 0 && op->kind < LMSF_OP_COUNT, "program_add: unknown operation %d", op->kind);
  for (int reg : {op->in0, op->in1}) LMSF_CHECK(reg < p->n_regs, "program_add: operation reads register %d before it is written", reg);
  LMSF_CHECK(op->out <= p->n_regs, "program_add: registers are numbered in the order they are written");
  p->ops.push_back(*op);
  if (op->out == p->n_regs) ++p->n_regs;
  return 0;
}

extern "C" int lmsf_program_seal(void* program) {
  Program* p = static_cast<Program*>(program);
  LMSF_CHECK(p, "program_seal: null pointer");
  p->last_use.assign(p->n_regs, -1);
  p->first_def.assign(p->n_regs, -1);
  p->long_lived.assign(p->n_regs, 0);
  p->tile_sizes.clear();
  for (size_t i = 0; i < p->ops.size(); ++i) {
    const LmsfOpDesc& op = p->ops[i];
    if (op.out >= 0 && p->first_def[op.out] < 0) p->first_def[op.out] = (int)i;
    for (int reg : {op.in0, op.in1})
      if (reg >= 0) p->last_use[reg] = (int)i;
    if (op.kind == LMSF_OP_ATTENTION) {
      const int tq = lmsf_attention_tile_tokens(op.nh, op.nkv);
      if (std::find(p->tile_sizes.begin(), p->tile_sizes.end(), tq) == p->tile_sizes.end()) p->tile_sizes.push_back(tq);
    }
  }
  LMSF_CHECK(p->tile_sizes.size() <= LMSF_MAX_PLANS, "program_seal: attention with more than %d tile sizes", LMSF_MAX_PLANS);
  // an unfinished value points into the memory of the register it was made from (a product not yet started reads
  // its operand when the norm runs it; scaled rows are finished from the stream): the operand lives as long
  for (int pass = 0; pass < 2; ++pass)
    for (size_t i = 0; i < p->ops.size(); ++i) {
      const LmsfOpDesc& op = p->ops[i];
      if (op.out < 0) continue;
      for (int reg : {op.in0, op.in1})
        if (reg >= 0) p->last_use[reg] = std::max(p->last_use[reg], p->last_use[op.out]);
    }
  for (int reg = 0; reg < p->n_regs; ++reg)
    p->long_lived[reg] = p->last_use[reg] - p->first_def[reg] > kLongLife;
  p->sealed = true;
  return 0;
}

extern "C" void lmsf_program_set_callback(void* program, LmsfCallbackFn fn) {
  if (program) static_cast<Program*>(program)->callback = fn;
}

// Host side of a step that is not all single tokens: the attention plan, for every tile size the program's
// attention operations use, written to ``out`` (host memory that the caller copies to the device with the step's
// other arrays; LmsfStepDesc.plan is its device address) and described in ``info``, which travels with the step
// (LmsfStepDesc.plan_info): nothing of a plan is kept here. Per tile size: pairs (first flat index, tokens) of
// the tiles of requests with several tokens, those with the most keys first, then the flat indices of the
// requests with one token, the longest context first. Returns the number of ints written, or -1.
extern "C" long lmsf_program_plan(void* program, int S, const int* seg_lens, const int* seg_first_pos, int* out,
                                  long capacity, LmsfPlanInfo* info) {
  const Program* p = static_cast<const Program*>(program);
  if (!p || !p->sealed || !info || S < 0 || (S > 0 && (!seg_lens || !seg_first_pos))) {
    lmsf_set_error("program_plan: bad arguments");
    return -1;
  }
  long at = 0;
  info->n_plans = 0;
  for (const int tq : p->tile_sizes) {
    std::vector<std::pair<int, std::pair<int, int>>> tiles;   // keys, (start, n)
    std::vector<std::pair<int, int>> single;                  // first position, flat index
    int flat = 0;
    for (int s = 0; s < S; ++s) {
      const int n = seg_lens[s], p0 = seg_first_pos[s];
      if (n == 1) {
        single.push_back({p0, flat});
      } else {
        for (int t = 0; t < n; t += tq) {
          const int m = std::min(tq, n - t);
          tiles.push_back({p0 + t + m, {flat + t, m}});
        }
      }
      flat += n;
    }
    std::stable_sort(tiles.begin(), tiles.end(), [](const auto& a, const auto& b) { return a.first > b.first; });
    std::stable_sort(single.begin(), single.end(), [](const auto& a, const auto& b) { return a.first > b.first; });
    const long need = (long)tiles.size() * 2 + (long)single.size();
    if (at + need + 8 > capacity) {
      lmsf_set_error("program_plan: %ld ints do not fit the %ld given", at + need, capacity);
      return -1;
    }
    const int i = info->n_plans++;
    info->tq[i] = tq;
    info->tiles_at[i] = at;
    info->n_tiles[i] = (int)tiles.size();
    for (const auto& t : tiles) {
      out[at++] = t.second.first;
      out[at++] = t.second.second;
    }
    at = (at + 3) / 4 * 4;
    info->single_at[i] = at;
    info->n_single[i] = (int)single.size();
    for (const auto& s : single) out[at++] = s.second;
    at = (at + 3) / 4 * 4;
  }
  return at;
}

// Ints that lmsf_program_plan writes at most for a step of N tokens.
extern "C" long lmsf_program_plan_capacity(void* program, int N) {
  Program* p = static_cast<Program*>(program);
  if (!p) return 0;
  return (long)std::max<size_t>(1, p->tile_sizes.size()) * (2L * N + N + 16);
}

// Runs the step. 0: done. LMSF_PROGRAM_NO_ROOM: the workspace is too small, nothing was launched. Other values:
// an error (lmsf_last_error), possibly after some kernels were launched. ``check_only``: walk the step, launch
// nothing (the workspace's address is then never used, only its size).
extern "C" int lmsf_program_run(void* program, const LmsfStepDesc* step, int check_only, hipStream_t stream) {
  Program* p = static_cast<Program*>(program);
  LMSF_CHECK(p && step, "program_run: null pointer");
  LMSF_CHECK(p->sealed, "program_run: the program is not sealed");
  LMSF_CHECK(step->n_tokens > 0 && step->n_segments > 0 && step->n_logit_rows >= 0, "program_run: an empty step");
  LMSF_CHECK(step->n_groups >= 0 && step->n_groups <= LMSF_MAX_GROUPS, "program_run: %d cache groups", step->n_groups);
  LMSF_CHECK(step->workspace != nullptr && step->workspace_bytes > 0 && (((uintptr_t)step->workspace) & 255) == 0,
             "program_run: the workspace must be 256-byte aligned device memory");
  LMSF_CHECK(step->token_ids && step->positions && step->seg_of, "program_run: the step's arrays are missing");
  LMSF_CHECK(!step->all_single || step->longest_first, "program_run: a step of single tokens carries their order");
  const int rc = run_pass(*p, *step, stream, true);
  if (rc != 0 || check_only) return rc;
  std::fill(p->stats, p->stats + LMSF_STAT_COUNT, 0L);
  return run_pass(*p, *step, stream, false);
}

// What the last step that ran launched, by kind (the indices of program.h); returns how many were written.
extern "C" int lmsf_program_stats(void* program, long* out, int capacity) {
  const Program* p = static_cast<const Program*>(program);
  if (!p || !out) return 0;
  const int n = std::min(capacity, (int)LMSF_STAT_COUNT);
  std::copy(p->stats, p->stats + n, out);
  return n;
}
