// Declarations of the kernel entry points of this library, for the code inside it that calls them (the step
// program) and for C or C++ callers outside. Each is documented where it is defined; all return 0 on success
// and non-zero with lmsf_last_error() set otherwise, unless they return a size.
#pragma once

#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif

// attention_generic.hip
int lmsf_paged_attention_generic(const void* q, long q_stride, void* out, long out_stride, const void* k_pages, const
    void* v_pages, long num_pages, const int* block_tables, int bt_width, const int* seg, const int* pos, int
    n_tokens, int nh, int nkv, int d, int ps, float scale, int window, int dtype, hipStream_t stream);

// attention_mfma.hip
int lmsf_attention_tile_tokens(int nh, int nkv);
int lmsf_paged_attention_prefill_mfma(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
    const void* v_pages, long num_pages, const int* block_tables, int btw, const int* tiles, int n_tiles, const int*
    seg, const int* pos, int nh, int nkv, int d, int ps, float scale, int window, int variant, hipStream_t stream);
long lmsf_attention_decode_scratch_floats(int n, int nh, int d, int n_splits);
int lmsf_paged_attention_decode_mfma(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
    const void* v_pages, long num_pages, const int* block_tables, int btw, const int* tok_idx, int n, const int* seg,
    const int* pos, int nh, int nkv, int d, int ps, float scale, int window, int chunk, int n_splits, float* scratch,
    int order, hipStream_t stream);

// blas.hip
int lmsf_blas_init(long workspace_bytes);
int lmsf_blas_ready();
int lmsf_blas_linear(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int M, int
    N, int K, hipStream_t stream);
int lmsf_blas_tune(const void* x, long ldx, const void* const* Ws, int n_weights, long ldw, const void* bias, void* y,
    long ldy, int M, int N, int K, int n_candidates, int reps, float* times_us, hipStream_t stream);
long lmsf_blas_plans();

// elementwise.hip
int lmsf_embedding(const int* ids, const void* table, int table_dtype, float* out, int n_tokens, int H, int V, float
    scale, int* bad_flag, hipStream_t stream);
int lmsf_gated_act(const void* in, void* out, int dtype, int n_tokens, int I, long in_stride, int kind, hipStream_t
    stream);

// gemm_large.hip
int lmsf_gemm_large_plan(int M, int N, int K, int act);
long lmsf_gemm_large_scratch_floats(int M, int N, int n_split);
int lmsf_gemm_large(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int M, int
    N, int K, int act, int plan, float* scratch, int reduce, hipStream_t stream);

// gemm_mid.hip
int lmsf_gemm_mid_splits(int M, int N, int K, int act);
long lmsf_gemm_mid_scratch_floats(int M, int N, int n_split, int act);
int lmsf_gemm_mid(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, int out_dtype, long
    ldy, int M, int N, int K, int act, int n_split, float* scratch, hipStream_t stream);
int lmsf_gemm_mid_scaled_fits(int M, int N, int K, int in_tiles);
int lmsf_gemm_mid_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int M,
    int N, int K, int act, const float* sumsq, int in_tiles, float eps, hipStream_t stream);
int lmsf_gemm_mid_partial(const void* x, long ldx, const void* W, long ldw, int M, int N, int K, int n_split, float*
    scratch, hipStream_t stream);
int lmsf_gemm_mid_reduce(const float* scratch, const void* bias, void* y, int out_dtype, long ldy, int M, int N, int
    n_split, hipStream_t stream);

// gemm_plain.hip
int lmsf_gemm_plain(const void* A, int a_dtype, long lda, const void* W, int w_dtype, long ldw, const void* bias,
    void* C, int c_dtype, long ldc, int M, int N, int K, hipStream_t stream);

// gemm_skinny.hip
int lmsf_gemm_skinny(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, int out_dtype, long
    ldy, int M, int N, int K, int variant, int act, hipStream_t stream);
int lmsf_gemm_qkv_rope_cache(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
    int M, int K, const int* positions, const float* table, int max_pos, const int* slots, void* k_pages, void*
    v_pages, long num_pages, int nh, int nkv, int d, int ps, int variant, hipStream_t stream);
int lmsf_gemm_skinny_add_norm(const void* x, long ldx, const void* W, long ldw, const void* bias, void* stream_f32,
    long ld_stream, const void* norm_weight, float weight_offset, void* xw, long ld_xw, float* sumsq, int M, int N,
    int K, int variant, hipStream_t stream);
int lmsf_gemm_skinny_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int
    M, int N, int K, int act, const float* sumsq, int in_tiles, float eps, int variant, hipStream_t stream);
int lmsf_gemm_qkv_rope_cache_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long
    ldy, int M, int K, const int* positions, const float* table, int max_pos, const int* slots, void* k_pages, void*
    v_pages, long num_pages, int nh, int nkv, int d, int ps, const float* sumsq, int in_tiles, float eps, hipStream_t
    stream);

// gemv.hip
int lmsf_gemv(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, int out_dtype, long ldy,
    int M, int N, int K, int act, hipStream_t stream);
int lmsf_gemv_qkv_rope_cache(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy,
    int M, int K, const int* positions, const float* table, int max_pos, const int* slots, void* k_pages, void*
    v_pages, long num_pages, int nh, int nkv, int d, int ps, hipStream_t stream);
int lmsf_gemv_add(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int M, int N,
    int K, hipStream_t stream);
int lmsf_gemv_partials(int N);
int lmsf_gemv_add_norm(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, const
    void* norm_weight, float weight_offset, void* xw, long ld_xw, float* sumsq, int M, int N, int K, hipStream_t
    stream);
int lmsf_gemv_scaled(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long ldy, int M, int
    N, int K, int act, const float* sumsq, int n_partials, float eps, hipStream_t stream);
int lmsf_gemv_scaled_qkv_rope_cache(const void* x, long ldx, const void* W, long ldw, const void* bias, void* y, long
    ldy, int M, int K, const int* positions, const float* table, int max_pos, const int* slots, void* k_pages, void*
    v_pages, long num_pages, int nh, int nkv, int d, int ps, const float* sumsq, int n_partials, float eps,
    hipStream_t stream);

// measure.hip
int lmsf_measure_read(const void* src, long bytes, void* sink, hipStream_t stream);
int lmsf_measure_copy(const void* src, void* dst, long bytes, hipStream_t stream);
double lmsf_measure_mfma(void* sink, int iters, int blocks, hipStream_t stream);

// norm.hip
int lmsf_add_rms_norm(const void* branch, int branch_dtype, float* residual, const void* weight, int weight_dtype,
    void* out, int out_dtype, const int* rows, int n_out, int H, float eps, float weight_offset, hipStream_t stream);
int lmsf_add_rms_norm_partial(const float* part, const void* bias, int n_split, int M, float* residual, const void*
    weight, int weight_dtype, void* out, int out_dtype, const int* rows, int n_out, int H, float eps, float
    weight_offset, hipStream_t stream);

// rope_cache.hip
int lmsf_rope_cache_write(void* q, void* k, void* v, int dtype, int n_tokens, long row_stride, const int* positions,
    const float* table, int rot, int neox, int max_pos, const int* slots, void* k_pages, void* v_pages, long
    num_pages, int nh, int nkv, int d, int ps, hipStream_t stream);
int lmsf_rope_cache_write_partial(const float* part, const void* bias, int n_split, void* y, long ldy, int n_tokens,
    const int* positions, const float* table, int rot, int neox, int max_pos, const int* slots, void* k_pages, void*
    v_pages, long num_pages, int nh, int nkv, int d, int ps, hipStream_t stream);

// runtime.hip
const char* lmsf_last_error();
int lmsf_abi_version();
int lmsf_device_arch(char* out, int cap);

// sampling.hip
long lmsf_sample_scratch_elems(int R, int V);
int lmsf_sample(const float* logits, long ld, int R, int V, const float* temperature, const int* top_k, const float*
    top_p, const float* min_p, const unsigned long long* seeds, const unsigned int* draws, int* out, void* scratch,
    hipStream_t stream);
int lmsf_apply_penalties(float* logits, long ld, int R, int V, const int* tokens, const int* offsets, const int*
    prompt_lens, int* counts, const float* presence, const float* frequency, const float* repetition, hipStream_t
    stream);

#ifdef __cplusplus
}
#endif
