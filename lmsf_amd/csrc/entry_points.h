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
// (``variant`` of the prefill and ``order`` of the decode entry may have LMSF_ATTENTION_WEIGHTS_F32 of common.h added)
int lmsf_attention_tile_tokens(int nh, int nkv);
int lmsf_paged_attention_prefill_mfma(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
    const void* v_pages, long num_pages, const int* block_tables, int btw, const int* tiles, int n_tiles, const int*
    seg, const int* pos, int nh, int nkv, int d, int ps, float scale, int window, int variant, hipStream_t stream);
long lmsf_attention_decode_scratch_floats(int n, int nh, int d, int n_splits);
int lmsf_paged_attention_decode_mfma(const void* q, long q_stride, void* out, long out_stride, const void* k_pages,
    const void* v_pages, long num_pages, const int* block_tables, int btw, const int* tok_idx, int n, const int* seg,
    const int* pos, int nh, int nkv, int d, int ps, float scale, int window, int chunk, int n_splits, float* scratch,
    int order, hipStream_t stream);

// group_norm.hip
int lmsf_group_norm(const void* branch, int branch_dtype, long branch_stride, const float* wb, float* residual,
    float* hist, long hist_stride, int hist_index, const float* mix, const float* wn, void* out, int out_dtype,
    long out_stride, const int* rows, int n_rows, int W, int groups, float eps_b, float eps_n, hipStream_t stream);

// latent.hip
int lmsf_latent_cache_write(const void* x, int dtype, long x_stride, const float* w, float eps, const int* positions,
    const float* table, int rot, int max_pos, const int* slots, void* k_pages, void* v_pages, long num_pages,
    int n_tokens, int R, int dr, int D, int ps, const void* qx, const float* qw, void* q_out, long q_out_stride,
    int Q, hipStream_t stream);
int lmsf_head_linear(const void* x, int dtype, long x_stride, int x_head, const void* W, void* y, long y_stride,
    int y_head, const void* gate, long gate_stride, int n_tokens, int H, int O, int K, const int* positions,
    const float* table, int rot, int max_pos, int x_at, int y_at, int dr, int gate_wide, hipStream_t stream);
int lmsf_rope_tail(const void* x, int dtype, long x_stride, int x_head, int x_at, void* y, long y_stride, int y_head,
    int y_at, const int* positions, const float* table, int rot, int max_pos, int n_tokens, int H, int dr,
    hipStream_t stream);

// moe.hip
int lmsf_table_moe(const void* h, int dtype, long h_stride, const void* Wgu, const void* Wd, const int* ids,
    const int* table, int vocab, int top, int E, float weight, const void* base, long base_stride,
    const float* pair_scale, const float* base_scale, void* act, void* out, long out_stride, int n_tokens, int F,
    int W, int* scratch_ints, float* scratch_rows, hipStream_t stream);
int lmsf_moe_route(const float* z, long z_stride, int n_tokens, int E, int top, int renorm, int extra, int* choice,
    float* weight, float* gate, hipStream_t stream);
long lmsf_table_moe_scratch_ints(int n_tokens, int top, int E);
int lmsf_table_moe_grouped(int dtype, int n_tokens, int top, int E, int F, int W, long h_stride);

// attn_prepare.hip
int lmsf_attn_prepare(const void* q, long q_stride, const void* k, long k_stride, const void* v, long v_stride, int
    dtype, const int* positions, const float* table, int rot, int max_pos, const int* slots, void* q_out, long
    qo_stride, void* k_pages, void* v_pages, long num_pages, int n_tokens, int H, int G, int dim, int vdim, int D, int
    ps, int unit_norm, float eps, float temp_coef, int temp_every, hipStream_t stream);
int lmsf_head_gate(const void* x, int dtype, long x_stride, int x_head, const void* gate, long gate_stride, void* out,
    long out_stride, int n_tokens, int H, int dv, hipStream_t stream);
int lmsf_rms_pair(const void* a, long a_stride, const void* b, long b_stride, int dtype, const float* wa, const float*
    wb, void* out, int n_rows, int W, float eps, float scale, hipStream_t stream);

// dyt_norm.hip
int lmsf_dyt_norm(const void* branch, int branch_dtype, float* residual, const float* w, const float* b, const float*
    alpha, void* out, int out_dtype, const int* rows, int n_rows, int H, hipStream_t stream);

// recurrent.hip
int lmsf_short_conv(const void* u, int dtype, long u_stride, const void* w, const void* bias, int act, float* state,
    long state_stride, const int* seg_of, const int* seg_starts, const int* state_slots, void* out, long out_stride,
    int n_tokens, int n_segments, int C, int taps, int single, hipStream_t stream);
long lmsf_selective_scan_entry_floats(int inner, int nstate);
int lmsf_selective_scan(const void* x, int dtype, long x_stride, const float* dt_pre, long dt_stride, const void* bc,
    long bc_stride, int b_at, int c_at, const void* z, long z_stride, const float* A_log, const float* Dw, float*
    state, long state_stride, const int* seg_starts, const int* state_slots, void* y, long y_stride, int n_tokens, int
    n_segments, int inner, int nstate, int chunk, int max_chunks, const int* scratch_base, float* scratch,
    hipStream_t stream);
long lmsf_mlstm_state_floats(int H, int d, int dv);
long lmsf_mlstm_chunk_scratch_floats(int n_tokens, int H, int dv);
int lmsf_mlstm_chunk_tokens(int d);
long lmsf_mlstm_chunk_entry_floats(int H, int d, int dv);
int lmsf_mlstm_chunked(const void* q, const void* k, const void* v, int dtype, long qkv_stride, const float* gates,
    long gates_stride, const void* og, long og_stride, const float* norm_w, float* state, long state_stride, const
    int* seg_starts, const int* state_slots, void* out, long out_stride, float* o_raw, int n_tokens, int n_segments,
    int H, int d, int dv, float qscale, float cap, float eps, const int* chunk_base, int max_chunks, long n_entries,
    float* entries, hipStream_t stream);
int lmsf_mlstm_tokens(const void* q, const void* k, const void* v, int dtype, long qkv_stride, const float* gates,
    long gates_stride, const void* og, long og_stride, const float* norm_w, float* state, long state_stride, const
    int* seg_starts, const int* state_slots, void* out, long out_stride, float* o_raw, int n_tokens, int n_segments,
    int H, int d, int dv, float qscale, float cap, float eps, hipStream_t stream);

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

// retention.hip
long lmsf_retention_state_floats(int H, int d, int dv);
int lmsf_retention_chunk_tokens(int d);
long lmsf_retention_chunk_entry_floats(int H, int d, int dv);
int lmsf_retention_chunked(const void* q, const void* k, const void* v, int dtype, long qkv_stride,
    const int* positions, const float* table, int rot, int max_pos, const float* decay, const void* og,
    long og_stride, float* state, long state_stride, const int* seg_starts, const int* state_slots, void* out,
    long out_stride, float* o_raw, int n_tokens, int n_segments, int H, int d, int dv, float kscale, float eps,
    const int* chunk_base, int max_chunks, long n_entries, float* entries, hipStream_t stream);
int lmsf_retention_tokens(const void* q, const void* k, const void* v, int dtype, long qkv_stride,
    const int* positions, const float* table, int rot, int max_pos, const float* decay, const void* og,
    long og_stride, float* state, long state_stride, const int* seg_starts, const int* state_slots, void* out,
    long out_stride, float* o_raw, int n_tokens, int n_segments, int H, int d, int dv, float kscale, float eps,
    hipStream_t stream);

// layer_scale.hip
int lmsf_scale_add_norm(const void* a, long a_stride, const float* sa, const void* b, long b_stride, const float* sb,
    int dtype, float* stream, const void* wn, int wn_dtype, void* out, int n_rows, int W, float eps,
    hipStream_t stream_);
int lmsf_logit_cap(float* logits, long stride, int R, int V, float scale, float cap, hipStream_t stream);

#ifdef __cplusplus
}
#endif
