// The entry points of the kernel library that launch work on a stream: one declaration each, seen by the
// file that defines it (so the two cannot drift apart) and by the step tape (tape.hip), which calls them
// by name with recorded arguments.  Every one returns 0, or non-zero with a message for zi_last_error().
// Pointers are device memory unless a comment at the definition says otherwise.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {

// attention_decode.hip
int zi_attention_decode(void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo, const void* kcache,
    const void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, int
    max_chunks, float* workspace, int64_t workspace_floats, hipStream_t stream);
// attention_decode.hip
int zi_attention_decode_fused(void* out, int dt, int n_idx, int64_t ldo, const float* sums, int splits, int64_t
    split_stride, int64_t ldp, const void* bias, int bias_dt, const float* table, int rot, const int32_t* slots,
    int64_t cache_slots, int write_kv, void* kcache, void* vcache, const int32_t* tok_index, const int32_t* tok_seq,
    const int32_t* tok_pos, const int32_t* block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int
    page_size, int window, float scale, int max_chunks, float* workspace, int64_t workspace_floats, hipStream_t
    stream);
// attention_decode.hip
int zi_attention_decode_project(float* sums, const float* workspace, int64_t workspace_floats, int n, const int32_t*
    tok_pos, int window, int max_chunks, const void* w, int dt, int64_t ldw, int N, int nh, int d, hipStream_t
    stream);
// attention_generic.hip
int zi_attention_generic(void* out, const void* q, int dt, int n, int64_t ldq, int64_t ldo, const void* kcache, const
    void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale,
    hipStream_t stream);
// attention_prefill.hip
int zi_attention_prefill(void* out, const void* q, int dt, int num_tiles, int64_t ldq, int64_t ldo, const void*
    kcache, const void* vcache, const int32_t* tile_entry, const int32_t* tile_off, const int32_t* entry_start, const
    int32_t* entry_len, const int32_t* entry_past, const int32_t* block_tables, int max_pages, int num_pages, int nh,
    int nkv, int d, int page_size, int window, float scale, int rows, int max_chunks, float* workspace, int64_t
    workspace_floats, int tile, int alone, int chunk_keys, hipStream_t stream);
// decode_layer.hip
int zi_decode_layer(float* resid, int n, int H, int I, const void* norm1, const void* norm2, int norm_dt, float eps1,
    float eps2, int add_one, const void* wqkv, int64_t ld_qkv, const void* bias, int bias_dt, const void* wo, int64_t
    ld_o, const void* wgu, int64_t ld_gu, const void* wd, int64_t ld_d, int dt, const float* table, int rot, const
    int32_t* slots, int64_t cache_slots, void* kcache, void* vcache, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, int
    max_keys, void* workspace, int64_t workspace_bytes, uint32_t* sync, int* err, int spin_limit, hipStream_t stream);
// elementwise.hip
int zi_embedding(void* out, int out_dt, const void* table, int table_dt, const int32_t* ids, int n, int hidden, int
    vocab, hipStream_t stream);
// elementwise.hip
int zi_gather_rows(void* out, const void* in, int dt, const int32_t* idx, int n_out, int n_in, int hidden, hipStream_t
    stream);
// elementwise.hip
int zi_add(void* c, int c_dt, const void* a, int a_dt, const void* b, int b_dt, int64_t n, hipStream_t stream);
// elementwise.hip
int zi_swiglu_t(void* out, const void* gut, int dt, int n, int inter, int64_t ldt, hipStream_t stream);
// elementwise.hip
int zi_swiglu(void* out, int out_dt, const void* gate, const void* up, int dt, int n, int inter, int64_t ld_gate,
    int64_t ld_up, int interleave, int splits, int64_t split_stride, hipStream_t stream);
// gemm_generic.hip
int zi_gemm_generic(void* out, int out_dt, const void* x, int x_dt, const void* w, int w_dt, const void* bias, int
    bias_dt, int M, int N, int K, int64_t ldx, int64_t ldw, int64_t ldo, hipStream_t stream);
// gemm_lt.hip
int zi_gemm_lt(void* out, int out_dt, const void* x, const void* weight, const void* bias, int transposed, int64_t M,
    int64_t N, int64_t K, int64_t ldx, int64_t ldw, int64_t ldo, void* workspace, int64_t workspace_bytes, hipStream_t
    stream);
// gemm_skinny.hip
int zi_gemm_skinny(void* out, int out_dt, int mode, const void* x, const void* w, const void* bias, int M, int N, int
    K, int64_t ldx, int64_t ldw, int64_t ldo, float* workspace, int64_t workspace_floats, hipStream_t stream);
// gemm_skinny.hip
int zi_reduce_splits(void* out, int out_dt, const float* sums, const void* bias, int M, int N, int64_t ldo, int
    splits, hipStream_t stream);
// norm.hip
int zi_rmsnorm(void* out, int out_dt, const void* x, int x_dt, const void* w, int w_dt, int n, int hidden, int64_t
    ldx, int64_t ldo, float eps, int add_one, hipStream_t stream);
// norm.hip
int zi_add_rmsnorm(void* out, int out_dt, float* resid, const void* delta, int delta_dt, int splits, int64_t
    split_stride, const void* w, int w_dt, int n, int hidden, float eps, int add_one, hipStream_t stream);
// rope_kv.hip
int zi_rope_kv_store(void* q, const void* k, const void* v, int dt, int n, int64_t ldq, int64_t ldk, int64_t ldv,
    const int32_t* slots, const float* table, void* kcache, void* vcache, int64_t cache_slots, int nh, int nkv, int d,
    int rot, int page_size, int write_kv, hipStream_t stream);
// rope_kv.hip
int zi_rope_kv_store_split(void* q_out, int dt, int64_t ldq, const float* part, int splits, int64_t split_stride,
    int64_t ldp, const void* bias, int bias_dt, int n, const int32_t* slots, const float* table, void* kcache, void*
    vcache, int64_t cache_slots, int nh, int nkv, int d, int rot, int page_size, int write_kv, hipStream_t stream);
// rope_kv.hip
int zi_rope(void* out, const void* in, int dt, int n, int64_t ld_in, int64_t ld_out, const int32_t* pos, const float*
    inv_freq, int nh, int d, int rot, hipStream_t stream);
// rope_kv.hip
int zi_rope_table(float* out, const int32_t* pos, const float* inv_freq, int n, int half, hipStream_t stream);
// elementwise.hip
int zi_gated_act(void* out, int out_dt, int64_t ldo, const void* gate, const void* up, int dt, int64_t ld_gate, int64_t
    ld_up, int n, int inter, int act, hipStream_t stream);
// latent.hip
int zi_rope_pairs(void* x, int dt, int64_t ld, const float* table, int n, int heads, int d, int rot, hipStream_t
    stream);
// latent.hip
int zi_latent_store(const float* dkv, int dt, int64_t ld, int n, const void* norm_w, int w_dt, float eps, const float*
    table, const int32_t* slots, void* c_cache, void* kr_cache, int64_t cache_slots, int rank, int rot, hipStream_t
    stream);
// latent.hip
int zi_latent_query(float* qa, const void* q, int dt, int64_t ldq, const void* w_uk, int w_dt, const float* table, int
    n, int heads, int dim, int rank, int rot, hipStream_t stream);
// latent.hip
int zi_latent_attention(float* out, const float* qa, const void* c_cache, const void* kr_cache, int dt, int n_idx, const
    int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* block_tables, int max_pages, int
    num_pages, int heads, int rank, int rot, int page_size, int window, float scale, hipStream_t stream);
// latent_cores.hip
int zi_latent_attention_cores(float* out, float* partial, int64_t partial_floats, const float* qa, const void* c_cache,
    const void* kr_cache, const int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_past, const int32_t*
    block_tables, int entries, int n, int max_pages, int num_pages, int heads, int rank, int rot, int page_size, int
    window, float scale, int waves, int chunk_keys, int chunks, hipStream_t stream);
// latent_cores.hip
int zi_headwise_linear(void* out, int out_dt, int64_t ldo, int os, const float* x, int64_t ldx, int xs, const void* w, int
    n, int heads, int N, int K, hipStream_t stream);
// latent_cores.hip
int zi_latent_query_rot(float* qa, const void* q, int dt, int64_t ldq, const float* table, int n, int heads, int dim, int
    rank, int rot, hipStream_t stream);
// latent.hip
int zi_latent_value(void* out, int out_dt, int64_t ldo, const float* o, const void* w_uv, int w_dt, int n, int heads,
    int vdim, int rank, hipStream_t stream);
// delta.hip
int zi_delta_prepare(float* qk, float* v, float* beta_g, const float* proj, int64_t ld, int n, const void* conv_w, const
    void* a_log, const void* dt_bias, int w_dt, const float* state, int64_t state_stride, int64_t conv_off, const
    int32_t* tok_seq, const int32_t* entry_start, const int32_t* entry_slot, int heads, int kvh, int dim, int vdim, int
    taps, hipStream_t stream);
// delta.hip
int zi_delta_conv_state(float* state, int64_t state_stride, int64_t conv_off, const float* proj, int64_t ld, const
    int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_slot, int entries, int channels, int taps,
    hipStream_t stream);
// delta.hip
int zi_delta_rule(float* out, const float* qk, const float* v, const float* beta_g, float* state, int64_t
    state_stride, const int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_slot, int entries, int
    heads, int kvh, int dim, int vdim, hipStream_t stream);
// delta.hip
int zi_gated_rmsnorm(void* out, int out_dt, const float* o, const void* w, int w_dt, const float* gate, int64_t
    ld_gate, int n, int heads, int vdim, float eps, hipStream_t stream);
// moe.hip
int zi_moe_route(int32_t* idx, float* wt, const float* z, const float* correction, int n, int experts, int top, float
    scale, hipStream_t stream);
// moe.hip
int zi_moe_group(int32_t* plan, int32_t* order, int32_t* place_of, const int32_t* idx, int pairs, int experts, int
    tile_rows, hipStream_t stream);
// moe.hip
int zi_moe_linear(void* out, int out_dt, int64_t ldo, const void* x, int x_dt, int64_t ldx, const void* w, int w_dt,
    const int32_t* plan, const int32_t* source, int source_div, int max_tiles, int tile_rows, int N, int K, int act,
    hipStream_t stream);
// moe.hip
int zi_moe_combine(float* out, const float* y, const float* wt, const int32_t* place_of, int n, int top, int hidden,
    hipStream_t stream);
// attention_generic.hip
int zi_attention_generic_sink(void* out, const void* q, int dt, int n, int64_t ldq, int64_t ldo, const void* kcache,
    const void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, const
    float* sinks, hipStream_t stream);
// attention_decode.hip
int zi_attention_decode_sink(void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo, const void* kcache,
    const void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, int
    max_chunks, float* workspace, int64_t workspace_floats, const float* sinks, hipStream_t stream);
// attention_prefill.hip
int zi_attention_prefill_sink(void* out, const void* q, int dt, int num_tiles, int64_t ldq, int64_t ldo, const void*
    kcache, const void* vcache, const int32_t* tile_entry, const int32_t* tile_off, const int32_t* entry_start, const
    int32_t* entry_len, const int32_t* entry_past, const int32_t* block_tables, int max_pages, int num_pages, int nh,
    int nkv, int d, int page_size, int window, float scale, int rows, int max_chunks, float* workspace, int64_t
    workspace_floats, int tile, int alone, int chunk_keys, const float* sinks, hipStream_t stream);
// attention_decode.hip
int zi_attention_decode_project_sink(float* sums, const float* workspace, int64_t workspace_floats, int n, const int32_t*
    tok_pos, int window, int max_chunks, const void* w, int dt, int64_t ldw, int N, int nh, int d, const float* sinks,
    hipStream_t stream);
// layer_norm.hip
int zi_layer_norm(void* out, int out_dt, int64_t ldo, float* resid, const void* x, int x_dt, int splits, int64_t
    split_stride, int64_t ldx, const void* w, const void* b, int w_dt, int n, int hidden, float eps, hipStream_t
    stream);
// conv_qkv.hip
int zi_conv_qkv(void* q_out, int dt, int64_t ldq, void* kcache, void* vcache, const void* proj, int proj_dt, int64_t ld,
    int splits, int64_t split_stride, const float* bias, const float* conv_w, float* state, int64_t state_stride, int
    move_tail, const float* q_norm, const float* k_norm, float eps, const float* table, int rot, int n, const int32_t* tok_seq, const int32_t* entry_start, const
    int32_t* entry_slot, const int32_t* slots, int64_t cache_slots, int nh, int nkv, int dim, int vdim, int D, int taps,
    int page_size, hipStream_t stream);
// conv_qkv.hip
int zi_conv_tail(float* state, int64_t state_stride, const void* proj, int proj_dt, int64_t ld, int splits, int64_t
    split_stride, const float* bias, const
    int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_slot, const int32_t* slots, int entries, int
    channels, int taps, hipStream_t stream);
// elementwise.hip
int zi_relu_squared(void* out, int out_dt, int64_t ldo, const void* z, int dt, int64_t ldz, int splits, int64_t
    split_stride, int n, int inter, hipStream_t stream);
// elementwise.hip
int zi_clamped_glu(void* out, int out_dt, int64_t ldo, const void* gate, const void* up, int dt, int64_t ld_gate, int64_t
    ld_up, int splits, int64_t split_stride, int n, int inter, float limit, float alpha, hipStream_t stream);
// elementwise.hip
int zi_softcap(float* x, int64_t total, float cap, hipStream_t stream);
// elementwise.hip
int zi_convert(void* out, int out_dt, const void* x, int dt, int64_t total, hipStream_t stream);
// moe.hip
int zi_moe_route_top(int32_t* idx, float* wt, const float* z, const float* bias, int n, int experts, int top,
    hipStream_t stream);
// sampling.hip
int zi_argmax(int32_t* out_idx, float* out_val, const void* logits, int dt, int rows, int vocab, int64_t ld, float*
    workspace, int64_t workspace_floats, hipStream_t stream);
// stream.hip
int zi_embedding_sum(float* out, const void* table, int table_dt, const void* pair, int pair_dt, const int32_t* ids,
    const int32_t* pos, const int32_t* tok_seq, const int32_t* entry_start, const int32_t* entry_len, const int32_t*
    entry_slot, int32_t* state, int64_t state_stride, const double* freq, int n, int hidden, int vocab, int buckets,
    int64_t mul_prev, int64_t mul_cur, hipStream_t stream);
// stream.hip
int zi_token_shift(void* out, int out_dt, int64_t ldo, const void* x, int x_dt, int64_t ldx, const void* w, int w_dt,
    float* state, int64_t state_stride, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* entry_start,
    const int32_t* entry_len, const int32_t* entry_slot, int n, int hidden, hipStream_t stream);
// stream.hip
int zi_stream_reenter(float* resid, const void* delta, int delta_dt, int splits, int64_t split_stride, const float*
    again, const void* row, int row_dt, int n, int hidden, hipStream_t stream);
// linear_attention.hip
int zi_lowrank_decay(float* out, int64_t ldo, const float* u, int64_t ldu, const void* w2, const void* bias, int w_dt,
    int n, int channels, int rank, float tau, hipStream_t stream);
// linear_attention.hip
int zi_linear_attention(float* out, int64_t ldo, const float* q, const float* k, const float* v, int64_t ld, const
    float* decay, int64_t ld_decay, const float* head_decay, float* state, int64_t state_stride, const int32_t*
    entry_start, const int32_t* entry_len, const int32_t* entry_past, const int32_t* entry_slot, int entries, int
    heads, int dim, int vdim, int act, float qscale, hipStream_t stream);
// linear_attention.hip
int zi_gate_heads(void* out, int out_dt, int64_t ldo, const void* x, int x_dt, int64_t ldx, int x_head, const float*
    gate, int64_t ld_gate, int n, int width, int head, int act, float scale, hipStream_t stream);
// delta.hip
int zi_gated_rmsnorm_act(void* out, int out_dt, int64_t ldo, const float* o, const void* w, int w_dt, const float*
    gate, int64_t ld_gate, int n, int heads, int vdim, float eps, int act, float scale, hipStream_t stream);
// attention_biased.hip
int zi_normed_kv_store(void* q_out, int dt, int64_t ldq, void* kcache, void* vcache, const float* proj, int64_t ld,
    int q_at, int k_at, int v_at, const int32_t* slots, int64_t cache_slots, int n, int nh, int nkv, int dim, int vdim,
    int d, int page_size, float eps, int norm_values, hipStream_t stream);
// attention_generic.hip
int zi_attention_generic_biased(void* out, const void* q, int dt, int n, int64_t ldq, int64_t ldo, const void* kcache,
    const void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, const
    float* sinks, float softcap, const float* bias, int bias_len, int keep_first, hipStream_t stream);
// attention_prefill.hip
int zi_attention_prefill_biased(void* out, const void* q, int dt, int num_tiles, int64_t ldq, int64_t ldo, const void*
    kcache, const void* vcache, const int32_t* tile_entry, const int32_t* tile_off, const int32_t* entry_start, const
    int32_t* entry_len, const int32_t* entry_past, const int32_t* block_tables, int max_pages, int num_pages, int nh,
    int nkv, int d, int page_size, int window, float scale, int rows, int max_chunks, float* workspace, int64_t
    workspace_floats, int tile, int alone, int chunk_keys, const float* sinks, float softcap, const float* bias, int
    bias_len, int keep_first, hipStream_t stream);
// attention_decode.hip
int zi_attention_decode_biased(void* out, const void* q, int dt, int n_idx, int64_t ldq, int64_t ldo, const void* kcache,
    const void* vcache, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int nh, int nkv, int d, int page_size, int window, float scale, int
    max_chunks, float* workspace, int64_t workspace_floats, const float* sinks, float softcap, const float* bias, int
    bias_len, int keep_first, hipStream_t stream);
// moe.hip
int zi_moe_route_table(int32_t* idx, float* wt, const int32_t* ids, const int32_t* table, int n, int vocab, int
    experts, int top, hipStream_t stream);
// rope_kv.hip
int zi_rope_table_scaled(float* out, const int32_t* pos, const float* inv_freq, int n, int half, float magnitude,
    hipStream_t stream);
// linear_attention.hip
int zi_linear_attention_grouped(float* out, int64_t ldo, const float* q, const float* k, const float* v, int64_t ld,
    const float* decay, int64_t ld_decay, const float* head_decay, float* state, int64_t state_stride, const int32_t*
    entry_start, const int32_t* entry_len, const int32_t* entry_past, const int32_t* entry_slot, int entries, int
    heads, int dim, int vdim, int act, float qscale, int share, int decay_heads, int single_tokens, hipStream_t stream);
// ssm.hip
int zi_ssm_prepare(float* out, int64_t ldo, const float* proj, int64_t ld, int n, const float* conv_w, const float*
    conv_b, const float* dt_bias, const float* a_log, const float* state, int64_t state_stride, const int32_t*
    tok_seq, const int32_t* entry_start, const int32_t* entry_slot, int heads, int vdim, int gn2, int taps,
    hipStream_t stream);
// ssm.hip
int zi_ssm_finish(void* out, int out_dt, int64_t ldo, const float* y, int64_t ldy, const float* x, int64_t ldx, const
    float* z, int64_t ldz, const float* skip, const float* gain, int n, int heads, int vdim, int parts, float eps,
    hipStream_t stream);
// pooled_attention.hip
int zi_norm_rope_store(void* q_out, int dt, int64_t ldq, void* kcache, void* vcache, const float* proj, int64_t ld,
    int splits, int64_t split_stride, const float* q_gain, const float* k_gain, float eps, const float* table, int rot,
    const float* vtable, const int32_t* slots, int64_t cache_slots, int n, int nh, int nkv, int dim, int vdim,
    hipStream_t stream);
// pooled_attention.hip
int zi_pool_blocks(float* kpool, float* vpool, int64_t pool_rows, const void* kcache, const void* vcache, int dt, const
    int32_t* pool_slots, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t* block_tables, int max_pages,
    int num_pages, int page_size, int n, int nkv, int dim, int vdim, int pool, hipStream_t stream);
// pooled_attention.hip
int zi_pooled_attention(void* out, int64_t ldo, const void* q, int64_t ldq, int dt, const void* kcache, const void*
    vcache, const float* kpool, const float* vpool, const int32_t* tok_seq, const int32_t* tok_pos, const int32_t*
    block_tables, int max_pages, int num_pages, int page_size, const int32_t* pool_tables, int pool_max_pages, int
    pool_num_pages, int pool_page_size, int n, int nh, int nkv, int dim, int vdim, int window, int pool, float scale,
    const float* vtable, const int32_t* entry_len, int long_len, hipStream_t stream);
// pooled_attention_cores.hip
int zi_pooled_attention_cores(void* out, int64_t ldo, const void* q, int64_t ldq, const void* kcache, const void*
    vcache, const float* kpool, const float* vpool, const int32_t* entry_start, const int32_t* entry_len, const
    int32_t* entry_past, int entries, int max_len, const int32_t* block_tables, int max_pages, int num_pages, int
    page_size, const int32_t* pool_tables, int pool_max_pages, int pool_num_pages, int pool_page_size, int nh, int nkv,
    int dim, int vdim, int window, int pool, float scale, const float* vtable, int long_len, int chunks, int
    chunk_blocks, float* partial, int64_t partial_floats, const int32_t* tok_seq, int n, hipStream_t stream);
// norm.hip
int zi_normed_add_norm(void* out, int out_dt, float* resid, const void* y, int y_dt, int64_t ldy, int splits, int64_t
    split_stride, const void* w1, const void* w2, int w_dt, int n, int hidden, float eps, float eps2, int add_one,
    hipStream_t stream);
// moe.hip
int zi_moe_route_sigmoid(int32_t* idx, float* wt, const float* z, int64_t ld, int n, int experts, int top,
    hipStream_t stream);
// moe.hip
int zi_moe_weighted_glu(void* out, int out_dt, int64_t ldo, const float* gu, int64_t ld, const float* wt, const
    int32_t* order, int pairs, int ff, hipStream_t stream);
// moe.hip
int zi_moe_sum_shared(float* out, const float* y, const int32_t* place_of, const float* shared, int splits, int64_t
    split_stride, const float* gate, int64_t ld_gate, int n, int top, int hidden, hipStream_t stream);
// sampling.hip
int zi_sample(int32_t* out, const float* logits, int64_t ld, float* work, int rows, int vocab, const float*
    temperature, const int32_t* top_k, const float* top_p, const float* penalty, const float* uniform, const int32_t*
    recent, const int32_t* recent_len, int max_recent, hipStream_t stream);
}

// Every entry point above, for code that wants them all (X is applied to each name).
#define ZI_STREAM_ENTRY_POINTS(X) \
    X(zi_attention_decode) \
    X(zi_attention_decode_fused) \
    X(zi_attention_decode_project) \
    X(zi_attention_generic) \
    X(zi_attention_prefill) \
    X(zi_decode_layer) \
    X(zi_embedding) \
    X(zi_gather_rows) \
    X(zi_add) \
    X(zi_swiglu_t) \
    X(zi_swiglu) \
    X(zi_gemm_generic) \
    X(zi_gemm_lt) \
    X(zi_gemm_skinny) \
    X(zi_reduce_splits) \
    X(zi_rmsnorm) \
    X(zi_add_rmsnorm) \
    X(zi_rope_kv_store) \
    X(zi_rope_kv_store_split) \
    X(zi_rope) \
    X(zi_rope_table) \
    X(zi_gated_act) \
    X(zi_rope_pairs) \
    X(zi_latent_store) \
    X(zi_latent_query) \
    X(zi_latent_attention) \
    X(zi_latent_attention_cores) \
    X(zi_headwise_linear) \
    X(zi_latent_query_rot) \
    X(zi_latent_value) \
    X(zi_delta_prepare) \
    X(zi_delta_conv_state) \
    X(zi_delta_rule) \
    X(zi_gated_rmsnorm) \
    X(zi_moe_route) \
    X(zi_moe_group) \
    X(zi_moe_linear) \
    X(zi_moe_combine) \
    X(zi_attention_generic_sink) \
    X(zi_attention_decode_sink) \
    X(zi_attention_prefill_sink) \
    X(zi_attention_decode_project_sink) \
    X(zi_layer_norm) \
    X(zi_conv_qkv) \
    X(zi_conv_tail) \
    X(zi_relu_squared) \
    X(zi_clamped_glu) \
    X(zi_softcap) \
    X(zi_convert) \
    X(zi_moe_route_top) \
    X(zi_embedding_sum) \
    X(zi_token_shift) \
    X(zi_stream_reenter) \
    X(zi_lowrank_decay) \
    X(zi_linear_attention) \
    X(zi_gate_heads) \
    X(zi_gated_rmsnorm_act) \
    X(zi_normed_kv_store) \
    X(zi_attention_generic_biased) \
    X(zi_attention_prefill_biased) \
    X(zi_attention_decode_biased) \
    X(zi_moe_route_table) \
    X(zi_rope_table_scaled) \
    X(zi_linear_attention_grouped) \
    X(zi_ssm_prepare) \
    X(zi_ssm_finish) \
    X(zi_norm_rope_store) \
    X(zi_pool_blocks) \
    X(zi_pooled_attention) \
    X(zi_pooled_attention_cores) \
    X(zi_normed_add_norm) \
    X(zi_moe_route_sigmoid) \
    X(zi_moe_weighted_glu) \
    X(zi_moe_sum_shared) \
    X(zi_argmax) \
    X(zi_sample)
