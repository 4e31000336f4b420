// Every launcher of the kernel library that takes a stream, declared in one place: the files that
// define them include this header, so that a declaration that has drifted from its definition does
// not compile, and launch_plan.hip builds its table of launchers from it.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {
// attention_decode.hip
int mgpt_paged_attention_split_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool, const
    void* vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const int*
    q_req, int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    hipStream_t stream);
// attention_decode.hip
int mgpt_paged_attention_split_fast_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool,
    const void* vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const
    int* q_req, int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window,
    hipStream_t stream);
// attention_decode_wide.hip
int mgpt_paged_attention_decode_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool, const
    void* vpool, const int* block_tables, int max_blocks, const int* positions, const int* q_req, const int*
    cu_q, int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, int num_pages, float scale,
    int window, int identity, hipStream_t stream);
// attention_generic.hip
int mgpt_kv_write(const void* qkv, int dtype, long ld, int k_off, int v_off, void* kpool, void* vpool, const
    int* slot_mapping, int n_tokens, int n_kv_head, int head_dim, int page_size, hipStream_t stream);
// attention_generic.hip
int mgpt_paged_attention_generic(const void* q, long ldq, void* out, long ldo, const void* kpool, const void*
    vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, const int* q_req,
    int n_tokens, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window, int dtype,
    int fast_exp, hipStream_t stream);
// attention_prefill.hip
int mgpt_prefill_attention_bf16(const void* q, long ldq, void* out, long ldo, const void* kpool, const void*
    vpool, const int* block_tables, int max_blocks, const int* cu_q, const int* seq_lens, int n_req, int
    max_q_len, int n_head, int n_kv_head, int head_dim, int page_size, float scale, int window, int
    single_below, hipStream_t stream);
// embed_norm.hip
int mgpt_embed(const int* ids, const int* pos, const void* tok, const void* postab, float* x, int n_tokens,
    int width, int table_dtype, hipStream_t stream);
// embed_norm.hip
int mgpt_layernorm(const float* x, const float* w, const float* b, void* out, const int* rows, int n_rows, int
    width, float eps, int out_dtype, hipStream_t stream);
// fold_norm.hip
int mgpt_fold_layernorm(const void* w, const float* gain, const float* beta, const float* bias, void* w_out,
    float* colsum, float* bias_out, int n_out, int k_dim, hipStream_t stream);
// fold_norm.hip
int mgpt_pack_weight(const void* w, void* packed, int n_out, int k_dim, hipStream_t stream);
// fused_decode.hip
int mgpt_fused_attention_decode(const float* base, const float* partials, int n_parts, long part_stride, const
    void* tok_table, const void* pos_table, const int* ids, const int* token_positions, float* settled, const
    void* normed, const float* gain, const float* beta, float eps, const void* wqkv_packed, const float* bqkv,
    const void* wproj_packed, const float* bproj, float* out_partials, long out_part_stride, void* kpool, void* vpool,
    const int* slot_mapping, const int* block_tables, int max_blocks, const int* positions, const int* q_req,
    int n_rows, int width, int n_head, int head_dim, int page_size, int num_pages, float scale, hipStream_t
    stream);
// fused_decode.hip
int mgpt_fused_mlp_decode(const float* base, const float* partials, int n_parts, long part_stride, const void*
    tok_table, const void* pos_table, const int* ids, const int* token_positions, float* settled, const float*
    gain, const float* beta, float eps, const void* wfc_packed, const float* bfc, const void* wproj_packed,
    const float* bproj, float* out_partials, long out_part_stride, int n_rows, int width, int hidden,
    hipStream_t stream);
// fused_decode.hip
int mgpt_residual_layernorm(const float* base, const float* partials, int n_parts, long part_stride, const
    void* tok_table, const void* pos_table, const int* ids, const int* token_positions, const float* gain,
    const float* beta, float eps, const int* rows, void* out, int out_dtype, int n_rows, int width, float*
    settled, hipStream_t stream);
// fused_decode.hip
int mgpt_residual_settle(const float* base, const float* partials, int n_parts, long part_stride, const void*
    tok_table, const void* pos_table, const int* ids, const int* token_positions, float* settled, int n_rows,
    int width, hipStream_t stream);
// linear_generic.hip
int mgpt_linear_generic(const void* A, int a_dtype, long lda, const void* W, int w_dtype, const float* bias,
    void* out, int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue, hipStream_t stream);
// linear_mfma.hip
int mgpt_linear_mfma_parts(const void* act, long lda, const void* w, const float* bias, float* partials,
                           long partials_floats, int n_rows, int n_out, int k_dim, hipStream_t stream);
int mgpt_linear_mfma(const void* act, long lda, const void* w, const float* bias, void* out, int out_dtype,
    long ldo, int n_rows, int n_out, int k_dim, int epilogue, float* partials, long partials_floats,
    hipStream_t stream);
// linear_mfma.hip
int mgpt_linear_mfma_shape(int shape, int k_parts, const void* act, long lda, const void* w, const float*
    bias, void* out, int out_dtype, long ldo, int n_rows, int n_out, int k_dim, int epilogue, float* partials,
    long partials_floats, hipStream_t stream);
// linear_mfma.hip
int mgpt_linear_mfma_qkv(const void* act, long lda, const void* w, const float* bias, void* out, long ldo, int
    n_rows, int n_out, int k_dim, void* kpool, void* vpool, const int* slot_mapping, int q_width, int
    kv_width, int head_dim, int n_kv_head, int page_size, int shape, hipStream_t stream);
// linear_skinny.hip
int mgpt_linear_skinny(const void* act, long lda, const float* x, const int* rows, const float* colsum, float
    eps, const void* w, const void* w_packed, const float* bias, void* out, int out_dtype, long ldo, int
    n_rows, int n_out, int k_dim, int epilogue, void* kpool, void* vpool, const int* slot_mapping, int
    q_width, int kv_width, int head_dim, int n_kv_head, int page_size, int mode, float* partials, long
    partials_floats, hipStream_t stream);
// linear_skinny.hip
int mgpt_linear_head_best(const void* act, long lda, const float* x, const int* rows, const float* colsum,
    float eps, const void* w, const void* w_packed, const float* bias, float* out, long ldo, int n_rows, int
    n_out, int k_dim, float* best_val, int* best_idx, int best_limit, hipStream_t stream);
// linear_decode_rows.hip
int mgpt_linear_decode_parts(const void* act, long lda, const void* w, const void* w_packed, const float* bias,
    float* partials, int n_rows, int n_out, int k_dim, hipStream_t stream);
// sampling.hip
int mgpt_sample(const float* logits, long ld, int n_rows, int vocab, int real_vocab, const float* temperature,
    const int* top_k, const float* top_p, const uint64_t* request_seed, const int* out_index, uint64_t
    engine_seed, int* out_tokens, const float* tile_best, const int* tile_best_idx, int n_tiles, hipStream_t
    stream);
// sampling.hip
int mgpt_sample_advance(const float* logits, long ld, int n_rows, int vocab, int real_vocab, const float*
    temperature, const int* top_k, const float* top_p, const uint64_t* request_seed, int* out_index, uint64_t
    engine_seed, int* out_tokens, int* token_ids, int* positions, int* seq_lens, const int* q_req, int*
    slot_mapping, const int* block_tables, const int* page_sizes, int n_groups, int n_stride, int r_stride,
    int max_blocks, int* history, int* history_pos, int history_rows, int history_stride, const float*
    tile_best, const int* tile_best_idx, int n_tiles, hipStream_t stream);
}

// MGPT_FOR_EACH_LAUNCHER(X) expands X(name) for every launcher above
#define MGPT_FOR_EACH_LAUNCHER(X) \
  X(mgpt_paged_attention_split_bf16) \
  X(mgpt_paged_attention_split_fast_bf16) \
  X(mgpt_paged_attention_decode_bf16) \
  X(mgpt_kv_write) \
  X(mgpt_paged_attention_generic) \
  X(mgpt_prefill_attention_bf16) \
  X(mgpt_embed) \
  X(mgpt_layernorm) \
  X(mgpt_fold_layernorm) \
  X(mgpt_pack_weight) \
  X(mgpt_fused_attention_decode) \
  X(mgpt_fused_mlp_decode) \
  X(mgpt_residual_layernorm) \
  X(mgpt_residual_settle) \
  X(mgpt_linear_generic) \
  X(mgpt_linear_mfma) \
  X(mgpt_linear_mfma_parts) \
  X(mgpt_linear_mfma_shape) \
  X(mgpt_linear_mfma_qkv) \
  X(mgpt_linear_skinny) \
  X(mgpt_linear_head_best) \
  X(mgpt_linear_decode_parts) \
  X(mgpt_sample) \
  X(mgpt_sample_advance)
