// The entry points of the HIP kernels (the .hip files beside this folder), as the host calls
// them: raw device pointers, sizes and a stream in, 0 or a hipError_t value out.  Shapes are
// checked by the callers in ops.cpp; a kernel never sees a size it was not written for.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstddef>
#include <cstdint>

#include "../gemv_params.h"
#include "../tile_params.h"
#include "../no_alloc.h"
#include "../norm_params.h"

extern "C" {
// elementwise.hip
int celeg_embed(const void* table, int table_dtype, const int* ids, float* out, int rows, int width, int vocab,
                float scale, hipStream_t stream);
int celeg_scale_f32(float* x, size_t total, float scale, hipStream_t stream);
int celeg_rmsnorm(void* x, int x_dtype, const void* delta, int delta_dtype, const float* w, void* out, int out_dtype,
                  const int* rows, int n_rows, int width, float eps, int write_back, hipStream_t stream);
int celeg_swiglu(const void* gu, void* out, int dtype, int rows, int ff, hipStream_t stream);
int celeg_add_bias(void* x, int dtype, const float* bias, int rows, int width, hipStream_t stream);
int celeg_cast(const void* src, int src_dtype, void* dst, int dst_dtype, size_t total, hipStream_t stream);
int celeg_table_update(int* table, int stride, int n_slots, const int* updates, int capacity, hipStream_t stream);
int celeg_step_prologue(int* table, int stride, int n_slots, const int* updates, int capacity, int* token_ids,
                        const int* token_slot, const int* last_tokens, int n, hipStream_t stream);
int celeg_resolve_tokens(int* token_ids, const int* token_slot, const int* last_tokens, int n, hipStream_t stream);
int celeg_fold_weight(const void* w, const float* scale, void* out, int rows, int K, int packed, hipStream_t stream);
int celeg_zero_words(void* p, size_t words, hipStream_t stream);
// hyper.hip
int celeg_streams_spread(const float* h, float* xs, int rows, int streams, int width, hipStream_t stream);
int celeg_streams_sum(const float* xs, float* h, int rows, int streams, int width, hipStream_t stream);
int celeg_hyper_step(float* xs, const void* y, int y_dtype, const float* mix, const float* out_w, const float* in_w,
                     const float* w, float eps, void* normed, int out_dtype, int rows, int streams, int width,
                     hipStream_t stream);
// latent.hip
int celeg_latent_prepare(void* proj, int ld, int dtype, int q_off, int dkv_off, int heads, int dim, int rot, int rank,
                         const float* weight, float eps, const float* inv_freq, int rotary, int pairing,
                         const int* positions, const int* token_slot, const int* table, int table_stride, void* pool,
                         int n_layers, int layer, int page_tokens, int write, int n_tokens, hipStream_t stream);
int celeg_headwise_linear(const void* x, int ldx, int x_head, const void* w, int dtype, int heads, int N, int K, void* out,
                          int ldo, int o_head, int tail, const void* gate, int ldg, int rows, int matrix_cores,
                          hipStream_t stream);
int celeg_latent_attention(const void* q, int ldq, const void* pool, int dtype, const int* table, int table_stride,
                           const int* token_slot, const int* positions, const float* sink, void* out, int ldo,
                           int n_tokens, int heads, int rank, int rot, int page_tokens, int n_layers, int layer,
                           float scale, hipStream_t stream);
// latent_fast.hip
int celeg_latent_attention_fast_ok(int rank, int rot);
int celeg_latent_attention_tile_rows(int rank, int rot);
int celeg_latent_attention_fast(int form, const void* q, int ldq, const void* pool, const int* table, int table_stride,
                                const int* cu_seqlens, const int* seq_slot, const int* seq_start, int n_seqs, int max_tiles,
                                const int* token_slot, const int* positions, int n_single, const float* sink, void* out,
                                int ldo, float* ws_o, float* ws_ml, int n_splits, int blocks_per_split, int heads, int rank,
                                int rot, int page_tokens, int n_layers, int layer, float scale, hipStream_t stream);
// moe.hip
int celeg_moe_route(const float* logits, int rows, int experts, int top, int score, int renorm, int groups, int keep,
                    float renorm_eps, float scale, int* ids, float* weights, hipStream_t stream);
int celeg_moe_router(const void* x, int x_dtype, const float* w, int rows, int width, int experts, int top, int score,
                     int renorm, int groups, int keep, float renorm_eps, float scale, int* ids, float* weights,
                     hipStream_t stream);
int celeg_moe_tile_rows(int matrix_cores);
int celeg_moe_plan(const int* ids, int n, int experts, int tile_rows, int* offsets, int* place_of, int* entry_at, int* tile_expert,
                   int* tile_row0, int* n_tiles, hipStream_t stream);
int celeg_moe_gather(const void* x, int dtype, const int* entry_at, const float* weights, void* a, int n, int top, int width,
                     hipStream_t stream);
int celeg_moe_product(const void* a, const void* w, void* out, int dtype, int N, int K, int gated, int act, const int* offsets,
                      const int* tile_expert, const int* tile_row0, const int* n_tiles, int max_tiles, int tile_rows, int wide,
                      hipStream_t stream);
int celeg_moe_combine(const void* y, int dtype, const int* place_of, const float* weights, const void* base, void* out, int rows,
                      int top, int width, hipStream_t stream);
// gemm_f32.hip
int celeg_gemm_f32(const float* X, int ldx, const float* W, int ldw, const float* bias, float* Y, int ldy, int M,
                   int N, int K, hipStream_t stream);
// short_conv.hip
int celeg_short_conv(const void* bcx, int ld_bcx, int dtype, const float* w, const float* bias, float* state,
                     size_t state_slot_stride, void* out, const int* positions, const int* token_seq,
                     const int* seq_start, const int* seq_slot, const int* cu_seqlens, int n_tokens, int n_seqs,
                     int width, int taps, hipStream_t stream);
// attention.hip
int celeg_rope_table(const float* inv_freq, int half, int n_positions, float* out, hipStream_t stream);
int celeg_qk_norm_rope_store(void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype,
                             const float* q_weight, const float* k_weight, float eps, const float* inv_freq,
                             const float* cos_sin, int rotary_dim, int pairing, const int* positions, const int* token_slot,
                             const int* table, int table_stride, void* k_pool, void* v_pool, int n_layers, int layer,
                             int page_tokens, int n_tokens, int q_heads, int kv_heads, int head_dim, int store_kv,
                             hipStream_t stream);
int celeg_paged_attention(const void* q, int ldq, const void* k_pool, const void* v_pool, int dtype, const int* table,
                          int table_stride, const int* token_slot, const int* positions, void* out, int ldo,
                          int n_tokens, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers,
                          int layer, float scale, int window, hipStream_t stream);
// attention_fast.hip
int celeg_attention_rows_bf16(const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
                              int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start,
                              int n_seqs, int n_tokens, void* out, int ldo, int q_heads, int kv_heads, int head_dim,
                              int page_tokens, int n_layers, int layer, float scale, int window, int rows_per_tile,
                              int form, int context_hint, hipStream_t stream);
int celeg_attention_decode_bf16(const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
                                int table_stride, const int* token_slot, const int* positions, float* ws_o,
                                float* ws_ml, int n_splits, void* out, int ldo, int n_rows, int q_heads,
                                int kv_heads, int head_dim, int page_tokens, int n_layers, int layer, float scale,
                                int window, int whole, int split_rounds, int n_parts, hipStream_t stream);
int celeg_attention_decode_fresh_bf16(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv,
                                      const float* q_weight, const float* k_weight, float eps, const float* cos_sin,
                                      void* k_pool, void* v_pool, const int* table, int table_stride, const int* token_slot,
                                      const int* positions, float* ws_o, float* ws_ml, int n_splits, void* out, int ldo,
                                      int n_rows, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers,
                                      int layer, float scale, int window, int whole, int split_rounds, int n_parts,
                                      hipStream_t stream);
// sampling.hip
int celeg_argmax_rows(const float* logits, int ld, int rows, int vocab, const float* fparams, const int* iparams,
                      uint8_t* seen, size_t seen_stride, int* out_tokens, int* last_tokens,
                      unsigned long long* best, unsigned int* arrived, hipStream_t stream);
int celeg_argmax_merge(const unsigned long long* best, int ld, int parts, int rows, const int* iparams, int* out_tokens,
                       int* last_tokens, hipStream_t stream);
int celeg_sample(const float* logits, int ld, int rows, int vocab, const float* fparams, const int* iparams,
                 uint8_t* seen, size_t seen_stride, int* out_tokens, int* last_tokens, const unsigned long long* best,
                 int best_ld, int best_parts, int best_cols, hipStream_t stream);
int celeg_mark_seen(uint8_t* seen, size_t stride, int n_slots, int vocab, const int* tokens, const int* slots, int n,
                    hipStream_t stream);
// gemv_slices.hip, gemm_rows.hip, gemv_fused.hip: the fused products for up to 64 rows
int celeg_gemv_params_size();
int celeg_gemv_slices_blocks(int M, int N, int K);
int celeg_gemv_slices_cols(int M, int N, int K);
int celeg_gemv_slices(const GemvParams* params, int epi, hipStream_t stream);
int celeg_stream_prepare(const float* h, int ldh, void* xb, int ldx, long long xb_k8, float* stats, int stats_ld,
                         int rows, int width, hipStream_t stream);
int celeg_embed_stream(const void* table, const int* ids, float* out, void* xb, int ldx, long long xb_k8, float* stats,
                       int stats_ld, int rows, int width, int vocab, hipStream_t stream);
int celeg_embed_stream_prologue(const void* table, int* ids, float* out, void* xb, int ldx, long long xb_k8, float* stats,
                                int stats_ld, int rows, int width, int vocab, int* block_table, int stride, int n_slots,
                                const int* updates, int capacity, const int* token_slot, const int* last_tokens,
                                hipStream_t stream);
int celeg_gemm_rows_blocks(int M, int N, int K, int epi);
int celeg_gemm_rows_workgroups(int M, int N, int K, int epi);
int celeg_gemm_rows_cols(int M, int N, int K, int epi);
int celeg_gemm_rows(const GemvParams* params, int epi, hipStream_t stream);
int celeg_gemv_fused(const GemvParams* params, int amode, int epi, int shape, hipStream_t stream);
int celeg_embed_stats(const void* table, const int* ids, float* out, float* stats, int stats_ld, int rows, int width,
                      int vocab, hipStream_t stream);
// gemm_tiles.hip: the fused products of many rows
int celeg_gemm_tiles_blocks(int M, int N, int K);
int celeg_gemm_tiles_params_size();
int celeg_gemm_tiles(const TileParams* params, int epi, hipStream_t stream);
// norm_step.hip
int celeg_norm_step(float* h, const void* y, int y_dtype, CelegNorm post, CelegNorm pre, void* out, int out_dtype,
                    const int* rows, int n_rows, int width, int write_back, hipStream_t stream);
int celeg_concat_rows(const float* a, const float* b, void* out, int out_dtype, int rows, int width, hipStream_t stream);
// sigmoid_attention.hip
int celeg_sigmoid_attention(const void* q, int ldq, const void* k_pool, const void* v_pool, int dtype, const int* table,
                            int table_stride, const int* token_slot, const int* positions, const float* temp,
                            const float* bias, const void* gate, int ldg, void* out, int ldo, int n_tokens, int q_heads,
                            int kv_heads, int head_dim, int page_tokens, int n_layers, int layer, float scale, int window,
                            hipStream_t stream);
int celeg_sigmoid_attention_fast_ok(int head_dim);
int celeg_sigmoid_attention_fast(int form, const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table,
                                 int table_stride, const int* cu_seqlens, const int* seq_slot, const int* seq_start, int n_seqs,
                                 int max_tiles, const float* temp, const float* bias, const void* gate, int ldg, void* out,
                                 int ldo, int q_heads, int kv_heads, int head_dim, int page_tokens, int n_layers, int layer,
                                 float scale, int window, hipStream_t stream);
// delta_rule.hip
int celeg_delta_prepare(const void* proj, int ld, int dtype, int col_b, int col_a, const float* conv_w, const float* a_log,
                        const float* dt_bias, const float* conv_state, size_t state_stride, const int* positions,
                        const int* token_seq, const int* seq_start, const int* token_slot, float* qk, float* v_out,
                        float* beta_decay, int n_tokens, int G, int H, int D, int V, int taps, hipStream_t stream);
int celeg_delta_conv_state(const void* proj, int ld, int dtype, float* conv_state, size_t state_stride, const int* cu_seqlens,
                           const int* seq_slot, int n_seqs, int n_channels, int taps, hipStream_t stream);
int celeg_delta_scan(const float* qk, const float* v, const float* beta_decay, float* state, size_t state_stride,
                     const int* cu_seqlens, const int* seq_slot, float* out, int n_seqs, int G, int H, int D, int V,
                     int general, const int* token_seq, float* pairs, int n_tokens, hipStream_t stream);
int celeg_delta_gated_norm(const float* o, const float* w, const void* gate, int ldg, int dtype, float eps, void* out,
                           int n_tokens, int H, int V, int act, hipStream_t stream);
// layer_glue.hip
int celeg_activation_bias(const void* x, int ldx, const float* bias, void* out, int ldo, int dtype, int rows, int cols, int act,
                          hipStream_t stream);
int celeg_residual_sum(float* h, const void* a, int lda, const void* b, int ldb, void* copy, int dtype, int rows, int width,
                       hipStream_t stream);
int celeg_token_gate(const void* z, int ldz, const void* table, int ld_table, int offset, const int* token_ids, void* g, int dtype,
                     int rows, int dim, hipStream_t stream);
int celeg_normed_mean(const void* a, int lda, const float* wa, const void* b, int ldb, const float* wb, float eps, float factor,
                      void* out, int dtype, int rows, int width, hipStream_t stream);
int celeg_depth_mix(float* history, size_t entry_stride, float* h, const float* w, int n, int rows, int width, hipStream_t stream);
int celeg_stream_add(float* h, const float* rows, const float* vec, int n_rows, int width, hipStream_t stream);
int celeg_softcap(float* x, size_t n, float cap, hipStream_t stream);
// conv_rope.hip
int celeg_conv_rope_store(const void* proj, int ld, int dtype, const float* conv_w, const float* conv_state, size_t state_stride,
                          const int* positions, const int* token_seq, const int* seq_start, const int* token_slot,
                          const float* inv_freq, int rotary_dim, int pairing, void* q_out, int ldq, void* k_pool, void* v_pool,
                          const int* table, int table_stride, int n_tokens, int H, int G, int D, int V, int taps, int page_tokens,
                          int n_layers, int layer, hipStream_t stream);
// biased_attention.hip
int celeg_kv_store(const void* k, int ldk, const void* v, int ldv, int dtype, void* k_pool, void* v_pool, const int* table,
                   int table_stride, const int* token_slot, const int* positions, int n_tokens, int kv_heads, int head_dim, int v_dim,
                   int page_tokens, int n_layers, int layer, hipStream_t stream);
int celeg_biased_attention(const void* q, int ldq, int dtype, const void* k_pool, const void* v_pool, const int* table,
                           int table_stride, const int* token_slot, const int* positions, const float* r1, const float* r2,
                           const void* gate, int ldg, void* out, int ldo, int n_tokens, int q_heads, int kv_heads, int head_dim,
                           int v_dim, int page_tokens, int n_layers, int layer, float scale, float coef, int every, int window,
                           int keep_first, int sink_one, hipStream_t stream);
// biased_attention_fast.hip
int celeg_biased_attention_fast_ok(int head_dim, int v_dim);
int celeg_biased_attention_fast(int form, const void* q, int ldq, const void* k_pool, const void* v_pool, const int* table, int table_stride,
                                const int* cu_seqlens, const int* seq_slot, const int* seq_start, int n_seqs, int max_tiles,
                                const float* r1, const float* r2, const void* gate, int ldg, void* out, int ldo, int q_heads,
                                int kv_heads, int head_dim, int v_dim, int page_tokens, int n_layers, int layer, float scale, float coef,
                                int every, int window, int keep_first, int sink_one, hipStream_t stream);
// linear_scan.hip
int celeg_lru_gates(const void* x, int ldx, int dtype, const float* conv_w, const float* conv_b, const float* ra_t, const float* ra_b,
                    const float* ri_t, const float* ri_b, const float* lam, const float* conv_state, size_t state_stride,
                    const int* positions, const int* token_seq, const int* seq_start, const int* token_slot, float* decay,
                    float* input, int n_tokens, int width, int blocks, int taps, float decay_scale, hipStream_t stream);
int celeg_lru_scan(const float* decay, const float* input, const void* y, int ldy, int dtype, float* state, size_t state_stride,
                   const int* cu_seqlens, const int* seq_slot, void* out, int ldo, int n_seqs, int width, int longest, hipStream_t stream);
int celeg_channel_decay(const void* z, int ldz, int dtype, const float* a_log, const float* dt_bias, float* decay, int n_tokens,
                        int heads, int dim, hipStream_t stream);
int celeg_gla_prepare(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, const void* z, int ldz, int dtype,
                      const float* z_bias, float inv_tau, float q_scale, float* qk, float* v32, float* decay, int n_tokens,
                      int qk_cols, int v_cols, hipStream_t stream);
int celeg_channel_scan(const float* qk, const float* v, const float* decay, const float* beta, int ld_beta, float* state,
                       size_t state_stride, const int* cu_seqlens, const int* seq_slot, float* out, int n_seqs, int G, int H, int D,
                       int V, int general, hipStream_t stream);
}
