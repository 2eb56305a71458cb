// The entry points of the kernels in this folder, for the native step program (host/program.cpp),
// which launches them without a round trip through Python. Every function returns 0 on success and
// leaves a message for me_last_error() otherwise; a refused size launches nothing.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

extern "C" {
const char* me_last_error();
int me_embed(void* x, const void* table, const int* ids, int num_tokens, int hidden, int vocab, float scale, int dtype,
             hipStream_t stream);
int me_embed_fed(void* x, const void* table, const int* ids, const int* fed_rows, const int* fed_tokens, int num_tokens,
                 int hidden, int vocab, float scale, int dtype, hipStream_t stream);
int me_scale_f32(float* x, float scale, long long count, hipStream_t stream);
int me_add_rmsnorm(void* x, const void* delta, const float* parts, int num_parts, long long part_stride, const float* w,
                   void* h, const int* rows, int num_rows, int dim, float eps, int write_x, int dtype, hipStream_t stream);
int me_residual_add(void* x, const void* delta, const float* parts, int num_parts, long long part_stride, int num_rows, int dim,
                    int dtype, hipStream_t stream);
int me_rmsnorm(const void* in, const float* w, void* out, int num_rows, int dim, float eps, int dtype, hipStream_t stream);
int me_swiglu(const void* gu, void* act, int num_tokens, int inter, int gate, int dtype, hipStream_t stream);
int me_qk_norm_rope_scatter(const void* qkv, const float* q_w, const float* k_w, const float* rope_table,
                            const int* positions, const int* token_item, const int* block_table, int table_width,
                            void* q_out, void* k_cache, void* v_cache, int num_tokens, int nh, int nkv, int d, int rd, int bs,
                            float eps, int write_kv, int dtype, const int* item_start, int num_items, int num_segments,
                            hipStream_t stream);
int me_attention_general(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                         const int* token_item, const int* block_table, int table_width, void* out, int num_tokens, int nh,
                         int nkv, int d, int bs, int window, float scale, int dtype, int items, hipStream_t stream);
int me_attention_general_ext(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                             const int* token_item, const int* block_table, int table_width, void* out, int num_tokens, int nh,
                             int nkv, int d, int dv, int bs, int window, int keep_first, const float* unturn, int un_pairing,
                             float scale, int dtype, int items, hipStream_t stream);
int me_qkv_rotate_scatter(const void* qkv, const float* q_w, const float* k_w, const float* rope_table, int rd, int pairing,
                          const float* v_table, int v_pairing, const int* positions, const int* token_item,
                          const int* block_table, int table_width, void* q_out, void* k_cache, void* v_cache, int num_tokens,
                          int nh, int nkv, int d, int dv, int bs, float eps, int dtype, hipStream_t stream);
int me_qkv_rotate_scatter_tiles(const void* qkv, const float* q_w, const float* k_w, const float* rope_table, int rd, int pairing,
                                const float* v_table, int v_pairing, const int* positions, const int* token_item,
                                const int* block_table, int table_width, void* q_out, void* k_cache, void* v_cache,
                                int num_tokens, int nh, int nkv, int d, int dv, int bs, float eps, int dtype,
                                const int* item_start, int num_items, int num_segments, hipStream_t stream);
int me_add_group_rmsnorm(void* x, const void* delta, const float* parts, int num_parts, long long part_stride, float delta_scale,
                         const float* w, void* h, const int* rows, int num_rows, int dim, int groups, float eps, int write_x,
                         int dtype, hipStream_t stream);
int me_add_group_rmsnorm2(void* x, const void* delta, const float* parts, int num_parts, long long part_stride, const void* delta2,
                          const float* parts2, int num_parts2, long long part_stride2, float delta_scale, const float* w, void* h,
                          const int* rows, int num_rows, int dim, int groups, float eps, int write_x, int dtype,
                          hipStream_t stream);
int me_residual_add_scaled(void* x, const void* delta, const float* parts, int num_parts, long long part_stride, float scale,
                           int num_rows, int dim, int dtype, hipStream_t stream);
int me_decay_state_padded_dim(int d);
long long me_decay_state_workspace(long long tokens, long long items, int heads, int d, int dv);
int me_decay_state(const void* proj, const float* rope_table, int rd, int pairing, const int* positions, const float* decay,
                   const float* norm_w, float* state, const int* item_start, const int* state_slots, void* out, void* workspace,
                   int num_tokens, int items, int heads, int d, int dv, int in_act, float key_scale, int norm_kind, int gate_act,
                   float eps, int dtype, int longest_item, hipStream_t stream);
int me_attention_mfma_supported(int d, int bs);
int me_attention_decode_fused_supported(int d, int bs, int rotary_dim, int group);
int me_attention_prefill_columns(int wide);
int me_attention_decode_bf16(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                             const int* block_table, int table_width, void* out, float* part_o, float* part_ml, int items,
                             int nh, int nkv, int d, int bs, int window, float scale, int split_keys, int num_splits,
                             int max_ctx, const int* live_items, int full_splits, int waves_wanted, const int* step_flags,
                             hipStream_t stream);
int me_attention_decode_fused_bf16(const void* qkv, const float* q_w, const float* k_w, const float* rope_table,
                                   int rotary_dim, float eps, int write_kv, void* k_cache, void* v_cache, const int* item_ctx,
                                   const int* block_table, int table_width, void* out, float* part_o, float* part_ml,
                                   int items, int nh, int nkv, int d, int bs, int window, float scale, int split_keys,
                                   int num_splits, int max_ctx, const int* live_items, int full_splits, int waves_wanted,
                                   const int* step_flags, hipStream_t stream);
// Decode steps of very few items: the launch leaves its splits' partial results (out == nullptr) and the output
// projection adds them up itself.
int me_attention_decode_leaves_parts(int items, int nh, int nkv, int d, int num_splits);
int me_attention_out_product_runs(int nh);
int me_attention_out_product_supported(int items, int nh, int d, int n, int num_splits);
int me_attention_out_product_bf16(const float* part_o, const float* part_ml, int num_splits, const void* W, float* parts,
                                  int items, int nh, int d, int n, hipStream_t stream);
int me_attention_prefill_bf16(const void* q, const void* k_cache, const void* v_cache, int num_items, const int* block_table,
                              int table_width, void* out, const int* work, const int* bundle_first, int num_bundles,
                              float* part_o, float* part_ml, const int* token_chunks, int max_chunks, int num_tokens, int nh,
                              int nkv, int d, int bs, int window, float scale, int columns, hipStream_t stream);
int me_attention_prefill_bf16_kept(const void* q, const void* k_cache, const void* v_cache, int num_items, const int* block_table,
                                   int table_width, void* out, const int* work, const int* bundle_first, int num_bundles,
                                   float* part_o, float* part_ml, const int* token_chunks, int max_chunks, int num_tokens,
                                   int nh, int nkv, int d, int bs, int window, int keep_first, float scale, int columns,
                                   hipStream_t stream);
int me_attention_decode_bf16_kept(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                                  const int* block_table, int table_width, void* out, float* part_o, float* part_ml, int items,
                                  int nh, int nkv, int d, int bs, int window, int keep_first, float scale, int split_keys,
                                  int num_splits, int max_ctx, const int* live_items, int full_splits, int waves_wanted,
                                  const int* step_flags, hipStream_t stream);
int me_attention_prefill_bf16_pooled(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                     int pool_block, int num_items, const int* block_table, int table_width, void* out,
                                     long long out_row, int out_col, float out_scale, const int* work, const int* bundle_first,
                                     int num_bundles, float* part_o, float* part_ml, const int* token_chunks, int max_chunks,
                                     int num_tokens, int nh, int nkv, int d, int bs, int window, float scale, int columns,
                                     hipStream_t stream);
int me_attention_decode_bf16_pooled(const void* q, const void* k_cache, const void* v_cache, const void* k_pool, const void* v_pool,
                                    int pool_block, const int* item_ctx, const int* block_table, int table_width, void* out,
                                    long long out_row, int out_col, float out_scale, float* part_o, float* part_ml, int items, int nh,
                                    int nkv, int d, int bs, int window, float scale, int split_keys, int num_splits, int max_ctx,
                                    const int* live_items, int full_splits, int waves_wanted, const int* step_flags,
                                    hipStream_t stream);
int me_attention_general_gated(const void* q, const void* k_cache, const void* v_cache, const int* positions,
                               const int* token_item, const int* block_table, int table_width, void* out, int num_tokens, int nh,
                               int nkv, int d, int dv, int bs, int window, int keep_first, const float* unturn, int un_pairing,
                               float scale, const float* sink, const void* gate, long long gate_row, int dtype, int items,
                               hipStream_t stream);
int me_qkv_rotate_scatter_rows(const void* qkv, long long row_stride, const float* q_w, const float* k_w, const float* rope_table,
                               int rd, int pairing, const float* v_table, int v_pairing, float q_temp_coef, int q_temp_every,
                               const int* positions, const int* token_item, const int* block_table, int table_width, void* q_out,
                               void* k_cache, void* v_cache, int num_tokens, int nh, int nkv, int d, int dv, int bs, float eps,
                               int dtype, const int* item_start, int num_items, int num_segments, hipStream_t stream);
int me_streams_spread(float* xs, long long per_stream, int S, hipStream_t stream);
int me_streams_norm(float* xs, long long per_stream, int S, const void* delta, const float* parts, int num_parts,
                    long long part_stride, const float* mix_out, const float* w_in, const float* w, void* h, const int* rows,
                    int num_rows, int dim, float eps, int write_x, int dtype, hipStream_t stream);
int me_latent_prepare(const void* proj, long long row_stride, const float* norm_w, const float* rope, const int* positions,
                      const int* token_item, const int* block_table, int table_width, void* qa, void* k_cache, void* v_cache,
                      int num_tokens, int nh, int d, int r, int rank, int v_rows, int bs, float eps, int dtype, hipStream_t stream);
int me_head_product(const void* x, long long x_row, long long x_head, const void* W, void* out, long long out_row,
                    long long out_head, const void* gate, long long gate_row, int num_tokens, int heads, int n, int k, int dtype,
                    hipStream_t stream);
int me_latent_values_supported(int num_splits, int rank);
int me_latent_values_bf16(const float* part_o, const float* part_ml, int num_splits, int dk, int rank, const float* sink, const void* W_uv,
                          const void* gate, long long gate_row, void* out, int items, int nh, int dv, hipStream_t stream);
int me_head_gate(void* rows, const void* gate, long long gate_row, int num_tokens, int heads, int n, int dtype, hipStream_t stream);
int me_routed_ff_max_tiles(long long tokens, int E, int top);
long long me_routed_ff_workspace(long long tokens, int E, int top, int ff, int elem);
int me_routed_ff(const void* h, const float* Wr, const void* W_gu, const void* W_down, float* parts, void* workspace, int num_tokens,
                 int hidden, int E, int top, int ff, int act, int dtype, hipStream_t stream);
int me_attention_decode_bf16_sink(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx,
                                  const int* block_table, int table_width, void* out, float* part_o, float* part_ml, int items,
                                  int nh, int nkv, int d, int bs, const float* sink, float scale, int split_keys, int num_splits,
                                  int max_ctx, const int* live_items, int full_splits, int waves_wanted, const int* step_flags,
                                  hipStream_t stream);
int me_attention_prefill_bf16_sink(const void* q, const void* k_cache, const void* v_cache, int num_items, const int* block_table,
                                   int table_width, void* out, const int* work, const int* bundle_first, int num_bundles,
                                   float* part_o, float* part_ml, const int* token_chunks, int max_chunks, int num_tokens, int nh,
                                   int nkv, int d, int bs, const float* sink, float scale, int columns, hipStream_t stream);
int me_unturn_rows(void* rows, const float* table, int pairing, const int* positions, int num_tokens, int heads, int n,
                   int dtype, hipStream_t stream);
int me_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K, hipStream_t stream);
int me_gemm_plain(const void* A, const void* W, void* C, int M, int N, int K, int in_dtype, int out_dtype, hipStream_t stream);
int me_gemm_bf16_small(const void* X, const float* x_in, const void* delta, const float* w_norm, float eps, float* x_out,
                       const void* W, void* C, int M, int N, int K, int norm, int swiglu, int out_dtype, int k_splits,
                       hipStream_t stream);
int me_gemm_bf16_stream_splits(int M, int N, int K, int compute_units);
void me_gemm_bf16_stream_plan(int M, int N, int K, int gated, int k_splits, int compute_units, int* out);
int me_gemm_bf16_stream(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype, int k_splits,
                        int compute_units, hipStream_t stream);
int me_gemm_bf16_stream_scaled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                               int compute_units, const float* row_ss, int ss_blocks, int ss_dim, float eps, hipStream_t stream);
int me_gemm_bf16_stream_carry_blocks(int M, int N, int K, int compute_units);
int me_gemm_bf16_stream_carry(const void* X, const void* W, float* x, void* h, float* ss, const float* w_norm, int M, int N, int K,
                              int compute_units, hipStream_t stream);
int me_gemm_bf16_small_scaled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                              const float* row_ss, int ss_blocks, int ss_dim, float eps, hipStream_t stream);
int me_gemm_bf16_stream_norm_fits(int M, int K);
int me_gemm_bf16_stream_norm(const float* x_in, const void* delta, const float* parts, int num_parts, long long part_stride,
                             const float* w_norm, float eps, float* x_out, const void* W, void* C, int M, int N, int K,
                             int swiglu, int out_dtype, int compute_units, hipStream_t stream);
int me_gemm_bf16_stream_norm_streams(const float* xs, long long stream_stride, int streams, const void* delta, const float* parts,
                                     int num_parts, long long part_stride, const float* mix_out, const float* w_in, const float* w_norm,
                                     float eps, float* xs_out, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype,
                                     int compute_units, hipStream_t stream);
int me_gemm_bf16_tiled(const void* X, const void* W, void* C, int M, int N, int K, int swiglu, int out_dtype, int shape,
                       hipStream_t stream);
int me_gemm_bf16_library(const void* X, const void* W, void* C, int M, int N, int K, int out_dtype, hipStream_t stream);
int me_gemm_bf16_library_add(const void* X, const void* W, float* C, int M, int N, int K, hipStream_t stream);
int me_routed_ff_scored(const void* h, const float* Wr, const void* W_gu, const void* W_down, float* parts, void* workspace,
                        int num_tokens, int hidden, int E, int top, int ff, int act, float limit, int scoring, int n_groups,
                        int keep_groups, float route_scale, float* shared_gate, int dtype, hipStream_t stream);
int me_gated_rows(const void* gu, const float* row_gate, void* act_out, int num_tokens, int ff, int act, float limit, int dtype,
                  hipStream_t stream);
int me_attention_general_pooled(const void* q, const void* k_cache, const void* v_cache, const int* positions, const int* token_item,
                                const int* block_table, int table_width, void* out, int num_tokens, int nh, int nkv, int d, int dv,
                                int bs, int window, int keep_first, const float* unturn, int un_pairing, float scale, const float* sink,
                                const void* gate, long long gate_row, const void* k_pool, const void* v_pool, int pool,
                                long long out_row, int out_col, float out_scale, int dtype, int items, hipStream_t stream);
int me_whole_norm_scatter(const void* proj, long long row, int c_q, int c_k, int c_v, const float* q_w, const float* k_w,
                          const int* positions, const int* token_item, const int* block_table, int table_width, void* q_out,
                          void* k_cache, void* v_cache, void* k_pool, void* v_pool, int num_tokens, int nh, int nkv, int d, int dv,
                          int bs, int pool, float eps, int dtype, hipStream_t stream);
int me_whole_norm_scatter_step(const void* proj, long long row, int c_q, int c_k, int c_v, const float* q_w, const float* k_w,
                          const int* positions, const int* token_item, const int* block_table, int table_width, void* q_out,
                          void* k_cache, void* v_cache, void* k_pool, void* v_pool, int num_tokens, int nh, int nkv, int d, int dv,
                          int bs, int pool, float eps, int single_tokens, int dtype, hipStream_t stream);
int me_delta_rule(const void* proj, long long row, int c_r, int c_k, int c_v, int c_g, int c_a, int c_w1, const void* W2,
                  const float* w0, const float* a_bias, const float* norm_w, float* state, const int* item_start,
                  const int* state_slots, void* out, long long out_row, int out_col, float out_scale, int num_tokens, int items,
                  int heads, int d, int lora, float eps, float decay_coef, int dtype, hipStream_t stream);
long long me_delta_rule_workspace(long long tokens, int heads, int d);
int me_delta_rule_steps(const void* proj, long long row, int c_r, int c_k, int c_v, int c_g, int c_a, int c_w1, const void* W2,
                  const float* w0, const float* a_bias, const float* norm_w, float* state, const int* item_start,
                  const int* state_slots, void* out, long long out_row, int out_col, float out_scale, int num_tokens, int items,
                  int heads, int d, int lora, float eps, float decay_coef, int dtype, void* workspace, hipStream_t stream);
int me_sample_chunks(int vocab);
int me_sample(const float* logits, int num_rows, int vocab, const float* temperatures, const uint64_t* keys, int* out,
              void* workspace, hipStream_t stream);
int me_attention_general_capped(const void* q, const void* k_cache, const void* v_cache, const int* positions, const int* token_item,
                                const int* block_table, int table_width, void* out, int num_tokens, int nh, int nkv, int d, int dv,
                                int bs, int window, int keep_first, const float* unturn, int un_pairing, float scale, const float* sink,
                                const void* gate, long long gate_row, const void* k_pool, const void* v_pool, int pool,
                                long long out_row, int out_col, float out_scale, float softcap, int dtype, int items, hipStream_t stream);
int me_latent_prepare_for(const void* proj, long long row_stride, const float* norm_w, const float* rope, const int* positions,
                          const int* token_item, const int* block_table, int table_width, void* qa, void* k_cache, void* v_cache,
                          int num_tokens, int nh, int d, int r, int rank, int v_rows, int bs, float eps, int writes, int dtype,
                          hipStream_t stream);
int me_routed_ff_routed(const void* h, const float* Wr, const void* W_gu, const void* W_down, float* parts, void* workspace, int num_tokens,
                        int hidden, int E, int top, int ff, int act, float limit, int scoring, int n_groups, int keep_groups,
                        float route_scale, float* shared_gate, int n_identity, const float* correction, int dtype, hipStream_t stream);
int me_result_norm_add(float* x, const void* delta, const float* parts, int num_parts, long long part_stride, const float* w, void* h,
                       int num_tokens, int dim, float eps, float scale, int dtype, hipStream_t stream);
int me_token_gate(const void* z, const void* table, const int* ids, const int* fed_rows, const int* fed_tokens, void* out, int num_tokens,
                  int n, long long table_row, int col0, int vocab, int act, int dtype, hipStream_t stream);
int me_act_rows(const void* in, void* out, long long total, int act, int dtype, hipStream_t stream);
int me_conv_norm_rope_scatter(const void* proj, long long row, int c_q, int c_k, int c_v, const float* conv_w, int taps, float* state,
                              const int* state_slots, const int* item_start, const float* q_w, const float* k_w, const float* rope,
                              int rotary, const int* positions, const int* token_item, const int* block_table, int table_width,
                              void* q_out, void* k_cache, void* v_cache, int num_tokens, int items, int nh, int nkv, int d, int dv, int bs,
                              float eps, int dtype, hipStream_t stream);
int me_time_shift(const void* h, float* state, long long state_row, long long prev_at, const int* state_slots, const int* item_start,
                  const int* token_item, const int* positions, const float* mu, void* const* outs, long long out_stride, int num_tokens, int items,
                  int width, int dtype, hipStream_t stream);
long long me_time_mix_workspace(long long tokens, int heads, int d);
int me_time_mix(const void* r, const void* k, const void* v, const void* gate, const void* z, const void* W2, const float* w0,
                const float* bonus, const float* norm_w, float* state, long long state_row, const int* state_slots, const int* item_start,
                void* out, long long out_row, int out_col, float out_scale, int num_tokens, int items, int heads, int d, int rank, float eps,
                long long in_stride, int dtype, void* workspace, hipStream_t stream);
int me_attention_decode_bf16_placed(const void* q, const void* k_cache, const void* v_cache, const int* item_ctx, const int* block_table,
                                    int table_width, void* out, long long out_row, int out_col, float out_scale, float* part_o,
                                    float* part_ml, int items, int nh, int nkv, int d, int bs, int window, float scale, float softcap,
                                    const float* sink, int split_keys, int num_splits, int max_ctx, const int* live_items, int full_splits,
                                    int waves_wanted, const int* step_flags, hipStream_t stream);
int me_attention_prefill_bf16_placed(const void* q, const void* k_cache, const void* v_cache, int num_items, const int* block_table,
                                     int table_width, void* out, long long out_row, int out_col, float out_scale, const int* work,
                                     const int* bundle_first, int num_bundles, float* part_o, float* part_ml, const int* token_chunks,
                                     int max_chunks, int num_tokens, int nh, int nkv, int d, int bs, int window, float scale, float softcap,
                                     const float* sink, int columns, hipStream_t stream);
}
