// C entry points of the gfx950 kernel library.  Every function launches on the
// given stream, allocates nothing, and returns 0 or a negative code with a
// message behind pae_last_error().  dtype codes: 0 float32, 1 bfloat16.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {
const char* pae_last_error();
int pae_device_arch(char* out, int cap);  // "gfx950" on the card the kernels are built for

int pae_embedding(int dtype, void* out, const void* table, const int* ids, int num_tokens, int hidden,
                  int vocab, float scale, hipStream_t stream);
int pae_embedding_rows(int dtype, void* residual, const void* table, const int* ids, int num_tokens, int hidden,
                       int vocab, float scale, void* next_rows, const void* next_w, int next_w_is_f32,
                       float* next_stats, hipStream_t stream);
int pae_scaled_rows(void* out, const void* rows, const float* row_stats, int row_stat_tiles, float eps, int num_rows,
                    int hidden, hipStream_t stream);
int pae_logits_finish(float* logits, int64_t n, float scale, float cap, hipStream_t stream);
int pae_add_rmsnorm(int dtype, void* residual, const void* delta, int parts, int64_t part_stride,
                    const void* weight, int w_is_f32, float eps, const int* rows, void* out, int num_rows,
                    int hidden, int write_residual, hipStream_t stream);
int pae_residual_add(int dtype, void* residual, const void* delta, int64_t n, hipStream_t stream);
int pae_copy_i32(int* dst, const int* src, int n, hipStream_t stream);  // src: device or pinned host memory
int pae_scatter_i32(int* dst, const int* dst_idx, const int* src, const int* src_idx, int n, hipStream_t stream);
int pae_rope_table(float* cos_sin, const int* positions, const float* inv_freq, int num_tokens, int half,
                   hipStream_t stream);
int pae_rope_kv_write(int dtype, void* qkv, int64_t row_stride, int num_tokens, int nh, int nkv, int hd, int rot,
                      const void* bias, int b_is_f32, const float* cos_sin, const int* positions, const int* tok_seq, const int* block_tables,
                      int max_blocks, int bs, void* k_cache, void* v_cache, int write_kv, hipStream_t stream);
int pae_swiglu(int dtype, void* out, const void* x, int num_tokens, int inter, int block, hipStream_t stream);
int pae_gated_act(int dtype, void* out, const void* x, int num_tokens, int inter, int block, int kind,
                  hipStream_t stream);  // act(gate) * up, act by code: 0 gelu (erf), 1 gelu (tanh), 2 silu
int pae_gemm_plain_batched(int in_dtype, int out_dtype, void* C, int64_t ldc, int64_t batch_c, const void* A, int64_t lda,
                           int64_t batch_a, const void* W, int64_t batch_w, const void* bias, int b_is_f32, int M, int N,
                           int K, int batch, hipStream_t stream);
int pae_gemm_plain(int in_dtype, int out_dtype, void* C, int64_t ldc, const void* A, int64_t lda, const void* W,
                   const void* bias, int b_is_f32, int M, int N, int K, hipStream_t stream);
int pae_gemm_skinny(int epilogue, void* out, int64_t ldc, const void* A, int64_t lda, const void* W,
                    const void* bias, int b_is_f32, int M, int N, int K, int splits, int64_t part_stride,
                    float* ticket_parts, int* ticket_counters, const float* row_stats, int row_stat_tiles,
                    float row_eps, void* next_rows, int64_t ld_next, const void* next_w, int next_w_is_f32,
                    float* next_stats, hipStream_t stream);
int pae_gemm_skinny_act(void* out, int64_t ldc, const void* A, int64_t lda, const void* W, const void* bias,
                        int b_is_f32, int M, int N, int K, int splits, float* ticket_parts, int* ticket_counters,
                        int act, hipStream_t stream);
int pae_gemm_skinny_gated(void* out, int64_t ldc, const void* A, int64_t lda, const void* W, int M, int N, int K, int splits,
                          float* ticket_parts, int* ticket_counters, int act, hipStream_t stream);
int pae_skinny_ticket_slots(int M, int N);
int64_t pae_skinny_ticket_floats(int M, int N, int splits);
int pae_gemm_skinny_rope(void* q_out, int64_t ldq, const void* A, int64_t lda, const void* W, const void* bias,
                         int b_is_f32, int M, int K, int nh, int nkv, int hd, int rot, const float* cos_sin,
                         const int* positions, const int* tok_seq, const int* block_tables, int max_blocks, int bs,
                         void* k_cache, void* v_cache, int splits, float* ticket_parts, int* ticket_counters,
                         const float* row_stats, int row_stat_tiles, float row_eps, hipStream_t stream);
int pae_paged_attention_generic(int dtype, void* out, int64_t out_stride, const void* q, int64_t q_stride,
                                const void* k_cache, const void* v_cache, const int* positions,
                                const int* tok_seq, const int* block_tables, int max_blocks, int bs,
                                int num_tokens, int nh, int nkv, int hd, float scale, int window,
                                hipStream_t stream);
// attention with values of their own width `vd`, a cap on the scores (0: none) and per-head sinks (null: none)
int pae_paged_attention_capped(int dtype, void* out, int64_t out_stride, const void* q, int64_t q_stride,
                               const void* k_cache, const void* v_cache, const int* positions, const int* tok_seq,
                               const int* block_tables, int max_blocks, int bs, int num_tokens, int nh, int nkv, int hd,
                               int vd, float scale, int window, float cap, const float* sinks, hipStream_t stream);
// the same with a mask in chunks, a bias by distance, an output gate, and values shared with the keys
int pae_paged_attention_masked(int dtype, void* out, int64_t out_stride, const void* q, int64_t q_stride,
                               const void* k_cache, const void* v_cache, const int* positions, const int* tok_seq,
                               const int* block_tables, int max_blocks, int bs, int num_tokens, int nh, int nkv, int hd,
                               int vd, float scale, int window, float cap, const float* sinks, int chunked,
                               const float* slopes, const void* gate, int64_t gate_stride, int shared_kv,
                               hipStream_t stream);
// a stream kept as several copies joined by hyper-connections: see hyper.hip
int pae_hyper_norm(int dtype, float* streams, int num_streams, const void* y, int parts, int64_t part_stride,
                   const void* ls, int ls_is_f32, const float* mix, const float* outw, const float* inw,
                   const void* weight, int w_is_f32, float eps, const int* rows, void* out, int num_rows, int hidden,
                   int write_back, hipStream_t stream);
int pae_hyper_spread(float* streams, const float* src, int num_rows, int num_streams, int hidden, hipStream_t stream);
int pae_hyper_collapse(float* out, const float* streams, int num_rows, int num_streams, int hidden, hipStream_t stream);
// rows [q | k | v | ..]: short causal convolutions with per-request state, per-head RMS norm, cache write
int pae_conv_norm_store(int dtype, const void* proj, int64_t row_stride, void* q_out, int64_t q_stride, int num_tokens,
                        int num_seqs, const int* tok_seq, const int* positions, const int* seq_runs, const int* slots,
                        const float* conv_w, float* conv_tail, int64_t tail_slot_stride, int taps, int nh, int nkv, int hd,
                        int vd, int norm_heads, float eps, const int* block_tables, int max_blocks, int bs, void* k_cache,
                        void* v_cache, hipStream_t stream);
// rows [q heads of (nope + rd) | latent + rd]: latent norm, rotation, write of the latent pages: see latent.hip
int pae_latent_prepare(int dtype, const void* proj, int64_t row_stride, void* q_full, int64_t qf_stride, int num_tokens,
                       int nh, int nope, int rd, int rot, int interleaved, int rank, const void* norm_w, int w_is_f32,
                       float eps, const float* cos_sin, const int* positions, const int* tok_seq, const int* block_tables,
                       int max_blocks, int bs, void* latent, void* latent_t, hipStream_t stream);
int pae_heads_product_few(void* out, int64_t ldc, int64_t head_c, const void* a, int64_t lda, int64_t head_a, const void* w,
                          int M, int N, int K, int heads, hipStream_t stream);  // bfloat16, a few rows, one product per head
// latent attention on the matrix cores: see attention_latent.hip
int pae_latent_attn_supported(int kd, int C, int bs);
int pae_latent_attn_columns(int H, int ct);
int pae_latent_attn_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* latent,
                         const void* latent_t, const int* tiles, int num_tiles, int ct, const int* positions,
                         const int* block_tables, int max_blocks, int bs, int H, int kd, int C, float scale, int window,
                         int chunked, float* part_acc, float* part_ml, const float* sinks, hipStream_t stream);
int pae_latent_attn_split();
// rows [q | k | v]: RMS norm of q and of k over the whole projection, or head by head with one weight that the
// heads share (`per_head`; weights null: none), rotation, cache write
int pae_qk_norm_rotate_store(int dtype, void* qkv, int64_t row_stride, int num_tokens, int nh, int nkv, int hd, int vd,
                             const void* q_w, const void* k_w, int w_is_f32, float eps, int rot, int interleaved,
                             const float* cos_sin, float magnitude, const int* positions, const int* tok_seq,
                             const int* block_tables, int max_blocks, int bs, void* k_cache, void* v_cache, int write_kv,
                             int per_head, hipStream_t stream);
// blocks that normalise a branch's output: see branch_norm.hip
int pae_rows_from_residual(int dtype, void* out, const float* residual, int64_t n, hipStream_t stream);
int pae_norm_scale_add(int dtype, float* residual, const void* y, int parts, int64_t part_stride, const void* weight,
                       int w_is_f32, float eps, float scale, void* next, int num_rows, int hidden, hipStream_t stream);
int pae_activation(int dtype, void* x, int64_t n, int kind, hipStream_t stream);
// the gated delta rule over a step's projected rows: see delta_rule.hip
int pae_delta_rule_step(int dtype, const void* proj, int64_t row_stride, int num_tokens, int num_seqs, const int* tok_seq,
                        const int* positions, const int* seq_runs, const int* slots, const float* conv_w,
                        float* conv_tail, int64_t tail_slot_stride, int taps, int G, int H, int D, int V,
                        const float* a_log, const float* dt_bias, float unit_eps, float* state,
                        int64_t state_slot_stride, const void* norm_w, int w_is_f32, float norm_eps, float* work,
                        void* out, const void* gate_in, int64_t gate_stride, int gate_sigmoid, const void* b_in,
                        int64_t b_stride, const void* a_in, int64_t a_stride, int channel_decay, hipStream_t stream);
int64_t pae_delta_rule_work_floats(int num_tokens, int G, int H, int D, int V, int channel_decay);
// a matrix memory with exponential gates over a step's projected rows: see matrix_memory.hip
int pae_matrix_memory_step(int dtype, const void* proj, int64_t row_stride, const void* gate_in, int64_t gate_stride,
                           const float* gate_logits, int num_tokens, int num_seqs, const int* seq_runs, const int* slots,
                           int H, int D, int V, float gate_cap, float* state, int64_t state_slot_stride, float* maximum,
                           int64_t max_slot_stride, const void* norm_w, int w_is_f32, float norm_eps, float floor_eps,
                           float* work, void* out, hipStream_t stream);
int64_t pae_matrix_memory_work_floats(int num_tokens, int H, int D, int V);
// the embedding with a hashed table of token pairs added: see hashed_embedding.hip
int pae_embedding_pairs(int dtype, float* out, const void* table, const void* pair_table, const int* ids,
                        const int* positions, const int* tok_seq, const int* slots, int* last_token, int num_tokens,
                        int hidden, int vocab, float scale, int buckets, int mul_prev, int mul_cur, hipStream_t stream);
// residual += terms; two norms of the new residual: see parallel_norm.hip
int pae_sum_norm2(int dtype, float* residual, int num_terms, const void* const* term_ptr, const int* term_is_f32,
                  const int* term_parts, const int64_t* term_part_stride, const float* term_scale, const void* w1,
                  int w1_is_f32, const void* w2, int w2_is_f32, float eps, const int* rows, void* out1, void* out2,
                  int num_rows, int hidden, int write_residual, hipStream_t stream);
// a sublayer's output joins the stream through the norm after it; the norm before the next sublayer: see sandwich_norm.hip
int pae_norm_join(int dtype, float* residual, int num_terms, const void* const* term_ptr, const int* term_is_f32,
                  const int* term_parts, const int64_t* term_part_stride, const float* term_scale, const void* w_out,
                  int w_out_is_f32, float eps, const void* w_next, int w_next_is_f32, float eps_next, void* normed,
                  void* rows, int num_rows, int hidden, hipStream_t stream);
// gated linear attention over a step's projected rows: see linear_attention.hip
int pae_linear_attention_step(int dtype, const void* proj, int64_t row_stride, const void* z_in, int64_t z_stride,
                              const void* z_bias, int bias_is_f32, float tau, const void* gate_in, int64_t gate_stride,
                              int gate_sigmoid, int num_tokens, int num_seqs, const int* seq_runs, const int* slots, int H,
                              int D, int V, float* state, int64_t state_slot_stride, const void* norm_w, int w_is_f32,
                              float norm_eps, float* work, void* out, hipStream_t stream);
int64_t pae_linear_attention_work_floats(int num_tokens, int H, int D, int V);
// a learned row per position added to the embedding; a layer's columns of a second token table: see token_inputs.hip
int pae_embedding_positions(int dtype, float* out, const void* table, const int* ids, const void* rows,
                            const int* positions, int num_tokens, int hidden, int vocab, float scale, hipStream_t stream);
int pae_token_gate(int dtype, void* out, const void* gate, int64_t gate_stride, const void* columns, const int* ids,
                   int num_tokens, int dim, int kind, hipStream_t stream);
// float32 sums of a few output features from rows of either type: see moe.hip
int pae_project_f32(int dtype, float* out, int64_t ldo, const void* A, int64_t lda, const void* W, const void* bias,
                    int b_is_f32, int M, int N, int K, hipStream_t stream);
int pae_moe_route(const float* logits, int num_tokens, int experts, int groups, int keep, int top, float scale,
                  const float* choice_bias, int* chosen, float* weights, hipStream_t stream);
int pae_moe_gate_up(int dtype, void* act, const void* x, int64_t ldx, const void* gate_w, const void* up_w,
                    const int* chosen, int num_tokens, int top, int hidden, int inter, int act_kind, hipStream_t stream);
int pae_moe_tile_rows(int pairs);
int pae_moe_max_tiles(int pairs, int experts);
int pae_moe_tiles_supported(int hidden, int inter);
int pae_moe_experts_tiles(float* y, const void* x, int64_t ldx, const void* gate_w, const void* up_w, const void* down_w,
                          const int* chosen, const float* weights, int num_tokens, int top, int experts, int hidden,
                          int inter, int act_kind, int* order, int* tiles, void* act, hipStream_t stream);
int pae_moe_down(int dtype, float* out, const void* act, const void* down_w, const int* chosen, const float* weights,
                 int num_tokens, int top, int hidden, int inter, hipStream_t stream);
int pae_attn_decode_split();
int pae_attn_decode_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                         const void* v_cache, const int* dec_work, int num_dec, const int* block_tables,
                         int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window, void* part_acc,
                         void* part_ml, hipStream_t stream);
int pae_attn_prefill_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                          const void* v_cache, const int* tiles, int num_tiles, const int* positions,
                          const int* block_tables, int max_blocks, int bs, int nh, int nkv, int hd, float scale,
                          int window, hipStream_t stream);
// the two above with capped scores (cap > 0: s <- cap tanh(s / cap)) and per-head sinks (float32 [nh] or null)
int pae_attn_decode_capped_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                                const void* v_cache, const int* dec_work, int num_dec, const int* block_tables,
                                int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window, float cap,
                                const float* sinks, void* part_acc, void* part_ml, hipStream_t stream);
int pae_attn_prefill_capped_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                                 const void* v_cache, const int* tiles, int num_tiles, const int* positions,
                                 const int* block_tables, int max_blocks, int bs, int nh, int nkv, int hd, float scale,
                                 int window, float cap, const float* sinks, hipStream_t stream);
// the two with the window read as a chunk length (`chunked`), a bias by distance (`slopes` float32 [nh] or null:
// score -= slopes[h] (position - key)) and a gate on the output (`gate` bfloat16 rows [token][nh * hd] or null)
int pae_attn_decode_biased_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                                const void* v_cache, const int* dec_work, int num_dec, const int* block_tables,
                                int max_blocks, int bs, int nh, int nkv, int hd, float scale, int window, int chunked,
                                const float* slopes, const void* gate, int64_t gate_stride, void* part_acc, void* part_ml,
                                hipStream_t stream);
int pae_attn_prefill_biased_bf16(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* k_cache,
                                 const void* v_cache, const int* tiles, int num_tiles, const int* positions,
                                 const int* block_tables, int max_blocks, int bs, int nh, int nkv, int hd, float scale,
                                 int window, int chunked, const float* slopes, const void* gate, int64_t gate_stride,
                                 hipStream_t stream);
// A decode step's layers as one resident kernel (see decode_program.hip).
// A caller builds a list of phases in host memory with the put functions (each returns the bytes of
// LDS a quad of four wavefronts needs for the phase, or a negative code), copies it to the device and
// runs it.  pae_program_max_groups() must have been called once on the device, outside any capture.
struct SkinnyRope;
int pae_program_phase_bytes();
int pae_program_barrier_bytes();
int pae_program_max_rows();
int pae_program_max_groups();
int pae_program_lds_limit();
int pae_program_activation_bytes(int rows, int K, int splits);
int pae_program_put_product(void* phases, int index, int epilogue, void* out, int64_t ldc, const void* A, int64_t lda,
                            const void* W, const void* bias, int b_is_f32, int M, int N, int K, int splits,
                            float* ticket_parts, int* ticket_counters, const float* row_stats, int row_stat_tiles,
                            float row_eps, void* next_rows, int64_t ld_next, const void* next_w, int next_w_is_f32,
                            float* next_stats, const SkinnyRope* rope);
int pae_program_put_product_rope(void* phases, int index, void* q_out, int64_t ldq, const void* A, int64_t lda,
                                 const void* W, const void* bias, int b_is_f32, int M, int K, int nh, int nkv, int hd,
                                 int rot, const float* cos_sin, const int* positions, const int* tok_seq,
                                 const int* block_tables, int max_blocks, int bs, void* k_cache, void* v_cache,
                                 int splits, float* ticket_parts, int* ticket_counters, const float* row_stats,
                                 int row_stat_tiles, float row_eps);
int pae_program_put_attention(void* phases, int index, void* out, int64_t out_stride, const void* q, int64_t q_stride,
                              const void* k_cache, const void* v_cache, const int* dec_work, int num_dec,
                              const int* block_tables, int max_blocks, int bs, int nh, int nkv, int hd, float scale,
                              int window, void* part_acc, void* part_ml);  // two phases: index and index + 1
int pae_program_run(const void* phases, int num_phases, void* barrier, int* host_error, int groups, int quad_lds_bytes,
                    int activation_lds_bytes, int spin_limit, long long* trace, hipStream_t stream);

int pae_sample_chunks(int vocab);
int pae_sample(int* tokens, const float* logits, int64_t ld, const float* temperature, const float* uniform,
               int num_rows, int vocab, float* chunk_max, int* chunk_arg, double* chunk_sum, hipStream_t stream);

// pae_sample without a workspace argument, for callers that cannot allocate device memory (code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
// counterpart in the reference.  The chunk results live in a buffer that is part of the library's
// image on every GPU (16 bytes a slot, PAE_SAMPLE_STATIC_SLOTS slots = 512 KiB, held by each GPU
// the library runs on until the process ends); its device address is looked up once per device, for
// the device that `stream` belongs to (the current device for the null stream), at the first call
// there or by pae_sample_static_prepare() with that device current.  That first lookup asks the
// runtime and must not fall inside a stream capture (it is refused there): prepare, or call once,
// before capturing.  num_rows * pae_sample_chunks(vocab) beyond the slots is refused.  The call
// itself calls no hipMalloc, hipFree or other allocating routine.  Every call on a GPU uses that
// GPU's one buffer: calls that overlap on one GPU (several streams or threads) race, so issue them
// one after the other.  Nothing in the buffer needs clearing between calls: a call writes every
// slot before it reads it.  Same results as pae_sample, bit for bit.
#define PAE_SAMPLE_STATIC_SLOTS 32768
int pae_sample_static_slots();
int pae_sample_static_prepare();
int pae_sample_static(int* tokens, const float* logits, int64_t ld, const float* temperature,
                      const float* uniform, int num_rows, int vocab, hipStream_t stream);
}
