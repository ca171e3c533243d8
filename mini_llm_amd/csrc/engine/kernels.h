// The C entry points of the kernel libraries (csrc/kernels/*.hip), declared in one place for the
// native engine. Every launcher returns 0, a positive HIP error code, or a negative code when it
// refuses the sizes; none of them allocates.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>

#include "score_shape.h"

extern "C" {

// elementwise.hip
int mllm_embed(const int* ids, const int* pos, const void* wte, const void* wpe, float* x, int T, int D,
               int dtype, const int* src, const int* prev, int n_prev, hipStream_t stream, float scale = 1.f);
int mllm_depth_mix(float* x, float* kept, size_t stride, int n_old, const float* w, size_t n, hipStream_t stream);
int mllm_select_tokens(int* ids, const int* src, const int* prev, int n, int n_prev, hipStream_t stream);
int mllm_reset_state(void* state, size_t slot_bytes, int n_slots, const int* slots, const int* starts, int B,
                     hipStream_t stream);
int mllm_layernorm(const float* x, const int* rows, const float* gamma, const float* beta, void* y, int n,
                   int D, float eps, int out_dtype, hipStream_t stream);
int mllm_kv_append(const void* src, int src_stride, int k_col, int v_col, void* k_pages, void* v_pages,
                   int kv_dim, const int* slots, int T, int dtype, hipStream_t stream);

// gemm_f32.hip, gemm_bf16.hip
int mllm_gemm_f32(const float* A, int lda, const float* W, int ldw, const float* bias, void* C, int ldc,
                  int M, int N, int K, int mode, hipStream_t stream);
int mllm_gemm_bf16_plain(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                         int M, int N, int K, int mode, hipStream_t stream);
int mllm_gemm_bf16(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                   int M, int N, int K, int mode, void* workspace, size_t workspace_bytes, hipStream_t stream);
int mllm_gemm_bf16_kv(const void* A, int lda, const void* W, int ldw, const float* bias, void* C, int ldc,
                      int M, int N, int K, const int* slots, void* k_pages, void* v_pages, int q_cols, int kv_dim,
                      hipStream_t stream);
int mllm_gemm_bf16_merged(const float* split_o, const float* split_ml, int n_splits, int n_heads, int head_dim,
                          const void* W, int ldw, const float* bias, void* C, int ldc, int M, int N, int mode,
                          hipStream_t stream);
int mllm_ln_gemm_bf16(const float* x, int ldx, const int* rows, const float* gamma, const float* beta, float eps,
                      const void* W, int ldw, const float* bias, void* C, int ldc, int M, int N, int K, int mode,
                      hipStream_t stream);
int mllm_rms_gemm_bf16(const float* x, int ldx, const int* rows, const float* gamma, float eps, const void* W, int ldw,
                       const float* bias, void* C, int ldc, int M, int N, int K, int mode, hipStream_t stream);

// attention.hip, attention_decode.hip, attention_prefill.hip
int mllm_paged_attention_generic(const void* q, int q_stride, int q_col, const void* k_pages,
                                 const void* v_pages, int kv_dim, const int* block_tables, int max_blocks,
                                 const int* token_seq, const int* positions, int n_tokens, int n_heads,
                                 int n_kv_heads, int head_dim, int page_size, float scale, int window,
                                 void* out, int out_stride, int dtype, hipStream_t stream);
int mllm_paged_attention_tiled(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                               int kv_dim, const int* block_tables, int max_blocks, const int* cu_q, const int* ctx_len,
                               int n_seqs, int n_tiles_upper, int n_heads, int n_kv_heads, int head_dim, int page_size,
                               float scale, int window, void* out, int out_stride, int dtype, hipStream_t stream,
                               const MllmScoreShape* shape = nullptr, const float* gate = nullptr, int ldg = 0);
int mllm_decode_attention(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                          int kv_dim, const int* block_tables, int max_blocks, const int* token_seq,
                          const int* positions, int n_q, int n_heads, int n_kv_heads, int head_dim,
                          int page_size, float scale, int window, int nsplit, int waves, void* out,
                          int out_stride, float* ws, int* counters, int k_col, int v_col, const int* slots,
                          int partial_out, int dtype, hipStream_t stream, const MllmScoreShape* shape = nullptr,
                          const float* gate = nullptr, int ldg = 0);
int mllm_merge_attention_splits(const float* ws, int n_q, int n_heads, int head_dim, int nsplit, void* out,
                                int out_stride, int dtype, hipStream_t stream);
int mllm_prefill_attention_bf16(const void* q, int q_stride, int q_col, const void* k_pages, const void* v_pages,
                                int kv_dim, const int* block_tables, int max_blocks, const int* cu_q,
                                const int* ctx_len, int n_seqs, int n_tiles_upper, int n_heads, int n_kv_heads,
                                int head_dim, int page_size, float scale, int window, void* out, int out_stride,
                                hipStream_t stream, const MllmScoreShape* shape = nullptr, const float* gate = nullptr, int ldg = 0);

// norm_gate.hip
int mllm_rmsnorm(const float* x, int ldx, const int* rows, const float* w, const float* gate, int ldg, void* y, int ldy,
                 int n, int D, int groups, float eps, int out_dtype, int parts, size_t part_stride, hipStream_t stream);
int mllm_rmsnorm_gate_after(const float* x, int ldx, const float* w, const float* gate, int ldg, void* y, int ldy, int n, int D, int groups,
                            float eps, int out_dtype, int parts, size_t part_stride, hipStream_t stream);
int mllm_softcap(float* x, size_t n, float cap, hipStream_t stream);
int mllm_rmsnorm_add(float* y, const float* w, const float* scale, float mult, float eps, float* x, int n, int D,
                     int clear, hipStream_t stream);
int mllm_rmsnorm_add_many(const float* y, size_t y_stride, const float* w, size_t w_stride, int n_in, float mult, float eps,
                          float* x, int n, int D, hipStream_t stream);
int mllm_glu_clamped(const void* gate, int ldg, const void* up, int ldu, void* out, int ldo, int T, int F, float limit,
                     float alpha, int dtype, hipStream_t stream);
int mllm_fill_zero(void* p, size_t bytes, hipStream_t stream);

// ssm.hip
int mllm_conv_silu(const float* proj, int ld, int col0, int C, const float* w, const float* bias, int taps,
                   const int* token_seq, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                   float* out, int ldo, int T, int B, int write, hipStream_t stream);
int mllm_conv_residual(const float* in, int ld, int C, const float* w, int taps, const int* token_seq, const int* cu_q,
                       const int* state_slots, float* state, size_t slot_floats, void* out, int ldo, int out_dtype, int T,
                       int B, int write, hipStream_t stream, int residual = 1);
int mllm_rmsnorm_conv_single(const float* x, int ldx, const float* wn, float eps, int C, const float* wc, int taps,
                             const int* state_slots, float* state, size_t slot_floats, void* out, int ldo, int out_dtype, int T,
                             int write, hipStream_t stream);
int mllm_stream_conv_single(float* x, int ldx, const float* y, int ldy, const float* wn, float eps, int C, const float* wc, int taps,
                            const int* state_slots, float* state, size_t slot_floats, void* out, int ldo, int out_dtype, int T,
                            int write, hipStream_t stream);
int mllm_ssm_scan(const float* xbc, int ldx, const float* raw_dt, int ldd, const float* dt_bias, const float* A_log,
                  const float* Dskip, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                  size_t scan_offset, float* y, int ldy, size_t part_stride, int T, int B, int max_q_len, int H, int P, int N,
                  int G, int write, float* workspace, hipStream_t stream);
int mllm_ssm_scan_parts(int N);
size_t mllm_ssm_scan_workspace_floats(int T, int B, int H, int P, int N);

// latent_attention.hip
int mllm_latent_prepare(const float* dq, int ld_dq, int Rq, const float* wq, void* cq, int ld_cq, const float* dkv, int ld_dkv,
                        int R, int Dr, const float* wkv, void* pages, void* vt_pages, int page_size, const int* slots,
                        const int* positions, int T, float eps, double base, int rot_dims, int dtype, hipStream_t stream);
int mllm_latent_absorb(const void* q, int ldq, const void* w_uk, int ldw, void* qa, int ldqa, const int* positions, int T, int H,
                       int Dn, int Dr, int R, double base, int rot_dims, int dtype, hipStream_t stream);
int mllm_latent_attention(const void* qa, int ldqa, const void* pages, const int* block_tables, int max_blocks,
                          const int* token_seq, const int* positions, int T, int H, int R, int Dr, int page_size, float scale,
                          int window, void* o_lat, int ldo, int dtype, hipStream_t stream);
int mllm_latent_attention_tiles(const void* qa, const void* k_pages, const void* vt_pages, const int* block_tables,
                                int max_blocks, const int* cu_q, const int* ctx_len, int n_seqs, int n_tiles_upper, int H,
                                int R, int Dr, int page_size, float scale, int window, void* o_lat, int n_rows, int nsplit,
                                float* partials, int single_tokens, hipStream_t stream);
int mllm_latent_expand(const void* o_lat, int ldo, const void* w_uv, int ldw, void* out, int ldout, int T, int H, int Dv, int R,
                       int dtype, hipStream_t stream);

// scored_attention.hip
int mllm_qk_prepare(const float* proj, int ld, int q_col, int k_col, int v_col, int T, int H, int G, int d, int dv,
                    int norm_mode, const float* wq, const float* wk, float eps, int rot_dims, double rot_base,
                    const int* positions, const int* slots, void* q_out, int ldq, void* k_pages, void* v_pages, int dtype,
                    hipStream_t stream, int interleaved = 0);
int mllm_scored_attention_rows(const void* q, int ldq, const void* k_pages, const void* v_pages, const int* block_tables,
                               int max_blocks, const int* token_seq, const int* positions, int n_tokens, int H, int G, int d,
                               int dv, int page_size, float scale, float softcap, int window, int chunk, const float* r1,
                               const float* r2, const float* gate, int ldg, void* out, int ldo, int dtype, hipStream_t stream,
                               int sigmoid_weights = 0, const float* score_bias = nullptr, int gate_per_head = 0,
                               const float* slope = nullptr, const float* sink = nullptr, int keep_first = 0);

int mllm_gate_mul(void* x, int ldx, const float* gate, int ldg, int T, int N, int dtype, hipStream_t stream);

// gated_recurrence.hip
int mllm_hgrn2_parts(int d);
int mllm_hgrn2_scan(const float* proj, int ld, int q_col, int f_col, int v_col, const float* f_bias, const float* lower,
                    const int* cu_q, const int* state_slots, float* state, size_t slot_floats, size_t state_offset, float* y, int ldy,
                    size_t part_stride, int T, int B, int max_q_len, int H, int d, int dv, int write, float* workspace,
                    hipStream_t stream);
int mllm_decay_scan(const float* proj, int ld, int q_col, int k_col, int v_col, const float* decay, int ldd, const float* head_decay,
                    float q_scale, float k_scale, const int* cu_q, const int* state_slots, float* state, size_t slot_floats,
                    size_t state_offset, float* y, int ldy, size_t part_stride, int T, int B, int max_q_len, int H, int d, int dv, int write,
                    float* workspace, hipStream_t stream);
int mllm_rotary_rows(float* proj, int ld, int col0, int T, int n_heads, int d, int rot_dims, double base, const int* positions,
                     hipStream_t stream);
int mllm_lowrank_decay(const float* proj, int ld, int a_col, int rank, const float* w, const float* bias, float tau, float* out, int ldo,
                       int T, int N, hipStream_t stream);
size_t mllm_hgrn2_workspace_floats(int T, int B, int H, int d, int dv);
int mllm_hgrn2_chunk();
int mllm_concat_cast(const float* a, const float* b, int T, int D, void* out, int dtype, hipStream_t stream);
int mllm_glu_act(const void* gu, int ld, int T, int F, int act, void* out, int ldo, int dtype, hipStream_t stream);

// moe.hip
int mllm_moe_act(const void* up, int ldu, const float* logits, int ldl, int E, int ff, int shared_ff, int top, float scale, void* out, int ldo,
                 float* weights_out, int ldw, int T, int dtype, hipStream_t stream);
int mllm_moe_glu_act(const void* up, int ldu, const float* logits, int ldl, int E, int ff, int shared_ff, int top, float scale,
                     int sigmoid_router, float limit, float shared_limit, float alpha, int weight_on_input, int shared_gate, void* out,
                     int ldo, int T, int dtype, hipStream_t stream);

// sampling.hip
int mllm_argmax_chunks(int V);
int mllm_argmax_mirrored(const float* logits, int ld, int n, int V, int* out, int* mirror, float* part_val, int* part_idx,
                hipStream_t stream);
int mllm_sample_mirrored(const float* logits, int ld, int n, int V, const float* temperature, const float* u, int* out, int* mirror,
                hipStream_t stream);

}  // extern "C"
