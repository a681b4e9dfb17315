// Host-side launchers of the gfx950 kernels (plain HIP, no torch types: the kernel translation
// units never include torch headers, so each compiles in seconds; torch_bindings.cpp adapts them).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace dli {

void launch_rms_norm(void* out, const void* x, const void* w, float eps, int rows, int H, int64_t x_stride,
                     int64_t out_stride, hipStream_t stream);
void launch_fused_add_rms_norm(void* x, void* residual, const void* w, float eps, int rows, int H, int64_t x_stride,
                               hipStream_t stream);
// act_limit > 0: the clamped gated activation min(g, limit) · sigmoid(1.702 ·) · (clamp(u, ±limit) + 1) instead of silu(g) · u
void launch_silu_and_mul(void* out, const void* x, int rows, int inter, int64_t x_stride, hipStream_t stream, float act_limit = 0.f);
void launch_rms_norm_quant(const void* x, void* residual, const void* w, float eps, int rows, int H, int64_t x_stride, void* q,
                           float* scales, hipStream_t stream);
void launch_quant_rows_fp8(bool silu, const void* x, int64_t x_stride, void* q, int64_t q_stride, float* scales, int rows,
                           int K, hipStream_t stream);

void launch_rope_and_cache(void* qkv, int64_t row_stride, const int* positions, const float* cos_sin,
                           const int* slot_mapping, void* k_cache, void* v_cache, int T, int Hq, int Hkv,
                           bool kv_fp8, float k_scale, float v_scale, const float* kv_scales, hipStream_t stream);
void launch_copy_pages(void* cache, const int* pairs, int n_pairs, int64_t page_bytes, hipStream_t stream);

void launch_paged_decode(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                         const int* block_tables, int max_blocks, const int* seq_lens, void* out, int64_t out_stride,
                         float* part_o, float* part_ml, int num_seqs, int Hq, int Hkv, int num_splits, float scale,
                         bool kv_fp8, float k_scale, float v_scale, const float* kv_scales, hipStream_t stream);
void launch_paged_decode_worklist(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                                  const int* block_tables, int max_blocks, const int* seq_lens, void* out,
                                  int64_t out_stride, float* part_o, float* part_ml, const int* work, const int* red,
                                  const int* counts, int items, int reds, int Hq, int Hkv, float scale, bool kv_fp8,
                                  float k_scale, float v_scale, const float* kv_scales, hipStream_t stream);
void launch_paged_prefill(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                          const int* block_tables, int max_blocks, const int* seq_lens, const int* query_start_loc,
                          const int* tile_seq, const int* tile_q0, int num_tiles, void* out, int64_t out_stride, int Hq,
                          int Hkv, float scale, bool kv_fp8, float k_scale, float v_scale, const float* kv_scales,
                          const int* counts, hipStream_t stream);

void launch_skinny_linear(void* out, int64_t out_stride, const void* x, int64_t x_stride, const void* w, const void* bias,
                          int M, int N, int K, bool swiglu, const float* w_scale, hipStream_t stream);
void launch_moe_skinny(bool down, const void* a, int64_t a_stride, const void* w, int64_t w_expert_stride,
                       const int* sorted_ids, const int* tile_expert, const int* meta, const float* topk_w, int top_k,
                       void* out, int64_t out_stride, int K, int N, int max_tiles, int max_rows, hipStream_t stream);
void launch_gather_sampled(int* input, const int* src, const int64_t* sampled, int n, hipStream_t stream);
void launch_sample(const void* logits, bool logits_fp32, int64_t row_stride, int B, int V, const float* temperature,
                   const float* top_p, const int* top_k, const int64_t* seeds, const int64_t* steps, const float* noise,
                   int64_t* out, hipStream_t stream);

// mixture of experts (moe.hip)
void launch_moe_route(const void* logits, int T, int E, int K, int* ids, float* weights, hipStream_t stream);
void launch_moe_align(const int* ids, int n, int expert_offset, int E_local, int* sorted_ids, int* tile_expert, int* meta,
                      int capacity_rows, int tile_rows, hipStream_t stream);
void launch_grouped_gemm(int epilogue, const void* A, int64_t a_stride, const void* W, int64_t w_expert_stride,
                         const int* sorted_ids, const int* tile_expert, const int* meta, const float* topk_w, int top_k,
                         void* out, int64_t out_stride, int K, int N_out, int max_tiles, int k_splits, int64_t slab_elems,
                         hipStream_t stream, float act_limit = 0.f);
// 256×256×64 tile (gemm256.hip): large-M grouped GEMM and dense GEMM with optional SwiGLU epilogue
void launch_grouped_gemm256(int epilogue, const void* A, int64_t a_stride, const void* W, int64_t w_expert_stride,
                            const int* sorted_ids, const int* tile_expert, const int* meta, const float* topk_w, int top_k,
                            void* out, int64_t out_stride, int K, int N_out, int max_tiles, int k_splits, int64_t slab_elems,
                            hipStream_t stream, float act_limit = 0.f);
void launch_dense_gemm256(bool swiglu, const void* x, int64_t x_stride, const void* W, void* out, int64_t out_stride, int M,
                          int K, int N_out, int k_splits, float* workspace, bool split_tail, hipStream_t stream);
void dense_gemm256_tail_plan(int M, int K, int N_out, bool swiglu, int* tail_tiles, int* tail_slices);
void launch_moe_sum(const void* y, bool y_fp32, int n_slabs, int64_t slab_elems, const int* ids, int expert_offset, int E_local,
                    int top_k, int T, int H, void* out, hipStream_t stream);

// heterogeneous decoder stacks (seqmix.hip): fp32 stream / statistics / state, activations bf16 or fp32 (the *_bf16 flags)
void launch_sm_layer_norm(const float* x, const float* w, const float* b, float eps, int rows, int W, void* out, bool out_bf16,
                          hipStream_t stream);
void launch_sm_ln_shift(const float* x, const float* add, float* xout, const float* w, const float* b, const float* mix,
                        float* state, const int* positions, const int* token_seq, const int* qsl, const int* state_slots,
                        const int* counts, int rows, int seqs, float eps, int W, void* out, bool out_bf16, hipStream_t stream);
void launch_sm_add_ln(float* x, const void* y, bool y_bf16, int64_t y_stride, const float* w1, const float* b1, float mult,
                      const float* w2, const float* b2, float eps, int rows, int W, void* out, bool out_bf16, hipStream_t stream);
void launch_sm_rms_gate(const float* o, int parts, const float* w, float eps, const void* gate, bool gate_bf16, int64_t gate_stride,
                        int rows, int N, void* out, bool out_bf16, int groups, bool silu, hipStream_t stream);
int sm_lightning_parts(int D);
void launch_sm_relu2(const void* x, void* out, int64_t n, bool bf16, hipStream_t stream);
void launch_sm_softcap(const void* x, bool bf16, float* out, float cap, int64_t n, hipStream_t stream);
void launch_sm_qk_norm_cache(void* qkv, bool bf16, int64_t row_stride, const float* qw, const float* kw, float eps,
                             const int* slot_mapping, void* k_cache, void* v_cache, int rows, int H, int G, int D, int Dv,
                             hipStream_t stream);
void launch_sm_latent_prep(void* q, bool bf16, int64_t q_stride, const void* dkv, int64_t dkv_stride, const float* cw, float eps,
                           const int* positions, const double* inv_freq, int rot_dims, const int* slot_mapping, void* cache,
                           int rows, int H, int D, int R, int C, hipStream_t stream);
void launch_sm_token_attention(void* out, int64_t o_ts, int64_t o_hs, const void* q1, int64_t q1_ts, int64_t q1_hs, int D1,
                               const void* q2, int64_t q2_ts, int64_t q2_hs, int D2, const void* kc, int rowk, const void* vc,
                               int rowv, int vhead, int Dv, const int* block_tables, int max_blocks, const int* positions,
                               const int* token_seq, int rows, int H, int G, float scale, int window, const float* temp,
                               const float* r1, const float* r2, bool bf16, int nsplit, float* part, const void* gate, int64_t g_ts, const float* sink,
                               hipStream_t stream);
int sm_token_attention_splits(int rows, int H, int G);
bool launch_sm_head_decode_attention(void* out, int64_t o_ts, int64_t o_hs, const void* q1, int64_t q1_ts, int64_t q1_hs, int D1,
                                     const void* q2, int64_t q2_ts, int64_t q2_hs, int D2, const void* kc, int rowk, const void* vc,
                                     int rowv, int vhead, int Dv, const int* block_tables, int max_blocks, const int* positions,
                                     const int* token_seq, int rows, int H, int G, float scale, int window, const float* temp,
                                     const float* r1, const float* r2, int nsplit, float* part, const void* gate, int64_t g_ts, const float* sink,
                                     hipStream_t stream);
int sm_head_decode_splits(int rows, int H, int G);
bool launch_sm_tile_attention(void* out, int64_t o_ts, int64_t o_hs, const void* q1, int64_t q1_ts, int64_t q1_hs, int D1,
                              const void* q2, int64_t q2_ts, int64_t q2_hs, int D2, const void* kc, int rowk, const void* vc,
                              int rowv, int vhead, int Dv, const int* block_tables, int max_blocks, const int* seq_lens,
                              const int* qsl, const int* tile_seq, const int* tile_q0, int num_tiles, const int* counts, int H,
                              int G, float scale, int window, const float* temp, const float* r1, const float* r2,
                              const void* gate, int64_t g_ts, const float* sink, hipStream_t stream);
void launch_sm_lightning_scan(const void* qkvg, bool bf16, int64_t row_stride, float* state, const int* positions, const int* qsl,
                              const int* state_slots, const int* counts, int seqs, int H, int D, int Dv, const float* decay,
                              float* out, int64_t out_part, const int* tile_seq, const int* tile_q0, int num_tiles, float* ws,
                              bool plain_act, hipStream_t stream);

// custom all-reduce over IPC-mapped peer buffers (custom_all_reduce.hip)
void* ar_alloc(size_t bytes, bool uncached);
void ar_free(void* p);
int ar_ipc_handle(void* p, void* handle_out64);
void* ar_ipc_open(const void* handle64);
size_t ar_signal_bytes();
void* ar_create(int rank, int world, const int64_t* staging, const int64_t* result, const int64_t* signal, size_t max_bytes);
void ar_destroy(void* st);
int ar_ipc_close(void* p);
int ar_max_blocks();
int ar_set_tuning(void* st, int n, const int64_t* thr, const int* algo, const int* blocks, int default_blocks,
                  int64_t one_shot_max_bytes);
int ar_error(void* st);
int ar_error_async(void* st, void* pinned_dst4, hipStream_t stream);
int launch_all_reduce(void* st, const void* in, void* out, int64_t bytes, int algo, int blocks, hipStream_t stream);
int launch_all_reduce_add_norm(void* st, void* residual, const void* weight, float eps, void* out, int T, int H, int blocks,
                               hipStream_t stream);
int launch_all_gather(void* st, const void* in, void* out, int64_t bytes, hipStream_t stream);
int launch_broadcast(void* st, void* buf, int64_t bytes, int root, hipStream_t stream);
// expert-parallel dispatch / combine over the same IPC buffers (custom_all_reduce.hip)
int64_t ep_layout(void* st, int64_t n_cap, int H, int64_t* ids_off, int64_t* wts_off, int64_t* meta_off);
void* ep_result_ptr(void* st);
void* ar_staging_ptr(void* st);
int64_t ep_max_bytes(void* st);
int launch_ep_dispatch(void* st, const void* x, int64_t x_stride, const int* ids, const float* wts, int n, int n_cap, int top_k,
                       int H, int local_experts, int* slot, void* recv_x, int* ids_local, float* w_local, int r_cap,
                       int* recv_total, int blocks, hipStream_t stream);
int launch_ep_combine(void* st, const int* ids, const int* slot, int n, int n_cap, int H, int local_experts, void* y_back, int blocks,
                      hipStream_t stream);

// gated parallel layers (dualmix.hip): same conventions as the seqmix launchers
void launch_dm_rms_scale(const float* x, const float* g1, const float* g2, float eps, int rows, int W, void* h1, void* h2, bool out_bf16,
                         hipStream_t stream);
void launch_dm_shift_mix(const void* h, bool bf16, int64_t h_stride, const float* mu, int S, float* state, const int* positions,
                         const int* token_seq, const int* qsl, const int* state_slots, const int* counts, int T, int seqs, int W,
                         void* out, hipStream_t stream);
void launch_dm_wide_norm_rope_cache(void* qkv, bool bf16, int64_t row_stride, const float* qw, const float* kw, float eps,
                                    const int* positions, const double* freq, float mag, int rot_dims, const int* slot_mapping,
                                    void* k_cache, void* v_cache, int rows, int H, int G, int D, int Dv, hipStream_t stream);
size_t dm_talk_attention_lds(int H, int D);
int dm_talk_attention_max_heads();
int dm_talk_attention_max_out();
void launch_dm_talk_attention(void* out, int64_t o_stride, const void* q, int64_t q_ts, int64_t q_hs, const void* gate, int64_t g_stride,
                              const void* k_cache, const void* v_cache, bool bf16, const int* block_tables, int max_blocks,
                              const int* positions, const int* token_seq, const float* sink, const float* talk, int rows, int H, int G,
                              int D, int Dv, float scale, hipStream_t stream);
void dm_prepare_kernels();
bool launch_dm_talk_tile_attention(void* out, int64_t o_stride, const void* q, int64_t q_ts, int64_t q_hs, const void* gate,
                                   int64_t g_stride, const void* k_cache, const void* v_cache, const int* block_tables, int max_blocks,
                                   const int* seq_lens, const int* qsl, const int* tile_seq, const int* tile_q0, int num_tiles,
                                   const int* counts, const float* sink, const float* talk, int H, int G, int D, int Dv, float scale,
                                   hipStream_t stream);
void launch_dm_decay(const void* a, bool bf16, int64_t a_stride, const void* w2, const float* w0, int rows, int Lr, int C, float* out,
                     hipStream_t stream);
void launch_dm_wkv_scan(const void* rkv, bool bf16, int64_t plane, const float* w, const float* u, float* state, const int* positions,
                        const int* qsl, const int* state_slots, const int* counts, int seqs, int H, int D, float* out,
                        hipStream_t stream);
void launch_dm_group_rms_gate(const float* o, int groups, const float* w, float eps, const void* gate, bool gate_bf16, int64_t g_stride,
                              int rows, int C, void* out, bool out_bf16, hipStream_t stream);
void launch_dm_sigmoid_route(const void* h, bool bf16, int64_t h_stride, const float* router, int router_rows, int E, int K, float scale,
                             int rows, int W, int* ids, float* wts, float* extra, hipStream_t stream);
void launch_dm_experts(const void* h, bool bf16, int64_t h_stride, const int* ids, const float* wts, int K, const void* up,
                       const void* down, int rows, int F, int W, void* act, void* out, int act_kind, int E, float limit,
                       hipStream_t stream);     // act_kind 0: relu², 1: silu-gated, 2: clamped gated (ids outside 0..E-1: identity experts)

// hyper-connected stacks (hypermix.hip): several fp32 copies of the stream, input convolution, retention, gated feed-forwards
void launch_hm_stream_mix_norm(float* x, const void* y, bool y_bf16, int64_t y_stride, const float* mix, const float* out_w,
                               const float* in_w, const float* norm_w, float eps, float w_offset, int rows, int S, int W, void* out,
                               bool out_bf16, bool center, hipStream_t stream);
int hm_max_streams();
int hm_max_taps();
void launch_hm_causal_conv_add(const float* h, const float* w, int taps, float* state, const int* positions, const int* token_seq,
                               const int* qsl, const int* state_slots, const int* counts, int rows, int seqs, int W, void* out,
                               bool out_bf16, hipStream_t stream);
void launch_hm_retention_prep(const void* qkvg, bool bf16, int64_t row_stride, const int* positions, const double* freq, int rot_dims,
                              int rows, int H, int D, int Dv, float k_scale, float* out, hipStream_t stream);
void launch_hm_act_mul(const void* x, bool bf16, int64_t x_stride, int rows, int F, bool silu, void* out, hipStream_t stream);
void launch_hm_softmax_route(const void* h, bool bf16, int64_t h_stride, const float* router, const float* bias, int E, int K, int rows,
                             int W, int* ids, float* wts, bool all, hipStream_t stream);
// gated linear recurrences and gated latent attention (recurmix.hip)
int rm_max_taps();
void launch_rm_causal_conv(const void* x, bool bf16, int64_t x_stride, const float* w, const float* bias, int taps, float* state,
                           const int* positions, const int* token_seq, const int* qsl, const int* state_slots, const int* counts,
                           int rows, int seqs, int C, void* out, bool out_bf16, hipStream_t stream);
void launch_rm_rglru_scan(const void* z, const void* u, const void* y, bool bf16, int64_t y_stride, const float* gate_bias,
                          const float* rate, float* state, const int* positions, const int* qsl, const int* state_slots,
                          const int* counts, int rows, int seqs, int B, int n, void* out, bool out_bf16, const int* tile_seq,
                          const int* tile_q0, int num_tiles, float* ws, hipStream_t stream);
int64_t rm_rglru_ws_floats(int rows, int seqs, int C);
void launch_rm_latent_norm_cache(const void* proj, bool bf16, int64_t p_stride, int Q, const float* qw, const float* cw, float eps,
                                 const int* positions, const double* freq, float mag, int rot_dims, const int* slot_mapping, void* cache,
                                 int rows, int C, int R, void* cq, hipStream_t stream);
void launch_rm_rotate_heads(void* q, bool bf16, int64_t q_stride, const int* positions, const double* freq, float mag, int rot_dims,
                            int rows, int H, int D, int R, hipStream_t stream);
void launch_rm_identity_add(void* out, const void* h, bool bf16, int64_t h_stride, const int* ids, const float* wts, int K, int E,
                            int rows, int W, hipStream_t stream);
void launch_rm_gate_heads(const void* o, const void* gate, bool bf16, int64_t g_stride, int H, int rows, int Dv, void* out,
                          hipStream_t stream);
void launch_dm_relu2_rows(const void* x, bool bf16, int64_t x_stride, int rows, int F, void* out, hipStream_t stream);
void launch_dm_gated_combine(float* x, float mult, const void* p0, const void* p1, float s0, float s1, const void* g1, int64_t g1_stride,
                             const float* b1, const void* ff, const void* shared, const float* sg, const void* g2, int64_t g2_stride,
                             const float* b2, bool bf16, int rows, int W, hipStream_t stream);

}  // namespace dli
