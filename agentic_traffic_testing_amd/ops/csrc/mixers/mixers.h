// Launchers of the sequence-mixer kernel library (raw pointers, current stream); return 0 or a
// hipError_t.  dtype: 0 = bf16 activations, 2 = fp32 activations.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

extern "C" {
int mixk_embed_pair(float* out, const void* table, const void* pair_table, const int* ids,
                    const int* positions, const int* seq_qstart, const int* seq_slot,
                    int* prev_token, int T, int S, int W, int64_t mul_prev, int64_t mul_cur,
                    int64_t buckets, int dtype, hipStream_t st);
int mixk_rms_norm_f32(void* out, const float* x, const void* w, int T, int W, float eps,
                      int one_plus, int dtype, hipStream_t st);
int mixk_relu_sq(void* out, const void* x, int T, int N, int64_t x_stride, int dtype,
                 hipStream_t st);
int mixk_residual_add(float* x, const void* a, float sa, const void* b, float sb, const void* c,
                      int64_t n, int dtype, hipStream_t st);
int mixk_add_norm(void* h, float* x, const void* a, float sa, const void* b, float sb,
                  const void* c, const void* w, int T, int W, float eps, int one_plus, int dtype,
                  hipStream_t st);
int mixk_gated_rms_norm(void* out, const float* o, const void* gate, int64_t gate_stride,
                        const void* w, int T, int H, int dv, float eps, int act, int dtype,
                        hipStream_t st);
int mixk_qk_norm_rope_cache(void* q_out, const void* qx, int64_t q_stride, const void* kx,
                            int64_t k_stride, const void* vx, int64_t v_stride, const void* q_norm,
                            const void* k_norm, float eps, const int* positions,
                            const int* slot_mapping, const float* cos_sin, int n_freq,
                            void* k_cache, void* v_cache, int T, int H, int G, int dim, int vdim,
                            int block_size, int half, int norm_last, const float* row_inv,
                            int dtype, hipStream_t st);
int mixk_rotary_table(float* out, const int* positions, const float* inv_freq, int T, int n_freq,
                      hipStream_t st);
int mixk_sink_attention(void* out, const void* q, const void* k_cache, const void* v_cache,
                        const int* block_tables, int bt_width, const int* seq_kvlen,
                        const int* seq_qstart, const int* tile_seq, const int* tile_qoff,
                        int num_tiles, int num_decode, int max_decode_kv, float* part,
                        int max_parts, int H, int G, int dim, int vdim, int block_size,
                        float scale, int sink, const float* sink_val, int window, int use_mfma,
                        int dtype, hipStream_t st);
int mixk_short_conv_silu(void* out, const void* x, int64_t x_stride, const void* w,
                         const void* bias, void* conv_state, const int* positions, const int* seq_qstart,
                         const int* seq_slot, int T, int S, int C, int taps, int dtype,
                         hipStream_t st);
int mixk_gated_delta_rule(float* out, const void* qkv, const void* beta, int64_t beta_stride,
                          const void* decay, int64_t decay_stride, int per_channel,
                          const float* a_log, const float* dt_bias, float* state,
                          const int* positions, const int* seq_qstart, const int* seq_slot, int S,
                          int H, int G, int dim, int vdim, int dtype, hipStream_t st);
int mixk_embed_scale(float* out, const void* table, const int* ids, int T, int W, int vocab,
                     float scale, int copies, int dtype, hipStream_t st);
int mixk_rms_norm_rows(void* out, const void* x, int64_t x_stride, const void* w, int T, int N,
                       float eps, int dtype, hipStream_t st);
int mixk_xielu_bias(void* out, const void* x, int64_t x_stride, const void* bias, int T, int N,
                    float ap, float aq, int dtype, hipStream_t st);
int mixk_group_rms_norm(void* out, const float* y, const void* gate, int64_t gate_stride,
                        const void* w, int T, int n_groups, int gs, float eps, int w_full,
                        int dtype, hipStream_t st);
int mixk_head_gate(void* out, const void* o, const void* gate, int64_t gate_stride, int T, int H,
                   int dv, int dtype, hipStream_t st);
int mixk_latent_rope_cache(void* q_out, const void* q_lat, const void* qx, const void* kvx,
                           int64_t kv_stride, const void* c_norm, float eps,
                           const int* slot_mapping, const float* cos_sin, int n_freq,
                           void* k_cache, void* v_cache, void* c_out, int T, int H, int qdim,
                           int rank, int rot, int block_size, int dtype, hipStream_t st);
int mixk_gated_linear_scan(float* out, float* state, const void* q, int64_t q_stride,
                           const void* k, int64_t k_stride, const void* v, int64_t v_stride,
                           const void* dt, int64_t dt_stride, const float* p0, const float* p1,
                           const float* p2, const int* positions, const int* seq_qstart,
                           const int* seq_slot, int S, int H, int G, int dk, int dv, int mode,
                           int dtype, hipStream_t st);
int mixk_hyper_update_norm(void* out, int out_f32, float* xs, const void* y, const float* mix,
                           const float* w_out, const float* w_in, const void* w, int T, int ns,
                           int W, float eps, int dtype, hipStream_t st);
int mixk_token_shift(void* out, const float* n, const float* mu, float* state,
                     const int* positions, const int* seq_qstart, const int* seq_slot, int T,
                     int S, int W, int dtype, hipStream_t st);
int mixk_gate_mul(void* out, const void* a, int64_t a_stride, const void* gate,
                  int64_t gate_stride, int T, int N, int act, int dtype, hipStream_t st);
int mixk_gelu(void* out, const void* x, int64_t x_stride, int T, int N, int tanh_form, int dtype,
              hipStream_t st);
int mixk_mingru_scan(void* out, float* state, const void* z, int64_t z_stride, const void* x,
                     int64_t x_stride, const void* g, int64_t g_stride, const int* positions,
                     const int* seq_qstart, const int* seq_slot, int S, int C, int few_rows,
                     int dtype, hipStream_t st);
int mixk_clamped_glu(void* out, const void* gu, const float* wts, int R, int ff, float limit,
                     float alpha, int dtype, hipStream_t st);
int mixk_pair_sum(void* out, const void* y, int y_f32, int T, int top, int W, int dtype,
                  hipStream_t st);
int mixk_moe_route(int* idx, float* wts, const float* logits, const float* correction, int T,
                   int E, int top, int softmax, int groups, int keep, int renorm, hipStream_t st);
int mixk_moe_experts(void* y, void* act, int* plan, const void* h, const int* idx,
                     const float* wts, const void* w_gate, const void* w_up, const void* w_down,
                     int T, int top, int E, int ff, int W, int64_t gu_estride, int max_tiles,
                     int tile_rows, int split, float limit,
                     float alpha, int glu, int dtype, hipStream_t st);
int mixk_moe_combine(void* out, const void* y, int y_f32, const int* idx, const float* wts,
                     const void* h, const void* addend, int T, int top, int split, int E, int W,
                     int dtype, hipStream_t st);
int mixk_norm_add_norm(void* h, float* x, const void* y, const void* w_post, const void* w_next,
                       int T, int W, float eps, int layer, int dtype, hipStream_t st);
int mixk_proj_inv_rms(float* out, const void* qx, int64_t q_stride, int nq, const void* kx,
                      int64_t k_stride, int nk, int T, float eps, int dtype, hipStream_t st);
int mixk_scale_softcap(float* out, const void* x, int64_t n, float scale, float cap, int dtype,
                       hipStream_t st);
}
