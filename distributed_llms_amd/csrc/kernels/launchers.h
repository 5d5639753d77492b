// Host-side launcher declarations (C++ ABI, pointers as uintptr_t, stream as uintptr_t).
// Every launcher validates the shapes its grid assumes before launching.
#pragma once
#include <stdint.h>
#include <stdexcept>
#include <string>

namespace dllm {

void rms_norm(uintptr_t y, uintptr_t x, uintptr_t residual, uintptr_t w, int rows, int hidden, float eps,
              uintptr_t stream);
void rms_norm_q8(uintptr_t y, uintptr_t x, uintptr_t residual, uintptr_t w, int rows, int hidden, float eps,
                 uintptr_t q8, uintptr_t qs, uintptr_t stream);
void splitk_add_rms_norm_q8(uintptr_t y, uintptr_t residual, uintptr_t ws, int S, int M, int N, uintptr_t w,
                            float eps, uintptr_t q8, uintptr_t qs, uintptr_t stream);
void embedding(uintptr_t out, uintptr_t ids, uintptr_t table, int tokens, int hidden, int vocab,
               uintptr_t stream);
void rope_cache_append(uintptr_t q_out, uintptr_t qkv, uintptr_t positions, uintptr_t cos_sin,
                       uintptr_t k_cache, uintptr_t v_cache, uintptr_t slots, int tokens, int hq, int hkv,
                       int d, int bs, int v_groups, uintptr_t stream);
void silu_mul(uintptr_t out, uintptr_t gu, int tokens, int inter, uintptr_t stream);
void add_inplace(uintptr_t a, uintptr_t b, long n, uintptr_t stream);
void argmax(uintptr_t out, uintptr_t logits, int rows, int vocab, long row_stride, uintptr_t stream);

void splitk_add_rms_norm(uintptr_t y, uintptr_t residual, uintptr_t ws, int S, int M, int N, uintptr_t w, float eps,
                         uintptr_t stream);
void splitk_reduce(uintptr_t out, uintptr_t ws, uintptr_t bias, int S, int M, int N, uintptr_t stream);
void splitk_reduce_ex(uintptr_t out, uintptr_t ws, uintptr_t bias, int S, int M, int N, int swiglu,
                      uintptr_t stream);
int gemm_wide(uintptr_t c, uintptr_t a, uintptr_t b, uintptr_t ws, long ws_floats, int M, int N, int K, int splits,
              int mode, int variant, uintptr_t stream);
int gemm_wide_fp8(uintptr_t c, uintptr_t a, uintptr_t a_scale, uintptr_t b, uintptr_t b_scale, uintptr_t ws,
                  long ws_floats, int M, int N, int K, int splits, int mode, int variant, uintptr_t stream);
void quant_fp8_rows(uintptr_t q, uintptr_t scale, uintptr_t x, int M, int K, uintptr_t stream);
int gemm_pp(uintptr_t c, uintptr_t a, uintptr_t b, uintptr_t ws, long ws_floats, int M, int N, int K, int splits,
            int mode, int variant, uintptr_t stream);
void gemm_pp_moe(uintptr_t y, uintptr_t x, uintptr_t gather, uintptr_t w, uintptr_t counts, uintptr_t offsets, int E,
                 int N, int K, int xrows, int slots, int mode, uintptr_t stream);
void gemm_pf(uintptr_t c, uintptr_t a, uintptr_t b, int M, int N, int K, int mode, int variant, uintptr_t stream);
int gemm_sq(uintptr_t c, uintptr_t a, uintptr_t b, uintptr_t ws, long ws_floats, int M, int N, int K, int splits,
            int mode, int variant, uintptr_t stream);

void moe_route(uintptr_t logits, int T, int E, int k, uintptr_t topk_w, uintptr_t topk_ids, uintptr_t counts,
               uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, uintptr_t stream);
void moe_grouped_gemm(uintptr_t y, uintptr_t x, uintptr_t gather, uintptr_t w, uintptr_t counts, uintptr_t offsets,
                      int E, int N, int K, int mode, int rows_hint, int variant, uintptr_t stream);
void moe_router_route(uintptr_t x, uintptr_t w, int T, int H, int E, int k, uintptr_t topk_w, uintptr_t topk_ids,
                      uintptr_t counts, uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, uintptr_t stream);
void moe_wide_gemm(uintptr_t y, uintptr_t x, uintptr_t gather, uintptr_t w, uintptr_t counts, uintptr_t offsets,
                   int E, int N, int K, int mode, uintptr_t stream);
void moe_wide_gemm_fp8(uintptr_t y, uintptr_t x, uintptr_t gather, uintptr_t w, uintptr_t counts, uintptr_t offsets,
                       int E, int N, int K, int mode, uintptr_t sa, uintptr_t wscale, uintptr_t stream);
void moe_combine(uintptr_t out, uintptr_t ysorted, uintptr_t topk_w, uintptr_t inv, int T, int H, int k,
                 uintptr_t stream);

void paged_attention_decode(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache,
                            uintptr_t block_tables, uintptr_t seq_lens, uintptr_t part_o, uintptr_t part_ml,
                            int batch, int hq, int hkv, int d, int block_size, int max_blocks, int num_splits,
                            int split_len, float scale, uintptr_t stream);
void paged_attention_decode_rope(uintptr_t out, uintptr_t qkv, uintptr_t positions, uintptr_t cos_sin, uintptr_t slots,
                                 uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables, uintptr_t seq_lens,
                                 uintptr_t part_o, uintptr_t part_ml, int batch, int hq, int hkv, int d,
                                 int block_size, int max_blocks, int num_splits, int split_len, float scale,
                                 uintptr_t qkv_part, int qkv_nparts, long qkv_slab, uintptr_t stream);
void paged_attention_prefill(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache,
                             uintptr_t block_tables, uintptr_t cu_seqlens_q, uintptr_t seq_lens, int batch,
                             int hq, int hkv, int d, int block_size, int max_blocks, int max_q_len, float scale,
                             int version, uintptr_t positions, uintptr_t cos_sin, int q_stride, uintptr_t stream);

// ---- layer-list models with per-sequence state (seqmix.hip, attention_window.hip); f32: activations
// are float (else bf16)
void sm_embed_f32(uintptr_t out, uintptr_t ids, uintptr_t table, int tokens, int width, int vocab, int f32,
                  uintptr_t stream);
void sm_embed_norm(uintptr_t x, uintptr_t h, uintptr_t ids, uintptr_t table, uintptr_t w, int tokens, int width,
                   int vocab, float eps, float offset, float scale, uintptr_t pos_table, uintptr_t positions,
                   int max_pos, int f32, uintptr_t stream);
void sm_stream_enter(uintptr_t x, uintptr_t x0, uintptr_t vec, int rows, int width, int f32, uintptr_t stream);
void sm_mix_add(uintptr_t x, uintptr_t o, uintptr_t w1, uintptr_t o2, uintptr_t w2, uintptr_t w_next, uintptr_t h,
                int rows, int width, float eps, float coef, int f32, uintptr_t stream);
void sm_token_shift(uintptr_t y, uintptr_t h, uintptr_t w, uintptr_t state, uintptr_t cu, uintptr_t positions,
                    uintptr_t tok_seq, uintptr_t slots, int tokens, int width, int f32, uintptr_t stream);
void sm_pool_blocks(uintptr_t k_cache, uintptr_t v_cache, uintptr_t kp_cache, uintptr_t vp_cache, uintptr_t block_tables,
                    int max_blocks, uintptr_t cu, uintptr_t positions, int seqs, int max_q_len, int G, int D, int Dv,
                    int bs, int pb, int pool, int f32, uintptr_t stream);
void la_scan(uintptr_t o, uintptr_t proj, long ld, int qcol, int kcol, int vcol, uintptr_t decay, uintptr_t z,
             uintptr_t z_bias, float inv_tau, float q_scale, int silu, uintptr_t state, uintptr_t cu, uintptr_t positions,
             uintptr_t slots, int seqs, int max_q_len, int H, int D, int Dv, int f32, uintptr_t stream);
void sm_rms_norm(uintptr_t y, uintptr_t x, uintptr_t w, int rows, int width, float eps, float offset, int f32,
                 uintptr_t stream);
void sm_post_norm_add(uintptr_t x, uintptr_t o, uintptr_t bias, uintptr_t w_post, uintptr_t w_next, uintptr_t h,
                      int rows, int width, float eps, float mult, float offset, uintptr_t o2, float s1, float s2,
                      int f32, uintptr_t stream);
void sm_causal_conv(uintptr_t y, uintptr_t u, long stride, uintptr_t w, uintptr_t bias, uintptr_t in_bias,
                    uintptr_t state, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, uintptr_t slots,
                    int tokens, int seqs, int C, int taps, int f32, int out_f32, int act, uintptr_t stream);
void sm_conv_tail(uintptr_t state, uintptr_t u, long stride, uintptr_t cu, uintptr_t positions, uintptr_t slots, int seqs,
                  int C, int taps, int f32, uintptr_t stream);
void sm_rglru_gates(uintptr_t a, uintptr_t g, uintptr_t u, uintptr_t ra_t, uintptr_t ra_b, uintptr_t ri_t,
                    uintptr_t ri_b, uintptr_t lam, int tokens, int nb, int bw, float scale, int f32,
                    uintptr_t stream);
void sm_rglru_scan(uintptr_t out, uintptr_t a, uintptr_t g, uintptr_t y_raw, long y_stride, uintptr_t y_bias,
                   uintptr_t state, uintptr_t cu, uintptr_t positions, uintptr_t slots, int seqs, int C, int max_q_len,
                   uintptr_t ab, int f32, uintptr_t stream);
void sm_clipped_glu(uintptr_t out, uintptr_t gu, uintptr_t bias, int tokens, int F, float limit, float alpha, int f32,
                    uintptr_t stream);
void sm_softcap(uintptr_t out, uintptr_t x, long n, float cap, int f32, uintptr_t stream);
void sm_attn_prep(uintptr_t q_out, uintptr_t qkv, uintptr_t conv_w, uintptr_t state, uintptr_t q_norm,
                  uintptr_t k_norm, uintptr_t freqs, int nrot, float mag, float eps, uintptr_t k_cache,
                  uintptr_t v_cache, uintptr_t slot_mapping, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq,
                  uintptr_t slots, int tokens, int seqs, int H, int G, int D, int Dv, int taps, int bs, int f32,
                  uintptr_t stream);
void sm_rownorm_rope(uintptr_t q_out, uintptr_t qkv, long ld, int col0, uintptr_t q_norm, uintptr_t k_norm,
                     uintptr_t freqs, int nrot, float eps, uintptr_t k_cache, uintptr_t v_cache, uintptr_t slot_mapping,
                     uintptr_t positions, int tokens, int H, int G, int D, int Dv, int bs, float mag, int v_from_k,
                     int f32, uintptr_t stream);
void sm_window_attn_decode(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                           int max_blocks, uintptr_t positions, uintptr_t tok_seq, int rows, int H, int G, int D,
                           int Dv, int bs, int window, int chunk, float scale, uintptr_t sinks, int splits, uintptr_t ws,
                           float softcap, uintptr_t kp, uintptr_t vp, int pool, int pbs, int f32, uintptr_t stream);
void sm_window_attn_prefill(uintptr_t out, uintptr_t q, uintptr_t k_cache, uintptr_t v_cache, uintptr_t block_tables,
                            int max_blocks, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, int seq0, int seqs,
                            int tokens, int max_q_len, int H, int G, int D, int Dv, int bs, int window, int chunk,
                            float scale, uintptr_t sinks, float softcap, uintptr_t kp, uintptr_t vp, int pool, int pbs,
                            int f32, uintptr_t stream);
// latent attention input stage and parallel layers on a float32 stream (latent.hip)
void lat_prep(uintptr_t cq, uintptr_t down, long ld, int q_off, int q_rank, uintptr_t qn_w, int c_off, int rank,
              uintptr_t cn_w, int r_off, int rot_dim, uintptr_t freqs, int nfreq, uintptr_t positions,
              uintptr_t slot_mapping, uintptr_t k_cache, uintptr_t v_cache, int bs, float eps, int tokens, int f32,
              uintptr_t stream);
void lat_q_pack(uintptr_t out, uintptr_t qa, uintptr_t q, int tokens, int H, int rank, int dim, int rot_dim,
                uintptr_t freqs, int nfreq, uintptr_t positions, int f32, uintptr_t stream);
void lat_q_fold(uintptr_t out, uintptr_t q, uintptr_t wuk, int tokens, int H, int rank, int dim, int rot_dim,
                uintptr_t freqs, int nfreq, uintptr_t positions, int f32, uintptr_t stream);
void lat_v_unfold(uintptr_t out, uintptr_t o, uintptr_t wuv_t, uintptr_t gate, long ld, int tokens, int H, int rank,
                  int vdim, int f32, uintptr_t stream);
void lat_head_gate(uintptr_t out, uintptr_t o, uintptr_t gate, long ld, int tokens, int H, int vdim, int f32,
                   uintptr_t stream);
void par_add(uintptr_t x, uintptr_t a, uintptr_t b, uintptr_t x_rounded, long n, int f32, uintptr_t stream);
void stream_cat(uintptr_t out, uintptr_t x, uintptr_t x0, int rows, int width, int f32, uintptr_t stream);
void stream_set(uintptr_t x, uintptr_t a, long n, int f32, uintptr_t stream);
void silu_glu(uintptr_t out, uintptr_t gu, int tokens, int F, int f32, uintptr_t stream);
void side_gate(uintptr_t g, uintptr_t z, uintptr_t table, uintptr_t ids, int tokens, int vocab, int total, int off,
               int dim, int f32, uintptr_t stream);
// grouped-choice router, squared ReLU and the weighted sum with a gated shared expert (moe.hip)
void moe_route_groups(uintptr_t logits, long ld, uintptr_t correction, int T, int E, int k, int groups, int keep,
                      float scale, int softmax_top, uintptr_t topk_w, uintptr_t topk_ids, uintptr_t counts,
                      uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, uintptr_t stream);
void moe_router_groups(uintptr_t x, uintptr_t w, int K, int rows, uintptr_t logits, uintptr_t correction, int T, int E,
                       int k, int groups, int keep, float scale, int softmax_top, uintptr_t topk_w, uintptr_t topk_ids,
                       uintptr_t counts, uintptr_t offsets, uintptr_t sorted_tok, uintptr_t inv, int f32,
                       uintptr_t stream);
void relu_sq(uintptr_t y, long n, int f32, uintptr_t stream);
// gated delta rule (delta.hip): everything float32 but the gate, the norm weight and the normed output
void dr_prep(uintptr_t u, long ld, uintptr_t ab, long ldab, int bcol, uintptr_t a_log, uintptr_t dt_bias, uintptr_t bd,
             int tokens, int H, int G, int dim, float qscale, float unit_eps, int f32, uintptr_t stream);
void dr_conv_prep(uintptr_t u, uintptr_t bd, uintptr_t x, long ld, int col0, int bcol, uintptr_t w, uintptr_t state,
                  uintptr_t a_log, uintptr_t dt_bias, uintptr_t cu, uintptr_t positions, uintptr_t tok_seq, uintptr_t slots,
                  int tokens, int H, int G, int dim, int vdim, int taps, float qscale, float unit_eps, int f32,
                  uintptr_t stream);
void dr_scan(uintptr_t o, uintptr_t u, long ld, uintptr_t bd, uintptr_t state, uintptr_t cu, uintptr_t positions,
             uintptr_t slots, int seqs, int max_q_len, int H, int G, int dim, int vdim, uintptr_t stream);
void dr_out_norm(uintptr_t y, long ldy, uintptr_t o, uintptr_t gate, long ldg, int gcol, uintptr_t w, int tokens, int H,
                 int vdim, float eps, float out_scale, int gate_sig, int f32, uintptr_t stream);
void moe_combine_gated(uintptr_t out, uintptr_t ysorted, uintptr_t topk_w, uintptr_t inv, uintptr_t shared,
                       uintptr_t gate_logits, long gate_ld, int T, int H, int k, int f32, uintptr_t stream);

long p2p_inbox_bytes(long chunk, int nslots);
void p2p_standin(uintptr_t src, uintptr_t s_inbox, long s_bytes, uint64_t s_seq0, uintptr_t dst, uintptr_t r_inbox,
                 long r_bytes, uint64_t r_seq0, long chunk, int nslots, int channels, uintptr_t abort_word,
                 double timeout_s, uintptr_t err, int lds_bytes, uintptr_t stream);
uintptr_t p2p_host_words(int n);
void p2p_host_words_free(uintptr_t p);

}  // namespace dllm
