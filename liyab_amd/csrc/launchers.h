// Declarations of the library's launchers, for code that calls them by name from inside the
// library (the replay of a recorded list of launches, replay.hip). Every .hip file that defines
// one includes this header, so that a declaration that does not match its definition is a
// compile error.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "epilogue.h"

extern "C" {

int liyab_fill(void* p, int elem_bytes, uint32_t bits, int64_t n, hipStream_t stream);
int liyab_add_into(float* y, const void* x, int dtype, int64_t n, hipStream_t stream);
int liyab_gather_rows(void* out, int out_dtype, const float* x, const int* rows, int n, int d, hipStream_t stream);
int liyab_scale(float* p, float scale, int64_t n, hipStream_t stream);
int liyab_embed(float* x, const void* tok, const void* pos, int dtype, const int* ids, const int* positions, int n, int d, float scale,
                const int* last_tokens, hipStream_t stream);
int liyab_add_rows(float* x, const void* table, int dtype, const int* rows, int n, int d, hipStream_t stream);
int liyab_kv_write(void* kc, void* vc, const void* src, int dtype, int64_t src_stride, int k_off, int v_off, const int* slots, int n,
                   int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream);
int liyab_layernorm(void* out, int out_dtype, const float* x, const float* w, const float* b, const int* rows, int n, int d, float eps,
                    hipStream_t stream);
int liyab_layernorm_parts(void* out, int out_dtype, const float* planes, int n_parts, int64_t part_stride, int x_rows, const float* w,
                          const float* b, const int* rows, int n, int d, float eps, hipStream_t stream);
int liyab_sum_parts(float* out, int x_rows, int d, const float* planes, int n_parts, int64_t part_stride, hipStream_t stream);
int liyab_gemm_simple(void* out, int out_dtype, int64_t ldo, const void* a, int64_t lda, const void* w, int dtype, const float* bias,
                      float* residual, int64_t ldr, int M, int N, int K, int epi, hipStream_t stream);
int liyab_gemm_mfma(const void* a, int64_t lda, const void* w, int M, int N, int K, int tile, const liyab::EpiParams* epi_in,
                    hipStream_t stream);
int liyab_gemm_mfma_dl(const void* a, int64_t lda, const void* w, int M, int N, int K, int tile, const liyab::EpiParams* epi_in,
                       hipStream_t stream);
int liyab_gemm_mfma_dl_parts(const void* a, int64_t lda, const void* w, int M, int N, int K, int kparts, int tile, float* parts,
                             int64_t part_stride, const float* bias, const float* base, int n_base, int64_t base_stride,
                             hipStream_t stream);
int liyab_gemm_skinny(const void* a, int64_t lda, const void* w, int M, int N, int K, int ksplit, int wide, int mtile,
                      const liyab::EpiParams* epi_in, hipStream_t stream);
int liyab_gemm_skinny_parts(const void* a, int64_t lda, const void* w, int M, int N, int K, int kparts, int ksplit, float* parts,
                            int64_t part_stride, const float* bias, const float* base, int n_base, int64_t base_stride,
                            hipStream_t stream);
int liyab_gemm_att_parts(const float* partials, int n_splits, int n_head, int hd, const void* w, int M, int N, int kparts, float* parts,
                         int64_t part_stride, const float* bias, const float* base, int n_base, int64_t base_stride,
                         hipStream_t stream);
int liyab_gemm_skinny_ln(const float* planes, int n_planes, int64_t plane_stride, const float* ln_weight, const float* ln_bias,
                         float eps, const void* w, int M, int N, int K, int wide, const liyab::EpiParams* epi_in, hipStream_t stream);
int liyab_gemm_skinny_dyt(const float* planes, int n_planes, int64_t plane_stride, const float* weight, const float* bias, const float* alpha,
                          const void* w, int M, int N, int K, int wide, const liyab::EpiParams* epi_in, hipStream_t stream);
int liyab_attention_generic(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc, int dtype,
                            const int* block_tables, int max_blocks, const int* tok_seq, const int* tok_pos, int n, float scale,
                            int window, int n_head, int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream);
int liyab_attention_decode(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc, int dtype,
                           const int* block_tables, int max_blocks, const int* tok_list, const int* tok_seq, const int* tok_pos, int n,
                           float scale, int window, int n_head, int n_kv_head, int hd, int page_size, int n_splits, int chunk,
                           int waves, int rows_are_requests, float* partials, int leave_splits, int num_pages, hipStream_t stream);
int liyab_attention_merge(void* out, int out_dtype, int64_t out_stride, const float* partials, int n, int n_head, int hd, int n_splits,
                          hipStream_t stream);
int liyab_attention_prefill(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc,
                            const int* block_tables, int max_blocks, const int* work, int n_tiles, int tile, int ksplit, float scale,
                            int window, int n_head, int n_kv_head, int hd, int page_size, int num_pages, hipStream_t stream);

int liyab_rmsnorm(void* out, int out_dtype, const float* x, const float* w, const int* rows, int n, int d, float eps, hipStream_t stream);
int liyab_gated_norm_add(float* x, void* cast_out, int cast_dtype, const float* y, int n_sum, const float* gate, int64_t gate_stride,
                         const float* w, float eps, int normalize, int n, int d, float* state, int ring, int n_slots,
                         const int* tok_seq, const int* positions, const int* context_lens, const int* state_slots, const int* n_real,
                         const float* next_w, float next_eps, hipStream_t stream);
int liyab_causal_conv(void* out, void* cast_out, int dtype, const float* x, const float* w, int taps, const float* state, int n_slots,
                      const int* tok_seq, const int* positions, const int* seq_starts, const int* state_slots, int n, int d,
                      hipStream_t stream);
int liyab_keep_rows(float* state, int ring, int n_slots, const float* x, const int* tok_seq, const int* positions,
                    const int* context_lens, const int* state_slots, const int* n_real, int n, int d, hipStream_t stream);
int liyab_latent_store(void* cache, int dtype, const void* src, int64_t src_stride, int col_off, const float* w, float eps,
                       const int* slots, int n, int rank, int page_size, int num_pages, hipStream_t stream);
int liyab_grouped_product(const void* a, int64_t lda, int a_div, int a_group_cols, const void* w0, const void* w1, int dtype, void* out,
                          int out_dtype, int64_t ldo, int out_group_cols, const int* rows_list, const int* tile_group, int n_tiles,
                          int block, int n_groups, const float* row_scale, const void* gate, int gate_dtype, int64_t gate_stride, int M, int N,
                          int K, int act, int out_div, int out_extra, hipStream_t stream);
int liyab_moe_route(const float* logits, int64_t ld, int n, int n_experts, int top, int* ids, float* weights, int mode, int n_groups, int keep,
                    hipStream_t stream);
int liyab_moe_route_align(const float* logits, int64_t ld, int n, int n_experts, int top, int* ids, float* weights, int block,
                          int* rows_list, int* tile_group, int max_tiles, int mode, int n_groups, int keep, hipStream_t stream);
int liyab_moe_align(const int* ids, int n_entries, int n_experts, int block, int* rows_list, int* tile_group, int max_tiles,
                    hipStream_t stream);

int liyab_attention_decode_scored(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc, int dtype,
                                  const int* block_tables, int max_blocks, const int* tok_list, const int* tok_seq, const int* tok_pos, int n,
                                  float scale, int window, int n_head, int n_kv_head, int hd, int page_size, int n_splits, int chunk,
                                  int waves, int rows_are_requests, float* partials, int leave_splits, int num_pages, float softcap,
                                  const float* bias_table, int max_dist, const float* sinks, hipStream_t stream);
int liyab_attention_prefill_scored(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc,
                                   const int* block_tables, int max_blocks, const int* work, int n_tiles, int tile, int ksplit, float scale,
                                   int window, int n_head, int n_kv_head, int hd, int page_size, int num_pages, float softcap,
                                   const float* bias_table, int max_dist, const float* sinks, hipStream_t stream);
int liyab_gate_rows(void* x, int dtype, int64_t ldx, const float* gate, int64_t ldg, int n, int d, float scale, hipStream_t stream);
int liyab_dyt(void* out, int out_dtype, const float* x, const float* w, const float* b, const float* alpha, const int* rows, int n, int d,
              hipStream_t stream);
int liyab_glu_clamped(void* out, int out_dtype, const float* gu, int64_t ld, int n, int ff, float limit, float slope, float shift,
                      hipStream_t stream);
int liyab_activate(void* out, int out_dtype, int64_t ldo, const float* in, int64_t ldi, int op, int n, int d, hipStream_t stream);
int liyab_mean_norm_add(float* x, const float* a, const float* b, const float* wa, const float* wb, float eps, float weight, int n, int d,
                        hipStream_t stream);
int liyab_scan_takes(int rows, int cols);
int liyab_wkv_scan(void* out, int out_dtype, const float* r, const float* k, const float* v, const float* wraw, const float* gate, int64_t ld,
                   const float* w0, const float* u, const float* norm_w, float eps, float* state, int64_t state_stride, int n_slots,
                   const void* keep_src, int keep_dtype, int64_t keep_ld, int keep_width, int64_t keep_off, const int* seq_starts,
                   const int* positions, const int* state_slots, int n_seqs, int H, int D, int seg_tokens, int max_segs, float* seg_state,
                   float* seg_decay, hipStream_t stream);
int liyab_ssd_scan(float* y, int64_t ldy, const float* xbc, int64_t ldx, const float* dtraw, int64_t ldp, const float* dt_bias,
                   const float* A_log, const float* Dskip, float* state, int64_t state_stride, int n_slots, const float* keep_src,
                   int64_t keep_ld, int keep_width, int keep_ring, int64_t keep_off, const int* seq_starts, const int* positions,
                   const int* state_slots, int n_seqs, int H, int P, int N, int G, int seg_tokens, int max_segs, float* seg_state,
                   float* seg_decay, hipStream_t stream);
int liyab_token_shift(void* out, int dtype, const void* h, const float* mu, int n_mix, const float* state, int64_t state_stride, int n_slots,
                      const int* tok_seq, const int* positions, const int* seq_starts, const int* state_slots, int n, int d,
                      hipStream_t stream);
int liyab_conv_act(float* out, int64_t ldo, const float* in, int64_t ldi, const float* w, const float* bias, int taps, const float* state,
                   int64_t state_stride, int n_slots, const int* tok_seq, const int* positions, const int* seq_starts,
                   const int* state_slots, int n, int C, int act, hipStream_t stream);
int liyab_gated_group_norm(void* out, int out_dtype, const float* y, int64_t ldy, const float* z, int64_t ldz, const float* w, float eps,
                           int n, int inner, int groups, hipStream_t stream);
int liyab_qk_prepare(const float* src, int64_t ld, int q_off, int k_off, int v_off, int H, int G, int dk, int dv, int dk_out, int dv_out,
                     void* q_out, void* kc, void* vc, int dtype, const int* slots, int page_size, int num_pages, const float* q_norm, const float* k_norm,
                     float eps, const double* freqs, int rot_dims, float temp_coef, int temp_every, const int* positions, int n,
                     int rot_halves, float rot_mag, float* v_keep, const float* v_first, const float* v_lam, hipStream_t stream);
int liyab_attention_scored(void* out, int64_t out_stride, const void* q, int64_t q_stride, const void* kc, const void* vc, int dtype,
                           const int* block_tables, int max_blocks, const int* tok_seq, const int* tok_pos, int n, float scale,
                           float softcap, int window, const float* bias_table, int max_dist, const float* gate, int64_t gate_stride,
                           int n_head, int n_kv_head, int dk, int dv, int page_size, int num_pages, const float* sinks, hipStream_t stream);

int liyab_norm_shift(void* out, int out_dtype, float* hbuf, const float* x, const float* w, float offset, float eps, const float* cw, int taps,
                     float* state, int64_t state_stride, int n_slots, const int* tok_seq, const int* positions, const int* seq_starts,
                     const int* state_slots, int n, int d, int S, int keep_single, hipStream_t stream);
int liyab_ring_keep(float* state, int64_t state_stride, int ring, int n_slots, const float* src, int64_t ld, int width, const int* tok_seq,
                    const int* positions, const int* context_lens, const int* state_slots, const int* n_real, int n, hipStream_t stream);
int liyab_normed_powers(void* out, int out_dtype, const float* z, int64_t ld, int n, int ff, const float* coef, float eps, hipStream_t stream);
int liyab_softcap(float* p, float cap, int64_t n, hipStream_t stream);
int liyab_delta_takes(int D);
int liyab_delta_prepare(float* prep, const float* k, const float* wraw, const float* araw, int64_t ld, int64_t ldw, const float* w0,
                        const float* a_bias, float decay_scale, float key_eps, int n, int H, int D, hipStream_t stream);
int liyab_delta_scan(float* out, const float* r, const float* k, const float* v, int64_t ld, const float* prep, float* state,
                     int64_t state_stride, int n_slots, const int* seq_starts, const int* positions, const int* state_slots, int n_seqs, int H,
                     int D, int seg_tokens, int max_segs, float* seg_state, float* seg_trans, float* seg_start, hipStream_t stream);
int liyab_delta_single_takes(int D);
int liyab_delta_single(void* out, int out_dtype, const float* r, const float* k, const float* v, const float* araw, const float* gate, int64_t ld,
                       const float* wraw, int64_t ldw, const float* w0, const float* a_bias, const float* norm_w, float eps, float decay_scale,
                       float key_eps, float* state, int64_t state_stride, int n_slots, const int* seq_starts, const int* positions,
                       const int* state_slots, int n_seqs, int H, int D, hipStream_t stream);
int liyab_head_norm_gate(void* out, int out_dtype, const float* o, const float* gate, int64_t ldg, const float* w, float eps, int n, int H, int D,
                         hipStream_t stream);
int liyab_maps_store(const float* src, int64_t ld, const float* cw, int taps, float* state, int64_t state_stride, int n_slots, void* q_out,
                     void* k1, void* k2, void* vc, int dtype, const int* slots, int page_size, int num_pages, const int* tok_seq,
                     const int* positions, const int* seq_starts, const int* state_slots, int n, int H, int G, int D, int V, int P,
                     int keep_single, hipStream_t stream);
int liyab_maps_join(void* out, const void* a1, const void* a2, int64_t lda, int dtype, float lam, float eps, float out_scale, int n, int H, int V,
                    int P, hipStream_t stream);


int liyab_weighted_sum(float* out, const float* a, const float* b, float wa, float wb, int64_t n, hipStream_t stream);
int liyab_lru_conv(float* out, void* split, const float* in, int64_t ldi, const float* w, const float* bias, int taps, const float* state,
                   int64_t state_stride, int n_slots, const int* tok_seq, const int* positions, const int* seq_starts, const int* state_slots,
                   int n, int C, int blocks, hipStream_t stream);
int liyab_lru_coeffs(float* decay, float* gated, const float* z, int64_t ldz, const float* u, const float* br, const float* bi, const float* lam,
                     float rate, int n, int C, int blocks, hipStream_t stream);
int liyab_lru_scan(void* out, int out_dtype, const float* z, int64_t ldz, const float* u, const float* decay, const float* gated, const float* br,
                   const float* bi, const float* lam, float rate, float out_scale, const float* y, int64_t ldy, float* state,
                   int64_t state_stride, int n_slots, const float* x, int64_t ldx, int taps, const int* seq_starts, const int* positions,
                   const int* state_slots, int n_seqs, int C, int blocks, int stretches, hipStream_t stream);

}  // extern "C"
