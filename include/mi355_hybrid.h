/*
 * mi355_hybrid.h -- C-ABI of libmi355_hybrid.so (same conventions as mi355_decode.h: raw device pointers, explicit stream, integer
 * status, mi355_last_error(); nothing allocates or synchronises, every call is graph-capturable).
 */
#ifndef MI355_HYBRID_H
#define MI355_HYBRID_H

#include "mi355_decode.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------------------------------------------------------------
 * libmi355_hybrid.so: dense linears on [out, in] weights and the kernels of the hybrid decoder family (parallel-residual or sequential
 * layers over an fp32 stream; token mixers: paged chunk-masked attention with a softmax sink and position-rotated values, and gated
 * linear recurrences with fp32 state slots; low-rank latent attention over one cached row per token, fixed-decay retention, PolyNorm,
 * sigmoid-gated branches, group-limited mixtures of experts over grouped linears; sliding-window and score-capped attention with
 * per-head output gates and normed queries and keys, a generalized delta-rule recurrence, hashed bigram embedding rows, a weighted
 * average over the depth of the stack).  act_dtype is MI355_ACT_BF16 or MI355_ACT_F32.  Sources: csrc/gemm_dense.hip,
 * csrc/hybrid_ops.hip; the argument conventions are documented at the definitions. */
int mi355_dense_linear(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias, void* y, int32_t ldy,
                       int32_t out_f32, int32_t gated, int32_t act, float softcap, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_embed(const int32_t* ids, int32_t rows, const void* table, int32_t W, int32_t vocab, float* out, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_residual_norm(float* x, const float* a, const float* b, float mult, const int32_t* rows, int32_t n, int32_t W, const void* w1,
                           const void* w2, float weight_offset, float eps, void* h1, void* h2, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_attn_prep(float* qkv, int32_t ld, int32_t koff, int32_t voff, const int32_t* geom, const float* kfreq, const float* vfreq,
                       int32_t v_norm, float eps, const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows,
                       void* kcache, void* vcache, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_attn_rows(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                       const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows, const void* kcache,
                       const void* vcache, void* out, int32_t splits, float* parts, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_attn_tiles(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                        const int32_t* pos, const int32_t* seq, const int32_t* block_table, const int32_t* tile_row0, const int32_t* tile_n,
                        int32_t tiles, const void* kcache, const void* vcache, void* out, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_scan(int32_t mode, const float* proj, int32_t ld, int32_t qo, int32_t ko, int32_t vo, const float* z, int32_t ldz,
                  const void* lower, const void* fbias, float tau, float qscale, int32_t H, int32_t dim, int32_t vdim,
                  const int32_t* row_start, const int32_t* slot, const int32_t* first_pos, int32_t nseq, float* state, float* out,
                  int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_head_norm(const float* o, int32_t rows, int32_t H, int32_t vdim, const void* w, float eps, const float* gate, int32_t ldg,
                       int32_t goff, void* out, int32_t act_dtype, mi355_stream_t stream);
int mi355_dense_grouped(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias, void* y, int32_t ldy,
                        int32_t out_f32, int32_t gated, int32_t act, int32_t act_dtype, int32_t G, int64_t xs, int64_t ys, const int32_t* offs,
                        const int32_t* gather, const int32_t* tiles, int32_t max_tiles, const float* egate, int32_t ldg, int32_t goff,
                        mi355_stream_t stream);
int mi355_hy_gated_residual_norm(float* x, const float* a, const float* b, const float* gate, int32_t ldg, float mult, const int32_t* rows, int32_t n,
                                 int32_t W, const void* w1, const void* w2, float weight_offset, float eps, void* h1, void* h2, const float* moe_y,
                                 const int32_t* moe_place, const float* moe_wts, int32_t moe_top, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_latent_prep(const float* proj, int32_t ld, int32_t doff, const int32_t* geom, const float* freq, float mag, const void* cw, float eps,
                         const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows, void* qn, float* qabs, void* cache,
                         int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_rotary(float* buf, int32_t ld, int32_t rows, int32_t off0, int32_t heads0, int32_t dim0, float scale0, int32_t off1, int32_t heads1,
                    int32_t dim1, float scale1, int32_t rdims, int32_t layout, const float* freq, float mag, const int32_t* pos, mi355_stream_t stream);
int mi355_hy_polynorm(const float* z, int32_t ld, int32_t rows, int32_t n, float ca, float cb, float cc, float ce, float eps, void* out, int32_t ldo,
                      int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_moe_route(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids, float* wts,
                       mi355_stream_t stream);
int mi355_hy_moe_align(const int32_t* ids, int32_t n, int32_t top, int32_t E, int32_t* offs, int32_t* src_row, int32_t* place_of, int32_t* tiles,
                       mi355_stream_t stream);
int mi355_hy_moe_route_align(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids, float* wts,
                             int32_t* offs, int32_t* src_row, int32_t* place_of, int32_t* tiles, mi355_stream_t stream);
int mi355_hy_moe_combine(const float* y, int32_t tokens, int32_t W, const int32_t* place_of, const float* wts, int32_t top, const float* extra, float* out,
                         mi355_stream_t stream);

/* Extended forms (optional steps as arguments; the short forms above call them with the steps switched off). */
int mi355_hy_embed_bigram(const int32_t* ids, int32_t rows, const void* table, int32_t W, int32_t vocab, float* out, const int32_t* prev,
                          const void* bigram, int32_t buckets, int64_t mul_prev, int64_t mul_cur, float* out2, int32_t act_dtype,
                          mi355_stream_t stream);
int mi355_hy_depth_mix_norm(float* x, const float* a, float* stack, int64_t plane, int32_t n, const float* coef, const int32_t* rows,
                            int32_t rows_n, int32_t W, const void* w1, float weight_offset, float eps, void* h1, int32_t act_dtype,
                            mi355_stream_t stream);
int mi355_hy_attn_prep_ex(float* qkv, int32_t ld, int32_t koff, int32_t voff, const int32_t* geom, const float* kfreq, const float* vfreq,
                          int32_t v_norm, float eps, const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows,
                          void* kcache, void* vcache, const void* qnorm, const void* knorm, float mag, float qt_coef, int32_t qt_every,
                          int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_attn_rows_ex(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                          const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows, const void* kcache,
                          const void* vcache, void* out, int32_t splits, float* parts, int32_t window, float softcap, const float* ogate,
                          int32_t ldg, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_attn_tiles_ex(const float* q, int32_t ldq, float scale, const int32_t* geom, int32_t chunk, const float* sink, const float* vfreq,
                           const int32_t* pos, const int32_t* seq, const int32_t* block_table, const int32_t* tile_row0, const int32_t* tile_n,
                           int32_t tiles, const void* kcache, const void* vcache, void* out, int32_t window, float softcap, const float* ogate,
                           int32_t ldg, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_head_norm_ex(const float* o, int32_t rows, int32_t H, int32_t vdim, const void* w, float eps, const float* gate, int32_t ldg,
                          int32_t goff, void* out, int32_t w_heads, int32_t gate_sigmoid, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_delta_scan(const float* proj, int32_t ld, int32_t ro, int32_t ko, int32_t vo, int32_t ao, const float* z, int32_t ldz,
                        float decay_mult, float unit_eps, int32_t H, int32_t dim, int32_t vdim, const int32_t* row_start, const int32_t* slot,
                        const int32_t* first_pos, int32_t nseq, float* state, float* out, mi355_stream_t stream);


/* Further extended forms: an activation with a parameter (act 5: clamped gated form g' sigmoid(1.702 g') (u' + 1)), routers that score by sigmoids, rank
 * groups by their two best experts and scale the weights, a query / key norm over all heads at once, an embedding with a multiplier, and the end of a
 * sublayer whose output is normed before it joins the stream (layer norm or RMS norm), also as the last norm on gathered rows. */
int mi355_dense_linear_ex(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias, void* y, int32_t ldy,
                          int32_t out_f32, int32_t gated, int32_t act, float act_param, float softcap, int32_t act_dtype, mi355_stream_t stream);
int mi355_dense_grouped_ex(const void* x, int32_t ldx, int32_t M, const void* w, int32_t N, int32_t K, const void* bias, void* y, int32_t ldy,
                           int32_t out_f32, int32_t gated, int32_t act, float act_param, int32_t act_dtype, int32_t G, int64_t xs, int64_t ys,
                           const int32_t* offs, const int32_t* gather, const int32_t* tiles, int32_t max_tiles, const float* egate, int32_t ldg,
                           int32_t goff, mi355_stream_t stream);
int mi355_hy_moe_route_ex(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids, float* wts,
                          int32_t score_sigmoid, int32_t group_top, float wscale, mi355_stream_t stream);
int mi355_hy_moe_route_align_ex(const float* z, int32_t ld, int32_t tokens, int32_t E, int32_t groups, int32_t keep, int32_t top, int32_t* ids, float* wts,
                                int32_t* offs, int32_t* src_row, int32_t* place_of, int32_t* tiles, int32_t score_sigmoid, int32_t group_top,
                                float wscale, mi355_stream_t stream);
int mi355_hy_attn_prep_ex2(float* qkv, int32_t ld, int32_t koff, int32_t voff, const int32_t* geom, const float* kfreq, const float* vfreq,
                           int32_t v_norm, float eps, const int32_t* pos, const int32_t* seq, const int32_t* block_table, int32_t rows,
                           void* kcache, void* vcache, const void* qnorm, const void* knorm, int32_t norm_whole, float mag, float qt_coef,
                           int32_t qt_every, int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_embed_scaled(const int32_t* ids, int32_t rows, const void* table, int32_t W, int32_t vocab, float scale, float* out, void* outh,
                          int32_t act_dtype, mi355_stream_t stream);
int mi355_hy_branch_norm(float* x, const float* a, float ca, const float* b, float cb, const float* sh, const float* sg, int32_t ldsg,
                         const float* moe_y, const int32_t* moe_place, const float* moe_wts, int32_t moe_top, const int32_t* self_rows, int32_t n,
                         int32_t W, const void* w, int32_t center, float eps, void* h, int32_t act_dtype, mi355_stream_t stream);

/* The chunked form of the fixed-decay recurrence (long prompt portions): a plan of chunks, mi355_hy_scan over the chunks from zero states, the prefix over a
 * sequence's chunks, and mi355_hy_scan in mode 6 / 7 adding what the chunk-start states contribute. */
int mi355_hy_chunk_plan(const int32_t* row_start, int32_t nseq, int32_t C, int32_t max_chunks, int32_t* cs, int32_t* sc, int32_t* ids, int32_t* zeros,
                        int32_t* ones, mi355_stream_t stream);
int mi355_hy_chunk_prefix(const int32_t* cs, const int32_t* sc, const int32_t* slot, const int32_t* first_pos, int32_t nseq, const float* decay, int32_t H,
                          int32_t per_head, float* chunk_state, float* state, mi355_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MI355_HYBRID_H */
