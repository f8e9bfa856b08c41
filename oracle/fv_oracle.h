/*
 * CPU restatement of fastvideo-rs's host-math SDPA / block-causal / VSA path.
 *
 * TEST INFRASTRUCTURE ONLY. This library is the parity checker and the timed
 * CPU baseline; nothing in the shipped HIP path may link, load or call it.
 * Every function cites the reference file:line (relative to the reference
 * checkout, crates/fastvideo-cudarc/src = C/, crates/fastvideo-gpucheck/src =
 * G/, crates/fastvideo-models/src = M/) whose arithmetic it follows.
 *
 * How each function is pinned (tests/test_oracle_*.py):
 *   fvo_bf16_*            closed form + torch's .to(bfloat16) on all edge classes
 *   fvo_matmul/softmax/sdpa_composed
 *                         closed-form-input vectors of C/rt/sdpa.rs:522-542,
 *                         softmax rows sum to 1, vs the f64 formula (<= 1e-6),
 *                         vs torch float64 SDPA, scale sensitivity, row-sampled
 *                         == full bit for bit
 *   fvo_sdpa_f64          vs torch float64 softmax(QK^T)V, brute force
 *   fvo_block_causal_*    known answers C/rt/attn.rs:883-930, M/wan/family.rs:146-191
 *   fvo_vdn_window_*      hand-counted visible sets for the reference's two window forms
 *                         (chunk 5 / radius 1: 10-15 frames, docs/ports/vdn-h3.md:103-105; the
 *                         centred window of G/kernels.rs:2860-2868), anchors and global rows
 *                         dense both ways, symmetry of the anchor rule, brute-force frame maths
 *   fvo_tile_plan/topk_for known answers C/rt/vsa.rs:480-530
 *   fvo_vsa_attention_host all-tiles + zero gate == dense (2e-5), gate tests,
 *                         C/rt/vsa.rs:534-696
 *   fvo_topk_*            brute-force sort on small n, ties, -0.0, both orders
 *   fvo_vsa_tile_mean     closed form on constant/linear inputs
 *   fvo_vsa_combine       f32 form vs numpy mul-then-add; round16 form vs torch's own bf16
 *                         multiply and add on CPU tensors, zero gate == bf16(sparse), padding
 *                         slots leave `out` untouched
 *   fvo_shard_ranges      known answers C/rt/sp.rs:66-84
 *   fvo_qk_norm_rope_bhsd / fvo_wan_qk_norm_rope16
 *                         the two against each other within 0.03 on the closed-form
 *                         inputs of C/wan/fuse.rs:627-663; no-rope == x*inv*w by hand;
 *                         RMS of the normalised row == 1 for w == 1; the rotation keeps
 *                         each pair's norm; rope with angle 0 == no rope
 *   fvo_split_heads_bhsd / fvo_merge_heads
 *                         brute-force index formula, merge(split(x)) == x
 */
#ifndef FV_ORACLE_H
#define FV_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* C/rt/kernels/core.cu:6-15, C/rt/quant.rs:60-62 */
uint16_t fvo_bf16_rne_bits(float x);
float fvo_bf16_round(float x);
void fvo_quantize_bf16(const float* x, float* y, size_t n);
void fvo_to_bf16_bits(const float* x, uint16_t* y, size_t n);
void fvo_from_bf16_bits(const uint16_t* x, float* y, size_t n);

/* C/rt/tensor.rs:1683-1702 — batched host matmul, i-t-j order, f32, no FMA.
 * a [batch,m,k] b [batch,k,n] out [batch,m,n]; threads split batch only. */
void fvo_matmul(const float* a, const float* b, float* out, size_t batch, size_t m,
                size_t k, size_t n, int threads);
/* C/rt/ops.rs:2178-2193 */
void fvo_softmax_last(const float* x, float* out, size_t rows, size_t width);

/* C/rt/sdpa.rs:328-342 — softmax(scale * q k^T + mask) v with the host tensor
 * ops above. mask is NULL or an additive [sq, sk] tensor broadcast over bh.
 * q [bh,sq,d], k/v [bh,sk,d], out [bh,sq,d]. Materialises one head's scores. */
void fvo_sdpa_composed(const float* q, const float* k, const float* v, const float* mask,
                       float* out, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                       int threads);
/* Same arithmetic for a subset of query rows (rows are independent in the
 * reference's loops, so each sampled row is bit-identical to a full run).
 * rows[nrows] index the query axis; out [bh, nrows, d]. mask_bc: NULL or
 * {block_tokens, window, sink} applied as the additive 0 / -1e9 mask of
 * C/rt/attn.rs:456-466. */
void fvo_sdpa_composed_rows(const float* q, const float* k, const float* v,
                            const int64_t* mask_bc, const int64_t* rows, size_t nrows,
                            float* out, size_t bh, size_t sq, size_t sk, size_t d,
                            float scale, int threads);

/* G/kernels_attn.rs:64-106 and G/kernels_wan.rs:29-72 — f64 checker.
 * mask_bc NULL = dense; masked keys get -inf scores. */
void fvo_sdpa_f64(const float* q, const float* k, const float* v, const int64_t* mask_bc,
                  float* out, size_t bh, size_t sq, size_t sk, size_t d, double scale,
                  int threads);
void fvo_sdpa_f64_rows(const float* q, const float* k, const float* v, const int64_t* mask_bc,
                       const int64_t* rows, size_t nrows, float* out, size_t bh, size_t sq,
                       size_t sk, size_t d, double scale, int threads);

/* C/rt/attn.rs:441-467 */
int fvo_block_causal_allows(size_t block_tokens, size_t window, size_t sink, size_t q, size_t k);
void fvo_block_causal_dense_mask(size_t block_tokens, size_t window, size_t sink, size_t sq,
                                 size_t sk, float* mask);
/* C/rt/attn.rs:630-645; returns 1 and fills out[3] = {block_tokens, window, sink}, or 0 */
int fvo_block_causal_for(size_t num_frames_per_block, int64_t local_attn_size,
                         size_t frame_tokens, size_t* out3);
/* C/rt/attn.rs:483-523 — VDN-H3 window mask */
int fvo_vdn_window_allows(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                          size_t radius, size_t q, size_t k);
void fvo_vdn_window_dense_mask(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                               size_t radius, size_t sq, size_t sk, float* mask);
/* M/wan/family.rs:80-111 */
void fvo_causal_temporal_mask(const size_t patch[3], size_t num_frames_per_block,
                              int64_t local_attn_size, size_t frames, size_t height,
                              size_t width, float* mask);

/* C/rt/vsa.rs:29-37 */
size_t fvo_topk_for(double sparsity, size_t num_tiles);
/* C/rt/vsa.rs:62-109. dims_out = {tiles_t, tiles_h, tiles_w, seq, padded}. The
 * arrays may be NULL to query dims only. Returns 0, or -1 for an empty grid. */
int fvo_tile_plan(size_t t, size_t h, size_t w, size_t dims_out[5], int32_t* slot_src,
                  uint32_t* token_slot, uint32_t* block_sizes);
/* C/rt/vsa.rs:116-262. selected_out: NULL or [b*heads, nb, topk]. */
int fvo_vsa_attention_host(const float* q, const float* k, const float* v, const float* gate,
                           const int32_t* slot_src, const uint32_t* block_sizes, size_t seq,
                           size_t nb, size_t topk, size_t b, size_t heads, size_t dim,
                           float scale, float* out, uint32_t* selected_out);

/* C/rt/kernels/core.cu:576-579 */
uint32_t fvo_sortable(float x);
/* C/rt/kernels/core.cu:580-618 — device order: key > T ascending index, then
 * key == T ascending index, zero pad. */
void fvo_topk_device_order(const float* scores, uint32_t* out, size_t rows, size_t n, size_t k);
/* C/rt/vsa.rs:203-212 — host order: score descending (total order), index ascending. */
void fvo_topk_host_order(const float* scores, uint32_t* out, size_t rows, size_t n, size_t k);

/* C/rt/kernels/core.cu:550-570 — f32 sequential sum in slot order, then / n. */
void fvo_vsa_tile_mean(const float* x, const int32_t* slot_src, const uint32_t* block_sizes,
                       float* out, size_t bh, size_t seq, size_t dim, size_t nb, int round16);
/* C/rt/kernels/core.cu:803-835 (bf16 gate: C/rt/kernels/attn3.cu:247-270) — out[token] =
 * coarse[tile] * gate[token] + sparse[slot] for the real tokens of tiles [q_base, q_base + q_tiles),
 * gate NULL = 1. round16: bf16(bf16(sparse) + bf16(bf16(coarse) * bf16(gate))), without a gate
 * bf16(bf16(sparse) + bf16(coarse)). sparse is [bh, q_tiles*64, dim] in tile-slot order. */
void fvo_vsa_combine(const float* sparse, const float* coarse, const float* gate, const int32_t* slot_src,
                     float* out, size_t bh, size_t seq, size_t dim, size_t nb, size_t q_base,
                     size_t q_tiles, int round16);
/* C/rt/vsa.rs:185-189 (stage 2 of vsa_attention_host): scores[qt,kt] = f32(f64 dot of the tile means,
 * d ascending from -0.0, times f64(scale)). The device computes the same chain, so block lists compare
 * bit for bit with the host oracle's (the reference's own device path runs cuBLAS f32 here,
 * C/rt/vsa.rs:385-388, whose summation order is unspecified). */
void fvo_vsa_coarse_scores(const float* qc, const float* kc, float* scores, size_t bh, size_t nb,
                           size_t dim, float scale);

/* C/rt/sp.rs:16-28; out [world][2] = (start, len) */
void fvo_shard_ranges(size_t seq, size_t world, size_t* out);

/* ---- producer / consumer either side of the SDPA call --------------------------- */

/* C/rt/ops.rs:2304-2350 (f32 op): RMSNorm of columns [col_off, col_off+heads*d) of each
 * row of src [batch, seq, src_width] across all heads (sum of squares in index order),
 * times w, optional interleaved RoPE (cos from the even slot, sin from the odd slot of
 * the pair, tables [seq, d]; NULL tables = no rotation), out [batch, heads, seq, d]. */
void fvo_qk_norm_rope_bhsd(const float* src, const float* w, const float* cos_t, const float* sin_t,
                           float* out, size_t batch, size_t seq, size_t heads, size_t d,
                           size_t src_width, size_t col_off, float eps);
/* C/wan/fuse.rs:321-342 with C/rt/fuse/host.rs:217-270 under WAN_QK_NORM_ROPE
 * (C/rt/fuse/policy.rs:404-412): bf16(bf16(x*inv)*w), rotation in f32, one rounding;
 * values are bf16-representable f32. */
void fvo_wan_qk_norm_rope16(const float* src, const float* w, const float* cos_t, const float* sin_t,
                            float* out, size_t batch, size_t seq, size_t heads, size_t d,
                            size_t src_width, size_t col_off, float eps);
/* C/rt/ops.rs:2352-2372 */
void fvo_split_heads_bhsd(const float* src, float* out, size_t batch, size_t seq, size_t heads,
                          size_t d, size_t src_width, size_t col_off);
/* C/rt/ops.rs:2374-2386 */
void fvo_merge_heads(const float* src, float* out, size_t batch, size_t heads, size_t seq, size_t d);

#ifdef __cplusplus
}
#endif
#endif
