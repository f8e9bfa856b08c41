/*
 * libfv_sdpa_hip.so — C ABI of the gfx950 (MI355X) SDPA path that sits behind
 * fastvideo-rs's `rt::sdpa::sdpa` entry.
 *
 * All paths below are relative to the reference's crates/fastvideo-cudarc/src.
 *
 * Conventions
 *   - every tensor pointer is DEVICE memory, contiguous row-major; attention
 *     operands are BHSD flattened to [bh, s, d] (rt/attn.rs:44-54);
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *     every call is asynchronous on it and allocates nothing unless stated;
 *   - return value: FV_OK (0) launched; FV_DECLINED (1) the kernel does not
 *     take this call (the reference's launcher returning Ok(None),
 *     rt/sdpa.rs:217-233) — nothing was launched and nothing is ever computed
 *     on the host instead; a negative value is -(hipError_t) and
 *     fv_sdpa_last_error() holds the message (thread-local).
 */
#ifndef FV_SDPA_HIP_H
#define FV_SDPA_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FV_OK 0
#define FV_DECLINED 1

/* Message of the calling thread's last non-zero return ("" if none). */
const char* fv_sdpa_last_error(void);
/* "gfx950" — the only code object in the library. */
const char* fv_sdpa_arch(void);

/* Per-device set-up of the current HIP device: raises the dynamic-LDS limit of the kernels that use
 * more than 64 KB (`hipFuncSetAttribute`, the reference's `opt_in_dynamic_shared`, rt/ops.rs:1445-1461).
 * Optional: every entry point does this itself at its first launch on a device; call it before
 * capturing a HIP graph whose first launch of a kernel would otherwise fall inside the capture.
 * Also resolves this device's address of the static split-KV buffer (fv_sdpa_dense_bf16_splitkv_static).
 * Idempotent, thread-safe. */
int fv_sdpa_init(void);

/* rt/attn.rs:112-128 `mma_sdpa_supported`: 1 when the fused kernel takes a
 * [b,h,sq,d] x [b,h,sk,d] call: d == 128 or d == 64, sq > 0, sk > 0,
 * 1 <= b*h <= 65535, lengths fit int32. */
int fv_sdpa_supported(size_t b, size_t h, size_t sq, size_t sk, size_t d);

/* No counterpart in the reference. The fused kernels work in base 2 with the softmax offset riding in the C
 * operand of the K Q^T MFMAs: P = 2^(scale * log2(e) * (s - offset)), one multiply and one v_exp_f32 per score.
 * A caller that folds its softmax scale and log2(e) into Q before Q's one rounding to bf16 (for Wan: pass
 * out_mul = scale * log2(e) to fv_qk_norm_rope_bhsd) and passes scale = FV_SDPA_SCALE_LOG2_DOMAIN gets
 * scale * log2(e) == 1 exactly, and every fused entry (dense, strided, split-KV, block-causal, VDN window) then
 * runs a form without that multiply: 1.7 % faster at H=12 S=32760, more at head dim 64. Same arithmetic
 * otherwise, same tolerance against the host math at the same operands and scale. fv_vsa_fine (and through it
 * fv_vsa_attention, whose coarse stage uses the scale as given) takes the same form at that scale.
 * fv_sdpa_is_log2_domain_scale: 1 when `scale` selects that form. */
#define FV_SDPA_SCALE_LOG2_DOMAIN 0.6931471805599453f /* ln 2 */
int fv_sdpa_is_log2_domain_scale(float scale);
/* Launches of that form of the dense / masked kernel since the library was loaded (all its entries together). */
uint64_t fv_sdpa_log2_domain_launches(void);

/* No counterpart in the reference (a diagnostic). Launches that write bf16 and in which every query sees key 0
 * (dense; block-causal without a window or with sink blocks; the VDN window) make their pass over the keys with every
 * query's softmax offset fixed at the largest score of its first 128 keys (no running max in the loop), check the row sums
 * and accumulators before anything is stored, and make the pass again with the running max in any workgroup where
 * a row's scores outgrew that offset by more than about 2^90: results are exact either way, the second pass only
 * costs time. This is the number of workgroups that took it on the current device since the library was loaded.
 * Blocks until the device's work so far is done (a device-to-host copy of the counter); 0 without a device. */
uint64_t fv_sdpa_exact_pass_reruns(void);

/* rt/attn.rs:283-421 `device_mma_sdpa_with` + kernels/attn2.cu:607-621
 * `flash_mma_fwd2_d128` / `_d64`: out = softmax(scale * q k^T) v.
 * q [bh,sq,128], k/v [bh,sk,128] bf16 bits; out is f32 [bh,sq,128] when
 * out_is_bf16 == 0, else bf16 bits (RNE). scale > 0.
 * Rounding: with out_is_bf16 == 0 every row follows its running maximum (its largest P is exactly 1); with
 * out_is_bf16 == 1 the softmax offset of a row is the largest score of its first 128 keys (see
 * fv_sdpa_exact_pass_reruns), so a row that one later key dominates carries that key's bf16-rounded P: up to 2^-8
 * relative on such a row, beside the 2^-8 of the result's own rounding. FASTVIDEO_SDPA_RUNNING_MAX=1 (read once)
 * keeps the running maximum in every launch. */
int fv_sdpa_dense_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                       int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                       void* stream);

/* fv_sdpa_dense_bf16 on row windows of longer planes: the (batch, head) planes of q / k / v sit
 * q_rows / k_rows / v_rows rows of d elements apart (0 = contiguous: sq / sk). The KV-cache window of
 * autoregressive generation (wan/causal.rs:700-704, wan/transformer.rs:292-294) is read in place
 * instead of being copied out by `narrow`. out is contiguous [bh, sq, d]. */
int fv_sdpa_dense_bf16_strided(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                               int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                               size_t q_rows, size_t k_rows, size_t v_rows, void* stream);

/* Split-KV form of the dense kernel for calls whose query tiles do not fill the GPU (a block of one
 * latent frame against a long KV cache, a few prefix rows against the whole sequence): every
 * (head, query tile) gets `splits` workgroups, each walking a contiguous share of the key tiles and
 * writing a normalised f32 partial + its base-2 log-sum-exp into `workspace`; a merge kernel combines
 * them into `out`. Same operands as fv_sdpa_dense_bf16_strided. No counterpart in the reference, whose
 * kernels run one CTA per query tile (rt/attn.rs:378-395). fv_sdpa_splitkv_choose: the split count this
 * library would pick for a shape on the current device (1 = none: use the plain entry; fv_rt_sdpa
 * applies it by itself); splits is clamped to the number of 64-key tiles and so that no split is empty. workspace: 256-byte aligned,
 * fv_sdpa_splitkv_workspace_bytes(bh, sq, d, splits) bytes. Results agree with the unsplit kernel
 * to rounding (each split normalises by its own row sum before the merge). */
size_t fv_sdpa_splitkv_choose(size_t bh, size_t sq, size_t sk);
size_t fv_sdpa_splitkv_workspace_bytes(size_t bh, size_t sq, size_t d, size_t splits);
int fv_sdpa_dense_bf16_splitkv(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                               int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                               size_t q_rows, size_t k_rows, size_t v_rows, size_t splits, void* workspace,
                               size_t workspace_bytes, void* stream);

/* fv_sdpa_dense_bf16_splitkv for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): no counterpart in the reference. The
 * partial results live in a buffer inside the library's own code object (a file-scope __device__ array of
 * fv_sdpa_splitkv_static_bytes() = 32 MiB per GPU, held until the process ends) instead of a caller
 * workspace, and the call makes no hipMalloc / hipFree of any kind. splits == 0 takes
 * fv_sdpa_splitkv_choose's count, stepped down to the largest count whose partials fit the buffer (down to
 * 1 = unsplit), so the library's own choice is never refused. An explicit count whose partials need more
 * than the buffer (fv_sdpa_splitkv_workspace_bytes(bh, sq, d, splits) > fv_sdpa_splitkv_static_bytes()) is
 * refused with -hipErrorInvalidValue and a message; nothing is launched.
 * fv_sdpa_splitkv_static_splits (host arithmetic only): the split count a call with these arguments runs
 * with (>= 1), or 0 when it would be refused. Every call on a GPU shares that GPU's one
 * buffer: calls that overlap on one GPU (two streams, two threads) race; calls on one stream are ordered.
 * Nothing in the buffer has to start at zero (every split writes all of its rows before the merge reads
 * them). Results are bit-identical to fv_sdpa_dense_bf16_splitkv with the same split count. */
size_t fv_sdpa_splitkv_static_bytes(void);
size_t fv_sdpa_splitkv_static_splits(size_t bh, size_t sq, size_t sk, size_t d, size_t splits);
int fv_sdpa_dense_bf16_splitkv_static(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                                      int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                                      size_t q_rows, size_t k_rows, size_t v_rows, size_t splits, void* stream);

/* rt/attn.rs:652-730 `device_mma_sdpa_causal` + kernels/attn2.cu:626-642
 * `flash_mma_fwd2_causal_d128`: the same under BlockCausal{block_tokens,
 * window, sink} (rt/attn.rs:441-453): query i sees key j iff
 * (tj <= ti && (window == 0 || ti - tj < window)) || tj < sink, t = idx / block_tokens.
 * Key tiles no query of a workgroup can see are never loaded. A query that sees no key at all (more queries than
 * keys under a window that has moved past the last key) gets a row of zeros, what the reference's fused kernel
 * stores for a row without a visible key (kernels/attn2.cu:150); its composed route with the additive -1e9 mask
 * (rt/attn.rs:455-467) would give such a row the mean of V. No reference fixture covers the case: parity unpinned.
 * Rounding of bf16 results as for fv_sdpa_dense_bf16 when every query sees key 0 (window == 0 or sink > 0); under a
 * window without a sink every row follows its running maximum. */
int fv_sdpa_block_causal_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                              int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d,
                              float scale, size_t block_tokens, size_t window, size_t sink,
                              void* stream);

/* rt/attn.rs:526-610 `device_mma_sdpa_window` + kernels/attn2.cu:356-578, 648-663
 * `flash_mma_fwd2_window_d128`: the dense kernel under the VDN-H3 window mask (see
 * fv_vdn_window_allows): a key-tile walk over at most three ranges per query tile (rows before the
 * video + frame 0, the window frames of the tile, the last frame + rows after the video), per-score
 * masking on boundary tiles only. Self-attention (sq == sk), frames > 0, frame_tokens > 0, the video
 * rows inside the sequence; otherwise declines. Rounding of bf16 results as for fv_sdpa_dense_bf16 (every query
 * sees key 0 under this mask). */
int fv_sdpa_vdn_window_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                            int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                            size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                            size_t radius, void* stream);

/* rt/ops.rs:258-265 `cast_f32_bf16_device` + kernels/core.cu:121: f32 -> bf16
 * bits, RNE, NaN quiet, overflow to inf (kernels/core.cu:6-15). */
int fv_cast_f32_bf16(const float* x, uint16_t* y, size_t n, void* stream);
/* No counterpart in the reference: y = bf16(x * mul), the product in f32, one RNE rounding to bf16. With
 * mul = scale * log2(e) this is Q for a call at FV_SDPA_SCALE_LOG2_DOMAIN: the softmax scale goes into Q
 * before Q's only rounding to bf16 (fv_rt_sdpa does this by itself for f32 queries). */
int fv_cast_f32_bf16_scaled(const float* x, uint16_t* y, size_t n, float mul, void* stream);
/* bf16 bits -> f32 (exact widening), rt/tensor.rs `to_f32_act`. */
int fv_cast_bf16_f32(const uint16_t* x, float* y, size_t n, void* stream);

/* rt/ops.rs:377-401 `softmax_last_device` / `softmax_last_bf16_device` + kernels/core.cu:177-252
 * (host form rt/ops.rs:2178-2193): softmax over the contiguous trailing axis of x [rows, width],
 * out[r, j] = exp(x[r, j] - max_r) * (1 / sum_r); out f32 (may alias x) or bf16 bits (RNE). The step
 * between the two GEMMs of the reference's materialised attention and VSA coarse stage; the fused
 * kernels here never call it. */
int fv_softmax_last(const float* x, void* out, int out_is_bf16, size_t rows, size_t width, void* stream);

/* rt/sdpa.rs:328-342 `sdpa_composed` on the device: out = softmax(scale * q k^T + mask) v,
 * f32 operands [bh, s, d] and f32 out; mask NULL, or additive [sq, sk] shared by every bh
 * (mask_per_bh == 0), or [bh, sq, sk] (mask_per_bh != 0). The path for masked calls and for
 * shapes the fused kernels decline (it replaces the reference's cuBLAS-materialised and
 * scalar-flash fallbacks, rt/attn.rs:59-88, 748-865). 1 <= d <= 256. */
int fv_sdpa_composed_f32(const float* q, const float* k, const float* v, const float* mask,
                         int mask_per_bh, float* out, size_t bh, size_t sq, size_t sk, size_t d,
                         float scale, void* stream);

/* ---- the one entry: rt::sdpa::sdpa(q, k, v, &Plan) (rt/sdpa.rs:141-164), flattened ------- */
typedef struct fv_tensor {
    void* data;        /* device pointer, contiguous row-major */
    int dtype;         /* 0 = f32, 1 = bf16 bits (rt/tensor.rs:28-32) */
    int rank;
    size_t shape[8];
    size_t plane_rows; /* 0: contiguous. Else (rank 4 only) the [b,h] planes of `data` sit plane_rows * d
                          elements apart, plane_rows >= shape[2]: a row window of a longer BHSD buffer
                          (a KV cache read in place), what rt/tensor.rs:825 `narrow(2, ..)` copies out */
} fv_tensor;

enum {
    FV_PLAN_DENSE = 0,        /* Plan::dense / Plan::masked / .fp8_first() (rt/sdpa.rs:56-88) */
    FV_PLAN_COMPOSED = 1,     /* Plan::composed (rt/sdpa.rs:93-98) */
    FV_PLAN_BLOCK_CAUSAL = 2, /* Plan::block_causal (rt/sdpa.rs:104-109) */
    FV_PLAN_VDN_WINDOW = 3,   /* Plan::vdn_window (rt/sdpa.rs:111-119) */
    FV_PLAN_KV_WINDOW = 4     /* Plan::kv_window / kv_window_with (rt/sdpa.rs:125-137) */
};

typedef struct fv_plan {
    int kind;
    int has_scale;            /* 0: scale = 1/sqrt(d) */
    float scale;
    const fv_tensor* mask;    /* additive [.., sq, sk] for DENSE / COMPOSED, else NULL */
    int fp8_first;            /* accepted and ignored: this library is bf16 only */
    size_t block_tokens, window, sink;   /* BLOCK_CAUSAL */
    size_t video_start, frame_tokens, frames, chunk, radius;   /* VDN_WINDOW (rt/attn.rs:474-481) */
    int kv_flash;             /* KV_WINDOW: -1 = FASTVIDEO_WAN_CAUSAL_FLASH, 0 composed f32, 1 dense route */
} fv_plan;

/* Runs the plan on `stream`. q [b,h,sq,d], k/v [b,h,sk,d], f32 or bf16. On FV_OK `out` describes
 * a NEW device buffer owned by the caller (free with fv_rt_free or hipFree): bf16 under bf16
 * activations (FASTVIDEO_BF16_ACT, default on), else f32 (rt/sdpa.rs:184-214). Temporaries are
 * allocated stream-ordered. Errors return a negative code; fv_sdpa_last_error() holds the
 * reference's message ("sdpa expects BHSD", "sdpa: every kernel of the route declined", ...). */
int fv_rt_sdpa(const fv_tensor* q, const fv_tensor* k, const fv_tensor* v, const fv_plan* plan,
               fv_tensor* out, void* stream);
int fv_rt_free(void* p, void* stream);
/* rt/tensor.rs `with_bf16_act`: per-thread override of FASTVIDEO_BF16_ACT; v < 0 clears it. */
void fv_rt_set_bf16_activations(int v);
int fv_rt_bf16_activations(void);
/* No counterpart in the reference. When q arrives as f32, fv_rt_sdpa itself makes the bf16 copy the fused
 * kernels read (rt/sdpa.rs:167-181 `act16_operands`, rt/attn.rs:283-300): with this switch on
 * (FASTVIDEO_SDPA_FOLD_SCALE=1; fv_rt_set_fold_scale overrides per thread, v < 0 clears) that one rounding is
 * taken of q * (scale * log2(e)) and the kernel runs at FV_SDPA_SCALE_LOG2_DOMAIN, the form without the per-score
 * multiply; fv_vsa_attention does the same with an f32 q in its tile pass. Q is still rounded once, from the same
 * f32 values, so the result is as close to the f32 host math as with the switch off (bf16(c q) in place of
 * c bf16(q): different last bits, same error size) -- but it is one rounding of q away from the host math on the
 * ROUNDED operands, which is what the reference's own check of its kernel compares with at rel_l2 <= 2e-3
 * (gpucheck/src/kernels.rs:2314-2320): measured 2.6 - 2.8e-3 with the switch on, 1.3 - 1.6e-3 off. Hence OFF by
 * default: the reference's order (round, then scale) exactly. bf16 queries are never touched. */
void fv_rt_set_fold_scale(int v);
int fv_rt_fold_scale(void);
/* rt/log.rs:17-37: the level FASTVIDEO_LOG selects (read once): 0 quiet ("0", "off", "false", "quiet",
 * "error"), 2 debug ("2", "debug", "trace", "verbose"), 1 info (unset or anything else). At info and above
 * fv_rt_sdpa writes one "[fastvideo] sdpa: <kernel> B= H= Sq= Sk= D=" line to stderr the first time a
 * (kernel, shape) pair runs (rt/attn.rs:306-310). fv_rt_parse_log_level parses a value (NULL = unset). */
int fv_rt_log_level(void);
int fv_rt_parse_log_level(const char* v);
/* rt/sdpa_rule.rs:178-219 `Backend`, `parse_backend`, `backend`: FASTVIDEO_SDPA. 0 dense (the
 * default and every unknown value), 1 cublas, 2 flash, 3 host, 4 sparse. fv_rt_set_backend is a
 * per-thread override of the environment (v < 0 clears it). */
int fv_rt_parse_backend(const char* v);
int fv_rt_backend(void);
void fv_rt_set_backend(int v);
/* rt/sdpa_rule.rs:363-437 `Shape::of` + `dense_route` with the NVIDIA alternates removed. Shapes are
 * rank 4. steps_out receives the route (0 retired: the call is refused; 1 the fused gfx950 kernel;
 * 2 the composed f32 kernel), the return value is its length; dims_out (optional) = {b,h,sq,sk,d}
 * when k and v are both [b,h,sk,d], else zeros. Route: unmasked dense -> {1, 2}; cublas / flash (the
 * reference's f32-score kernels) -> {2}; host / sparse -> {0}; masked -> {2}. Host only. */
int fv_rt_dense_route(const size_t* q_shape, const size_t* k_shape, const size_t* v_shape, int masked,
                      int backend, int steps_out[4], size_t dims_out[5]);
/* rt/stats.rs:27-72 analogue: {fused dense launches, block-causal launches, composed launches,
 * cast launches, dense masks materialised} since the library was loaded. */
void fv_rt_stats(uint64_t out5[5]);

/* ---- the KV cache of causal (Self-Forcing) Wan generation (wan/causal.rs) ----------------------
 * wan/causal.rs:289-336 `KvSpec::plan`: where n new tokens at current_start go in a cache in state
 * (global_end, local_end_prev). move_out = {evicted, local_start, local_end, window_start}. Host only;
 * a negative return carries the reference's message in fv_sdpa_last_error(). */
int fv_kv_plan(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens, int rolling,
               size_t global_end, size_t local_end_prev, size_t current_start, size_t n, size_t move_out[4]);
/* wan/causal.rs:199-232 `copy_tokens` on device buffers [bh, rows, d] (f32 or bf16 elements, rows of a
 * 16-byte multiple): dst[:, dst_off .. dst_off + len] = src[:, src_off .. src_off + len]. */
int fv_kv_copy_tokens(void* dst, size_t dst_rows, size_t dst_off, const void* src, size_t src_rows, size_t src_off,
                      size_t len, size_t bh, size_t d, int is_bf16, void* stream);
/* wan/causal.rs:234-248 `shift_tokens_down`: tokens [from, from + len) of t [bh, rows, d] move down to
 * [to, to + len), to < from, in launches no longer than the shift (none reads what it writes). */
int fv_kv_shift_tokens_down(void* t, size_t rows, size_t from, size_t to, size_t len, size_t bh, size_t d,
                            int is_bf16, void* stream);
/* wan/causal.rs:341-723 `CausalKvCache::new_static`: one persistent [b, h, capacity, d] K / V pair per
 * layer (allocated with hipMalloc at the layer's first write, kept by fv_kv_cache_reset). rope_policy
 * (wan/causal.rs:59-76 `KvRope`): absolute (keys arrive roped), relativistic (the caller caches
 * un-roped keys and ropes the window itself; the cache only carries the flag), rebased sink (absolute
 * keys, the sink re-roped in place by fv_kv_cache_rebase_sink). fv_kv_cache_update = `update`: rolls (wan/causal.rs:678-690), writes the block's k / v
 * [b, h, n, d] at current_start and returns the windows the block's queries read as row windows of
 * the layer's buffers (plane_rows = capacity; valid until the layer's next update): pass them to
 * fv_rt_sdpa with FV_PLAN_KV_WINDOW (or fv_sdpa_dense_bf16_strided). Errors carry the reference's
 * messages. One cache is driven from one thread at a time per layer (a mutex serialises the host
 * bookkeeping); the device work is ordered on `stream`. */
typedef struct fv_kv_cache fv_kv_cache;
enum { FV_KV_ROPE_ABSOLUTE = 0, FV_KV_ROPE_RELATIVISTIC = 1, FV_KV_ROPE_REBASED_SINK = 2 };
fv_kv_cache* fv_kv_cache_new(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens, int rolling,
                             int rope_policy, size_t layers);
/* wan/causal.rs:379-393 `CausalKvCache::new` (not static): every fv_kv_cache_update builds the layer's K / V
 * anew, exactly local_end tokens long (the tokens kept before the write position, then the block), in
 * stream-ordered allocations, and releases the previous pair on the same stream; the windows returned hold
 * the same values as the static cache's (plane_rows = local_end) and are valid until the layer's next
 * update. Nothing a HIP graph could replay: fv_kv_cache_set_pointers / _advance refuse such a cache. */
fv_kv_cache* fv_kv_cache_new_dynamic(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens,
                                     int rolling, int rope_policy, size_t layers);
/* wan/causal.rs:395-397 `is_static`. */
int fv_kv_cache_is_static(const fv_kv_cache* c);
void fv_kv_cache_free(fv_kv_cache* c);
void fv_kv_cache_reset(fv_kv_cache* c);
/* wan/causal.rs:396-418 `set_sink_guard`: a write that re-runs cached frames leaves the sink slots. */
void fv_kv_cache_set_sink_guard(fv_kv_cache* c, int on);
/* out4 = {global_end, local_end, sink_at, raw_valid} of a layer (wan/causal.rs:353-360, 431-445). */
int fv_kv_cache_pointers(const fv_kv_cache* c, size_t layer, size_t out4[4]);
/* wan/causal.rs:457-476 `set_pointers`: in4 = `layers` x {global_end, local_end, sink_at, raw_valid}, one
 * entry per layer of the cache (a HIP-graph replay of a block forward moves no host state). */
int fv_kv_cache_set_pointers(fv_kv_cache* c, const size_t* in4, size_t layers);
/* wan/causal.rs:503-536 `advance`: the host bookkeeping of one block forward of n tokens at current_start
 * (rebased-sink target frame sink_target, 0: none) on every layer, without its device work. */
int fv_kv_cache_advance(fv_kv_cache* c, size_t current_start, size_t n, size_t sink_target);
/* wan/causal.rs:477-502 `block_key`: out5 = {local_end, appends, evicted, rebase, take_raw} of a forward of
 * n tokens at current_start (from layer 0's pointers): forwards with equal keys launch the same device
 * work, so a captured graph of one serves the others. Errors as fv_kv_plan. */
int fv_kv_cache_block_key(const fv_kv_cache* c, size_t current_start, size_t n, size_t sink_target, size_t out5[5]);
/* wan/causal.rs:733-776 `rebase_sink` (static mode): re-rope every layer's sink keys to start at frame
 * `target`. orig_cos / orig_sin: tables of the sink's own frames (used once, to take the un-roped f32
 * copy by rotating back); new_cos / new_sin: tables of frames [target, target + sink): f32
 * [sink_tokens, d], even-slot, device memory. Layers already there, or not yet holding the sink, are
 * left alone. */
int fv_kv_cache_rebase_sink(fv_kv_cache* c, size_t target, const float* orig_cos, const float* orig_sin,
                            const float* new_cos, const float* new_sin, void* stream);
/* wan/causal.rs:250-274 `rope_bhsd_f32` / `rope_bhsd` (kernels/core.cu:1933-1955 `apply_rotary_bshd` on
 * BHSD): out[:, r, 2i] = x1*c - x2*s, out[:, r, 2i+1] = x1*s + x2*c for rows r < s of every plane, c / s
 * from the even slot 2i of the f32 [s, d] tables (negate_sin: the inverse rotation). x / out are f32 or
 * bf16 bits (the bf16 result is the f32 one rounded once), planes x_rows / out_rows rows apart (0 = s). */
int fv_rope_bhsd(const void* x, int x_is_bf16, size_t x_rows, const float* cos_t, const float* sin_t, int negate_sin,
                 void* out, int out_is_bf16, size_t out_rows, size_t bh, size_t s, size_t d, void* stream);
size_t fv_kv_cache_bytes(const fv_kv_cache* c);
int fv_kv_cache_update(fv_kv_cache* c, size_t layer, const fv_tensor* k, const fv_tensor* v, size_t current_start,
                       fv_tensor* k_window, fv_tensor* v_window, void* stream);

/* ---- Video Sparse Attention (rt/vsa.rs, rt/ops.rs:811-1619) --------------------------
 * Geometry: 64-token cubes (4x4x4 in t,h,w), TilePlan arrays as rt/vsa.rs:42-109:
 * slot_src [num_tiles*64] (token of each padded slot, -1 = padding), block_sizes
 * [num_tiles] (real tokens per tile). Tensors are [bh, seq, dim] in token order or
 * [bh, num_tiles*64, dim] in tile-slot order ("tile-ordered"). */

/* rt/vsa.rs:34-37 `topk_for`: clamp(ceil((1 - sparsity) * num_tiles), 1, max(num_tiles, 1)). Host. */
size_t fv_vsa_topk_for(double sparsity, size_t num_tiles);
/* wan/transformer.rs:2194: the sparsity a caller that names none builds its VsaCtx with:
 * FASTVIDEO_VSA_SPARSITY parsed as f64 (trimmed; unset or unparsable = 0.8). The reference's other VSA
 * switches (FASTVIDEO_VSA_TOPK, _VSA_KERNEL, _VSA_TMA, _VSA_FUSED, _VSA_GROUP) choose among its kernels or
 * bound its gather buffer; this library has one kernel per stage and no gather buffer, so they select nothing. */
double fv_vsa_default_sparsity(void);
/* rt/vsa.rs:62-109 `TilePlan::new`. Host arrays. dims_out = {tiles_t, tiles_h, tiles_w,
 * seq, padded}; pass NULL arrays to query the dims. Negative return for an empty grid. */
int fv_vsa_tile_plan(size_t t, size_t h, size_t w, size_t dims_out[5], int32_t* slot_src,
                     uint32_t* token_slot, int32_t* block_sizes);

/* kernels/core.cu:550-570 `vsa_tile_mean`, kernels/attn3.cu:208-226 `vsa_tile_mean_b16`
 * (rt/ops.rs:868-872): out[bh, tile, :] = mean of the tile's real tokens, f32 sum in slot
 * order then / n. x is f32 or bf16 bits [bh, seq, dim]; round16 pools bf16-rounded values
 * of an f32 x. dim % 4 == 0. slot_src NULL: x is already tile-ordered, [bh, num_tiles*64, dim]
 * with seq = num_tiles*64 (slot j of a tile is its row j). */
int fv_vsa_tile_mean(const void* x, int x_is_bf16, const int32_t* slot_src, const int32_t* block_sizes,
                     float* out, size_t bh, size_t seq, size_t dim, size_t num_tiles, int round16,
                     void* stream);
/* rt/vsa.rs:385-394 (cuBLAS f32 + kernels/core.cu:177-252 `softmax_last` there):
 * scores[bh, qt, kt] = the host oracle's arithmetic (rt/vsa.rs:185-189): qc . kc accumulated in f64 over d
 * ascending, times scale in f64, one rounding to f32 (kept raw: they drive the selection, so the selected
 * sets equal `vsa_attention_host`'s); coarse[bh, qt, :] = softmax(scores[bh, qt, :]) vc.
 * coarse may be NULL (scores only). num_tiles <= 4096; coarse needs dim == 128. */
int fv_vsa_coarse(const float* qc, const float* kc, const float* vc, float* scores, float* coarse,
                  size_t bh, size_t num_tiles, size_t dim, float scale, void* stream);
/* kernels/core.cu:584-619 `vsa_topk`, kernels/attn3.cu:279-363 `vsa_topk2` (rt/ops.rs:887-923):
 * per row of n scores, T = k-th largest key under the order-preserving map of
 * kernels/core.cu:576-579; out[row, :] = indices with key > T ascending, then key == T
 * ascending, up to k; zero padded when k > n. Bit-exact. 1 <= n <= 4096. */
int fv_vsa_topk(const float* scores, uint32_t* out, size_t rows, size_t n, size_t k, void* stream);
/* kernels/core.cu:1659-1672 `vsa_tile_qkv`, kernels/attn3.cu:230-244 `vsa_tile_qkv_b16`
 * (rt/ops.rs:1077-1094): token order -> tile-ordered bf16, padding slots zero. dim % 8 == 0. */
int fv_vsa_tile_qkv(const void* x, int x_is_bf16, const int32_t* slot_src, uint16_t* xt, size_t bh,
                    size_t seq, size_t padded, size_t dim, void* stream);
/* kernels/core.cu:1039-1179 `vsa_mma_attn` (+ `_tma`, `_tma2`; rt/ops.rs:1328-1381): for query
 * tiles [q_base, q_base + q_tiles) of every bh, online softmax over the tiles of
 * selected[bh, tile, 0..topk) in list order; key columns >= block_sizes[tile] are -inf.
 * qt/kt/vt tile-ordered bf16; out f32 [bh, q_tiles*64, 128] in tile-slot order. dim == 128. */
int fv_vsa_fine(const uint16_t* qt, const uint16_t* kt, const uint16_t* vt, const uint32_t* selected,
                const int32_t* block_sizes, float* out, size_t bh, size_t num_tiles, size_t topk,
                size_t dim, float scale, size_t q_base, size_t q_tiles, void* stream);
/* kernels/core.cu:807-835 `vsa_combine` (rt/ops.rs:1592-1601): out[bh, token, :] =
 * coarse[bh, tile, :] * gate[bh, token, :] + sparse[bh, slot, :] for the real tokens of tiles
 * [q_base, q_base + q_tiles); gate NULL = 1; gate f32 or bf16 bits. dim == 128. */
int fv_vsa_combine(const float* sparse, const float* coarse, const void* gate, int gate_is_bf16,
                   const int32_t* slot_src, float* out, size_t bh, size_t seq, size_t dim,
                   size_t num_tiles, size_t q_base, size_t q_tiles, void* stream);
/* `vsa_combine` with round16 = 1 (kernels/core.cu:825-830, rt/ops.rs:1574-1601
 * `vsa_combine_round_device`) and its bf16-gate twin kernels/attn3.cu:247-270 `vsa_combine_g16`:
 * the H3 family's bf16 combine, out = bf16(bf16(sparse) + bf16(bf16(coarse) * bf16(gate))), without
 * a gate bf16(bf16(sparse) + bf16(coarse)); out stays f32 storage holding bf16 values. Same
 * arguments as fv_vsa_combine. */
int fv_vsa_combine_round16(const float* sparse, const float* coarse, const void* gate, int gate_is_bf16,
                           const int32_t* slot_src, float* out, size_t bh, size_t seq, size_t dim,
                           size_t num_tiles, size_t q_base, size_t q_tiles, void* stream);
/* rt/vsa.rs:358-424 `vsa_attention_device` with FineKernel::Mma: tile means -> coarse ->
 * top-k -> tile permute -> fine -> combine, all on `stream`, using caller-provided scratch
 * (fv_vsa_workspace_bytes, 256-byte aligned). The combine runs in the fine kernel's epilogue
 * (same f32 arithmetic, mul then add), so no f32 sparse buffer is part of the scratch.
 * topk is clamped to [1, num_tiles]. q/k/v (and
 * gate) are f32 or bf16 bits in token order; out f32 [bh, seq, 128]. selected_out: NULL or
 * [bh, num_tiles, topk] to receive the block index lists. */
size_t fv_vsa_workspace_bytes(size_t bh, size_t num_tiles, size_t topk, size_t dim);
int fv_vsa_attention(const void* q, const void* k, const void* v, int qkv_is_bf16, const void* gate,
                     int gate_is_bf16, const int32_t* slot_src, const int32_t* block_sizes, float* out,
                     void* workspace, size_t workspace_bytes, uint32_t* selected_out, size_t bh,
                     size_t seq, size_t num_tiles, size_t topk, size_t dim, float scale, void* stream);

/* fv_vsa_attention on operands a producer already wrote in tile-slot order (fv_qk_norm_rope_tiles,
 * fv_split_heads_tiles): qt/kt/vt bf16 bits [bh, num_tiles*64, 128] with zero padding slots; gate
 * and out stay in token order. The tile means read the tiles in place and the tile pass (three
 * reads and writes of q/k/v) is skipped; the result is bit-identical to fv_vsa_attention on the
 * token-ordered bf16 tensors. No counterpart in the reference, whose op always re-tiles
 * (rt/vsa.rs:406-414). Needs only the first part of the workspace (fv_vsa_workspace_bytes is
 * enough). */
int fv_vsa_attention_tiled(const uint16_t* qt, const uint16_t* kt, const uint16_t* vt, const void* gate,
                           int gate_is_bf16, const int32_t* slot_src, const int32_t* block_sizes, float* out,
                           void* workspace, size_t workspace_bytes, uint32_t* selected_out, size_t bh,
                           size_t seq, size_t num_tiles, size_t topk, size_t dim, float scale, void* stream);

/* ---- producer / consumer either side of the SDPA call --------------------------------- */
/* q/k RMSNorm across all heads (+ interleaved RoPE) of columns [col_off, col_off + heads*d) of
 * src [batch, seq, src_width], written as BHSD [batch, heads, seq, d].
 * out_is_bf16 == 0: the f32 op, `x*inv*w`, rotation, f32 out — rt/ops.rs:528-572 /
 *   kernels/core.cu:373-413 `qk_norm_rope_bhsd` (host form rt/ops.rs:2304-2350).
 * out_is_bf16 == 1: the bf16 q/k kernel with its rounding points, `bf16(bf16(x*inv)*w)`, rotation
 *   in f32, one rounding, bf16 out — wan/fuse.rs:527-561 `wan_qk_norm_rope16` (policy
 *   rt/fuse/policy.rs:404-412, host twin rt/fuse/host.rs:217-276).
 * src and w are f32 or bf16 (flags); cos_t / sin_t are f32 [seq, d] (cos read from the even slot
 * of a pair, sin from the odd one) or both NULL for no rotation. Declines unless d, col_off and
 * src_width are multiples of 8.
 * out_mul (no counterpart in the reference; 1.0f = the reference's op, bit for bit): every output value is
 * multiplied by it in f32 after the rotation and before the write (before the ONE rounding of the bf16 form's
 * rotated values), so q can leave the producer as q * scale * log2(e) for an SDPA call at
 * FV_SDPA_SCALE_LOG2_DOMAIN without touching the norm weights. (Without rotation the bf16 form's value is
 * already a bf16 number when out_mul meets it: a second rounding, to be weighed by the caller.) */
int fv_qk_norm_rope_bhsd(const void* src, int src_is_bf16, const void* w, int w_is_bf16,
                         const float* cos_t, const float* sin_t, void* out, int out_is_bf16,
                         size_t batch, size_t seq, size_t heads, size_t d, size_t src_width,
                         size_t col_off, float eps, float out_mul, void* stream);
/* The same op writing VSA's tile-slot order: head planes are [padded, d] and token s lands in row
 * token_slot[s] (fv_vsa_tile_plan; every value < padded, others are skipped). Padding rows are not
 * written: zero `out` once, no call touches them afterwards. Feeds fv_vsa_attention_tiled. */
int fv_qk_norm_rope_tiles(const void* src, int src_is_bf16, const void* w, int w_is_bf16,
                          const float* cos_t, const float* sin_t, void* out, int out_is_bf16,
                          size_t batch, size_t seq, size_t heads, size_t d, size_t src_width,
                          size_t col_off, float eps, float out_mul, const uint32_t* token_slot, size_t padded,
                          void* stream);
/* rt/ops.rs:574-602 / kernels/core.cu:415-427 `split_heads_bhsd`: the value heads, a pure permute
 * of f32 or bf16 elements. */
int fv_split_heads_bhsd(const void* src, void* out, int is_bf16, size_t batch, size_t seq, size_t heads,
                        size_t d, size_t src_width, size_t col_off, void* stream);
/* fv_split_heads_bhsd into tile-slot order, as fv_qk_norm_rope_tiles. */
int fv_split_heads_tiles(const void* src, void* out, int is_bf16, size_t batch, size_t seq, size_t heads,
                         size_t d, size_t src_width, size_t col_off, const uint32_t* token_slot, size_t padded,
                         void* stream);
/* rt/ops.rs:604-620 / kernels/core.cu:429-443 `merge_heads`: BHSD -> [batch, seq, heads*d]. */
int fv_merge_heads(const void* src, void* out, int is_bf16, size_t batch, size_t heads, size_t seq, size_t d,
                   void* stream);

/* ---- host-side mask / sharding helpers ------------------------------------------------ */
/* rt/attn.rs:449-453 `BlockCausal::allows`. */
int fv_block_causal_allows(size_t block_tokens, size_t window, size_t sink, size_t q, size_t k);
/* rt/attn.rs:456-466 `BlockCausal::dense_mask`: host [sq, sk], 0 visible / -1e9 masked. */
void fv_block_causal_dense_mask(size_t block_tokens, size_t window, size_t sink, size_t sq,
                                size_t sk, float* mask);
/* rt/attn.rs:497-510 `VdnWindow::allows`: rows outside [video_start, video_start +
 * frames*frame_tokens) and the frames 0 and frames-1 are dense both ways; any other video query
 * frame sees the key frames of its window (chunk-aligned, radius chunks each side; chunk == 0 is a
 * centred frame window). */
int fv_vdn_window_allows(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                         size_t radius, size_t q, size_t k);
/* rt/attn.rs:513-523 `VdnWindow::dense_mask`: host [sq, sk], 0 visible / -1e9 masked. */
void fv_vdn_window_dense_mask(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                              size_t radius, size_t sq, size_t sk, float* mask);
/* rt/attn.rs:630-645 `block_causal_for`: 1 and out3 = {block_tokens, window, 0}, or 0 when the
 * token window does not cover whole blocks. */
int fv_block_causal_for(size_t num_frames_per_block, long long local_attn_size, size_t frame_tokens,
                        size_t out3[3]);
/* The key tiles (64 keys each) that the fused block-causal kernel walks for the 256 queries starting at
 * q0 (a multiple of 256): the loop bounds of the causal kernel body (kernels/attn2.cu:214-221), here up
 * to two ascending tile ranges, out4 = {0 .. n0 (sink tiles), a1 .. a1 + n1 (the band)} as
 * {n0, a1, n1, total}. total == 0: no query of the tile sees a key and its rows come out as zeros.
 * Host arithmetic only (the kernel runs the same function); 0, or FV_DECLINED for parameters the
 * kernel does not take. */
int fv_block_causal_tile_walk(size_t block_tokens, size_t window, size_t sink, size_t sq, size_t sk, size_t q0,
                              int out4[4]);
/* rt/sp.rs:16-28 `shard_ranges`: out[world][2] = (start, len). The library itself never
 * shards (the full sequence stays on one GPU); kept for callers that do. */
void fv_sp_shard_ranges(size_t seq, size_t world, size_t* out);

#ifdef __cplusplus
}
#endif
#endif
