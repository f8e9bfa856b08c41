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

/* rt/attn.rs:112-128 `mma_sdpa_supported`: 1 when the fused kernel takes a
 * [b,h,sq,d] x [b,h,sk,d] call: d == 128, sq > 0, sk > 0, 1 <= b*h <= 65535,
 * lengths fit int32. (The reference's d == 64 variant serves audio models that
 * are outside this library; such calls decline.) */
int fv_sdpa_supported(size_t b, size_t h, size_t sq, size_t sk, size_t d);

/* rt/attn.rs:283-421 `device_mma_sdpa_with` + kernels/attn2.cu:607-621
 * `flash_mma_fwd2_d128`: out = softmax(scale * q k^T) v.
 * q [bh,sq,128], k/v [bh,sk,128] bf16 bits; out is f32 [bh,sq,128] when
 * out_is_bf16 == 0, else bf16 bits (RNE). scale > 0. */
int fv_sdpa_dense_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                       int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                       void* stream);

/* rt/attn.rs:652-730 `device_mma_sdpa_causal` + kernels/attn2.cu:626-642
 * `flash_mma_fwd2_causal_d128`: the same under BlockCausal{block_tokens,
 * window, sink} (rt/attn.rs:441-453): query i sees key j iff
 * (tj <= ti && (window == 0 || ti - tj < window)) || tj < sink, t = idx / block_tokens.
 * Key tiles no query of a workgroup can see are never loaded. */
int fv_sdpa_block_causal_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                              int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d,
                              float scale, size_t block_tokens, size_t window, size_t sink,
                              void* stream);

/* rt/ops.rs:258-265 `cast_f32_bf16_device` + kernels/core.cu:121: f32 -> bf16
 * bits, RNE, NaN quiet, overflow to inf (kernels/core.cu:6-15). */
int fv_cast_f32_bf16(const float* x, uint16_t* y, size_t n, void* stream);
/* bf16 bits -> f32 (exact widening), rt/tensor.rs `to_f32_act`. */
int fv_cast_bf16_f32(const uint16_t* x, float* y, size_t n, void* stream);

#ifdef __cplusplus
}
#endif
#endif
