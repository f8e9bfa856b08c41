// C ABI of libfv_sdpa_hip.so: argument checks, decline rules and launches.
// Declarations and reference citations live in include/fv_sdpa_hip.h.
#include "../../include/fv_sdpa_hip.h"

#include <limits.h>
#include <stdio.h>

#include <string>

#include "fv_common.h"
#include "fv_internal.h"

static thread_local std::string g_last_error;
int fv_fail_hip(hipError_t e, const char* what) {
    char buf[256];
    snprintf(buf, sizeof buf, "%s: %s (hipError %d)", what, hipGetErrorString(e), (int)e);
    g_last_error = buf;
    return -(int)e;
}
int fv_decline(const char* why) {
    g_last_error = why;
    return FV_DECLINED;
}
int fv_invalid(const char* why) {
    g_last_error = why;
    return -(int)hipErrorInvalidValue;
}

namespace {

int fail_hip(hipError_t e, const char* what) { return fv_fail_hip(e, what); }
int decline(const char* why) { return fv_decline(why); }

__global__ void cast_f32_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y,
                                     size_t n) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 4 <= n && ((((uintptr_t)x) & 15) == 0) && ((((uintptr_t)y) & 7) == 0)) {
        const fv::f32x4 v = *reinterpret_cast<const fv::f32x4*>(x + i);
        fv::s16x4 o;
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = (short)fv::bf16_rne_bits(v[j]);
        *reinterpret_cast<fv::s16x4*>(y + i) = o;
    } else {
        for (size_t j = i; j < n && j < i + 4; j++) y[j] = fv::bf16_rne_bits(x[j]);
    }
}

__global__ void cast_bf16_f32_kernel(const uint16_t* __restrict__ x, float* __restrict__ y,
                                     size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = fv::bf16_bits_to_f32(x[i]);
}

int flash_common(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                 int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                 bool causal, size_t block_tokens, size_t window, size_t sink, void* stream) {
    if (!fv_sdpa_supported(1, bh, sq, sk, d)) return decline("sdpa: shape not taken by the fused kernel");
    if (!(scale > 0.0f) || !(scale < 3.0e38f)) return decline("sdpa: the fused kernel needs a finite scale > 0");
    if (!q || !k || !v || !out) return fv_invalid("sdpa: null operand");
    fv::FlashParams p;
    p.q = q;
    p.k = k;
    p.v = v;
    p.out_f32 = out_is_bf16 ? nullptr : (float*)out;
    p.out_bf16 = out_is_bf16 ? (uint16_t*)out : nullptr;
    p.out_is_bf16 = out_is_bf16 ? 1 : 0;
    p.sq = (int)sq;
    p.sk = (int)sk;
    p.sl2 = scale * 1.4426950408889634f;
    const size_t bm = (size_t)fv_internal_flash_block_m();
    p.nqt = (int)((sq + bm - 1) / bm);
    const size_t total = bh * (size_t)p.nqt;
    if (total > (size_t)INT_MAX / 2) return decline("sdpa: too many query tiles for one launch");
    p.total = (int)total;
    p.per_xcd = (int)((total + 7) / 8);
    p.ft = p.win = p.sink = 0;
    if (causal) {
        // rt/attn.rs:668-676
        const size_t lim = (size_t)INT_MAX;
        if (block_tokens == 0 || window > lim || sink > lim || (sq > sk ? sq : sk) + block_tokens > lim)
            return decline("sdpa: block-causal parameters outside the kernel's int range");
        p.ft = (int)block_tokens;
        p.win = (int)window;
        p.sink = (int)sink;
        // One block spanning both sequences: every key is visible to every query (tq == tk == 0
        // for any window), so this is the dense problem and runs on the dense kernel, bit for bit
        // (the reference asserts that identity for its own kernels, gpucheck kernels_wan.rs:230-261).
        if (block_tokens >= sq && block_tokens >= sk) causal = false;
    }
    hipError_t e = fv_internal_launch_flash(&p, causal ? 1 : 0, (int)d, (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip(e, causal ? "flash_fwd_pp2<causal>" : "flash_fwd_pp2<dense>");
    return FV_OK;
}

}  // namespace

extern "C" {

const char* fv_sdpa_last_error(void) { return g_last_error.c_str(); }
const char* fv_sdpa_arch(void) { return "gfx950"; }

int fv_sdpa_supported(size_t b, size_t h, size_t sq, size_t sk, size_t d) {
    if (b != 0 && h > (size_t)65535 / b) return 0;
    const size_t bh = b * h;
    return (d == 128 || d == 64) && sq > 0 && sk > 0 && bh >= 1 && bh <= 65535 && sq <= (size_t)INT_MAX &&
           sk <= (size_t)INT_MAX;
}

int fv_sdpa_dense_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                       int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                       void* stream) {
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, false, 0, 0, 0, stream);
}

int fv_sdpa_block_causal_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                              int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d,
                              float scale, size_t block_tokens, size_t window, size_t sink,
                              void* stream) {
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, true, block_tokens, window,
                        sink, stream);
}

int fv_cast_f32_bf16(const float* x, uint16_t* y, size_t n, void* stream) {
    if (n == 0) return FV_OK;
    const size_t threads = (n + 3) / 4;
    const size_t blocks = (threads + 255) / 256;
    if (blocks > (size_t)INT_MAX) return decline("cast: too many elements for one launch");
    hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, x, y, n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fail_hip(e, "cast_f32_bf16");
}

int fv_cast_bf16_f32(const uint16_t* x, float* y, size_t n, void* stream) {
    if (n == 0) return FV_OK;
    const size_t blocks = (n + 255) / 256;
    if (blocks > (size_t)INT_MAX) return decline("cast: too many elements for one launch");
    hipLaunchKernelGGL(cast_bf16_f32_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, x, y, n);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fail_hip(e, "cast_bf16_f32");
}

}  // extern "C"
