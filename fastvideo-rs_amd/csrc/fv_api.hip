// C ABI of libfv_sdpa_hip.so: argument checks, decline rules and launches.
// Declarations and reference citations live in include/fv_sdpa_hip.h.
#include "../../include/fv_sdpa_hip.h"

#include <limits.h>
#include <stdio.h>

#include <atomic>
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

// y = bf16(x * mul), RNE; mul == 1 is the plain cast (x * 1.0f is x)
__global__ void cast_f32_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ y,
                                     size_t n, float mul) {
    const size_t i = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 4 <= n && ((((uintptr_t)x) & 15) == 0) && ((((uintptr_t)y) & 7) == 0)) {
        const fv::f32x4 v = *reinterpret_cast<const fv::f32x4*>(x + i);
        fv::s16x4 o;
#pragma unroll
        for (int j = 0; j < 4; j++) o[j] = (short)fv::bf16_rne_bits(v[j] * mul);
        *reinterpret_cast<fv::s16x4*>(y + i) = o;
    } else {
        for (size_t j = i; j < n && j < i + 4; j++) y[j] = fv::bf16_rne_bits(x[j] * mul);
    }
}

__global__ void cast_bf16_f32_kernel(const uint16_t* __restrict__ x, float* __restrict__ y,
                                     size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) y[i] = fv::bf16_bits_to_f32(x[i]);
}

// ---- static split-KV buffer ------------------------------------------------------------------
// The partials of fv_sdpa_dense_bf16_splitkv_static: part of the code object, so every GPU the
// library runs on holds its own copy at its own address from module load to process end. In host
// code the array's NAME is only a handle for hipGetSymbolAddress, never a device address: kernels
// and copies get the per-device pointer resolved below.
constexpr size_t kStaticScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// This device's address of `scratch` (resolved once per device, with that device current).
hipError_t static_scratch(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p || (((uintptr_t)p) & 255) != 0) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(p, std::memory_order_release);   // racing first calls store the same address
    }
    *out = p;
    return hipSuccess;
}

enum { kMaskNone = 0, kMaskBlockCausal = 1, kMaskVdnWindow = 2 };

// The split count a launch settles on for `nkt` key tiles when `splits` are asked for: never more splits
// than key tiles (also keeps the sums below from wrapping on absurd counts), and no empty split.
size_t settle_splits(size_t nkt, size_t splits) {
    if (splits <= 1 || nkt <= 1) return 1;
    if (splits > nkt) splits = nkt;
    const size_t per = (nkt + splits - 1) / splits;
    return (nkt + per - 1) / per;
}

struct MaskArgs {
    int mode = kMaskNone;
    size_t q_rows = 0, k_rows = 0, v_rows = 0;   // rows per (batch, head) plane; 0 = contiguous (sq / sk)
    size_t splits = 1;                            // split-KV (dense only): key splits per query tile
    void* workspace = nullptr;                    // ... and their partial results
    size_t workspace_bytes = 0;
    size_t block_tokens = 0, window = 0, sink = 0;                           // block-causal
    size_t video_start = 0, frame_tokens = 0, frames = 0, chunk = 0, radius = 0;   // VDN window
};

int flash_common(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                 int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                 const MaskArgs& m, void* stream) {
    if (!fv_sdpa_supported(1, bh, sq, sk, d)) return decline("sdpa: shape not taken by the fused kernel");
    if (!(scale > 0.0f) || !(scale < 3.0e38f)) return decline("sdpa: the fused kernel needs a finite scale > 0");
    if (!q || !k || !v || !out) return fv_invalid("sdpa: null operand");
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0)
        return fv_invalid("sdpa: operands must be 16-byte aligned");
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
    const size_t q_rows = m.q_rows ? m.q_rows : sq, k_rows = m.k_rows ? m.k_rows : sk,
                 v_rows = m.v_rows ? m.v_rows : sk;
    if (q_rows < sq || k_rows < sk || v_rows < sk) return fv_invalid("sdpa: plane rows below the sequence length");
    const size_t plane_lim = (size_t)LONG_MAX / (d * (bh ? bh : 1));
    if (q_rows > plane_lim || k_rows > plane_lim || v_rows > plane_lim)
        return decline("sdpa: planes too large");
    p.q_plane = (long)(q_rows * d);
    p.k_plane = (long)(k_rows * d);
    p.v_plane = (long)(v_rows * d);
    const size_t bm = (size_t)fv_internal_flash_block_m();
    p.nqt = (int)((sq + bm - 1) / bm);
    const size_t total = bh * (size_t)p.nqt;
    if (total > (size_t)INT_MAX / 2) return decline("sdpa: too many query tiles for one launch");
    p.total = (int)total;
    p.per_xcd = (int)((total + 7) / 8);
    p.mask_mode = kMaskNone;
    p.ft = p.win = p.sink = 0;
    p.vs = p.ve = p.frames = p.chunk = p.radius = 0;
    int mode = m.mode;
    const size_t lim = (size_t)INT_MAX;
    if (mode == kMaskBlockCausal) {
        // rt/attn.rs:668-676
        if (m.block_tokens == 0 || m.window > lim || m.sink > lim || (sq > sk ? sq : sk) + m.block_tokens > lim)
            return decline("sdpa: block-causal parameters outside the kernel's int range");
        p.ft = (int)m.block_tokens;
        p.win = (int)m.window;
        p.sink = (int)m.sink;
        // One block spanning both sequences: every key is visible to every query (tq == tk == 0
        // for any window), so this is the dense problem and runs as the dense launch, bit for bit
        // (the reference asserts that identity for its own kernels, gpucheck kernels_wan.rs:230-261).
        if (m.block_tokens >= sq && m.block_tokens >= sk) mode = kMaskNone;
    } else if (mode == kMaskVdnWindow) {
        // rt/attn.rs:544-553: self-attention only, the video rows inside the sequence
        const size_t ve = m.video_start + m.frames * m.frame_tokens;
        if (sq != sk || m.frames == 0 || m.frame_tokens == 0 || m.frames > lim / m.frame_tokens || ve > sk ||
            m.chunk > lim || m.radius > lim / 2 || (m.chunk > 0 && m.radius > lim / (2 * m.chunk)))
            return decline("sdpa: VDN window parameters the kernel cannot run");
        p.ft = (int)m.frame_tokens;
        p.vs = (int)m.video_start;
        p.ve = (int)ve;
        p.frames = (int)m.frames;
        p.chunk = (int)m.chunk;
        // a radius past the clip means every frame: clamp so that (f/c + r + 1) * c stays in int range
        p.radius = (int)(m.radius > m.frames ? m.frames : m.radius);
        if (m.frames <= 2) mode = kMaskNone;   // anchors only: dense
    }
    p.mask_mode = mode;
    p.kv_split = 1;
    p.split_tiles = INT_MAX;
    p.part_o = nullptr;
    p.part_lse = nullptr;
    const size_t nkt = (sk + 63) / 64;
    size_t splits = mode == kMaskNone ? settle_splits(nkt, m.splits) : 1;
    if (splits > 1) {
        if (total * splits > (size_t)INT_MAX / 2) return decline("sdpa: too many workgroups for one launch");
        const size_t need = fv_sdpa_splitkv_workspace_bytes(bh, sq, d, splits);
        if (!m.workspace || m.workspace_bytes < need || (((uintptr_t)m.workspace) & 255) != 0)
            return fv_invalid("sdpa: split-KV needs a 256-byte aligned workspace of fv_sdpa_splitkv_workspace_bytes");
        p.kv_split = (int)splits;
        p.split_tiles = (int)((nkt + splits - 1) / splits);
        p.part_o = (float*)m.workspace;
        p.part_lse = (float*)((char*)m.workspace + ((splits * bh * sq * d * 4 + 255) & ~(size_t)255));
        p.total = (int)(total * splits);
        p.per_xcd = (p.total + 7) / 8;
    }
    hipError_t e = fv_internal_launch_flash(&p, mode != kMaskNone ? 1 : 0, (int)d, (hipStream_t)stream);
    if (e != hipSuccess) return fail_hip(e, mode != kMaskNone ? "flash_fwd_pp2<masked>" : "flash_fwd_pp2<dense>");
    if (p.kv_split > 1) {
        e = fv_internal_launch_splitkv_merge(p.part_o, p.part_lse, out, out_is_bf16 ? 1 : 0, bh * sq, (int)d, p.kv_split,
                                             (hipStream_t)stream);
        if (e != hipSuccess) return fail_hip(e, "splitkv_merge");
    }
    return FV_OK;
}

}  // namespace

extern "C" {

const char* fv_sdpa_last_error(void) { return g_last_error.c_str(); }
const char* fv_sdpa_arch(void) { return "gfx950"; }

int fv_sdpa_init(void) {
    hipError_t e = fv_internal_init_flash();
    if (e == hipSuccess) e = fv_internal_init_vsa();
    void* p = nullptr;
    if (e == hipSuccess) e = static_scratch(&p);
    return e == hipSuccess ? FV_OK : fail_hip(e, "fv_sdpa_init");
}

// the launcher's own test (flash_fwd.hip launch_flash): FlashParams::sl2, computed as below, equal to one
int fv_sdpa_is_log2_domain_scale(float scale) { return scale * 1.4426950408889634f == 1.0f ? 1 : 0; }

uint64_t fv_sdpa_exact_pass_reruns(void) {
    unsigned long long n = 0;
    return fv_internal_exact_pass_reruns(&n) == hipSuccess ? (uint64_t)n : 0;
}

int fv_sdpa_supported(size_t b, size_t h, size_t sq, size_t sk, size_t d) {
    if (b != 0 && h > (size_t)65535 / b) return 0;
    const size_t bh = b * h;
    return (d == 128 || d == 64) && sq > 0 && sk > 0 && bh >= 1 && bh <= 65535 && sq <= (size_t)INT_MAX &&
           sk <= (size_t)INT_MAX;
}

int fv_sdpa_dense_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                       int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                       void* stream) {
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, MaskArgs{}, stream);
}

int fv_sdpa_dense_bf16_strided(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                               int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                               size_t q_rows, size_t k_rows, size_t v_rows, void* stream) {
    MaskArgs m;
    m.q_rows = q_rows;
    m.k_rows = k_rows;
    m.v_rows = v_rows;
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, m, stream);
}

size_t fv_sdpa_splitkv_workspace_bytes(size_t bh, size_t sq, size_t d, size_t splits) {
    if (splits <= 1) return 0;
    return ((splits * bh * sq * d * 4 + 255) & ~(size_t)255) + ((splits * bh * sq * 4 + 255) & ~(size_t)255);
}

size_t fv_sdpa_splitkv_choose(size_t bh, size_t sq, size_t sk) {
    static const int cus = [] {
        int dev = 0, n = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
        return n;
    }();
    const size_t bm = (size_t)fv_internal_flash_block_m();
    const size_t wgs = bh * ((sq + bm - 1) / bm), nkt = (sk + 63) / 64;
    if (wgs == 0 || wgs >= (size_t)cus) return 1;               // the query tiles alone fill the CUs
    // Cost model (microseconds, measured on MI355X): a workgroup costs about 10 fixed + 1.7 per 64-key
    // tile, workgroups run in rounds of one per CU, and the merge reads `s` f32 partials at about
    // 4 TB/s. Take the cheapest split count, if it wins by more than 10 %.
    auto cost = [&](size_t sp) {
        const size_t per = (nkt + sp - 1) / sp, real = (nkt + per - 1) / per;
        const double rounds = (double)((wgs * real + cus - 1) / cus);
        const double merge = real > 1 ? (double)(real * bh * sq) * 128.0 * 4.0 / 4.0e6 + 5.0 : 0.0;
        return rounds * (10.0 + 1.7 * (double)per) + merge;
    };
    size_t best = 1;
    double best_cost = cost(1);
    for (size_t sp = 2; sp <= 16 && sp * 8 <= nkt; sp++) {        // at least 8 key tiles (4 phases) per split
        const double c = cost(sp);
        if (c < best_cost) best_cost = c, best = sp;
    }
    return best_cost < 0.9 * cost(1) ? best : 1;
}

int fv_sdpa_dense_bf16_splitkv(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                               int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                               size_t q_rows, size_t k_rows, size_t v_rows, size_t splits, void* workspace,
                               size_t workspace_bytes, void* stream) {
    MaskArgs m;
    m.q_rows = q_rows;
    m.k_rows = k_rows;
    m.v_rows = v_rows;
    m.splits = splits ? splits : 1;
    m.workspace = workspace;
    m.workspace_bytes = workspace_bytes;
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, m, stream);
}

size_t fv_sdpa_splitkv_static_bytes(void) { return kStaticScratchBytes; }

size_t fv_sdpa_splitkv_static_splits(size_t bh, size_t sq, size_t sk, size_t d, size_t splits) {
    const size_t nkt = (sk + 63) / 64;
    if (splits != 0) {   // the caller's count, settled as the launch would; refused when its partials do not fit
        splits = settle_splits(nkt, splits);
        return fv_sdpa_splitkv_workspace_bytes(bh, sq, d, splits) <= kStaticScratchBytes ? splits : 0;
    }
    // the library's own choice never refuses: it steps down to the largest count whose partials fit (1 = unsplit)
    for (size_t s = fv_sdpa_splitkv_choose(bh, sq, sk); s > 1; s--) {
        const size_t real = settle_splits(nkt, s);
        if (fv_sdpa_splitkv_workspace_bytes(bh, sq, d, real) <= kStaticScratchBytes) return real;
    }
    return 1;
}

int fv_sdpa_dense_bf16_splitkv_static(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                                      int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                                      size_t q_rows, size_t k_rows, size_t v_rows, size_t splits, void* stream) {
    if (!fv_sdpa_supported(1, bh, sq, sk, d)) return decline("sdpa: shape not taken by the fused kernel");
    const size_t run = fv_sdpa_splitkv_static_splits(bh, sq, sk, d, splits);
    if (run == 0) {
        char buf[200];
        snprintf(buf, sizeof buf,
                 "sdpa: split-KV partials of this call need %zu bytes, the static buffer holds %zu "
                 "(use fv_sdpa_dense_bf16_splitkv with a workspace)",
                 fv_sdpa_splitkv_workspace_bytes(bh, sq, d, settle_splits((sk + 63) / 64, splits)), kStaticScratchBytes);
        return fv_invalid(buf);
    }
    MaskArgs m;
    m.q_rows = q_rows;
    m.k_rows = k_rows;
    m.v_rows = v_rows;
    m.splits = run;
    if (run > 1) {
        void* p = nullptr;
        const hipError_t e = static_scratch(&p);
        if (e != hipSuccess) return fail_hip(e, "sdpa: resolving the static split-KV buffer");
        m.workspace = p;
        m.workspace_bytes = kStaticScratchBytes;
    }
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, m, stream);
}

int fv_sdpa_block_causal_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                              int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d,
                              float scale, size_t block_tokens, size_t window, size_t sink,
                              void* stream) {
    MaskArgs m;
    m.mode = kMaskBlockCausal;
    m.block_tokens = block_tokens;
    m.window = window;
    m.sink = sink;
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, m, stream);
}

int fv_sdpa_vdn_window_bf16(const uint16_t* q, const uint16_t* k, const uint16_t* v, void* out,
                            int out_is_bf16, size_t bh, size_t sq, size_t sk, size_t d, float scale,
                            size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                            size_t radius, void* stream) {
    MaskArgs m;
    m.mode = kMaskVdnWindow;
    m.video_start = video_start;
    m.frame_tokens = frame_tokens;
    m.frames = frames;
    m.chunk = chunk;
    m.radius = radius;
    return flash_common(q, k, v, out, out_is_bf16, bh, sq, sk, d, scale, m, stream);
}

int fv_cast_f32_bf16_scaled(const float* x, uint16_t* y, size_t n, float mul, void* stream) {
    if (n == 0) return FV_OK;
    const size_t threads = (n + 3) / 4;
    const size_t blocks = (threads + 255) / 256;
    if (blocks > (size_t)INT_MAX) return decline("cast: too many elements for one launch");
    hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0,
                       (hipStream_t)stream, x, y, n, mul);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fail_hip(e, "cast_f32_bf16");
}

int fv_cast_f32_bf16(const float* x, uint16_t* y, size_t n, void* stream) {
    return fv_cast_f32_bf16_scaled(x, y, n, 1.0f, stream);
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
