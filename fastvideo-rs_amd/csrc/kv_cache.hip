// The KV cache of causal Wan generation on the device (declarations and reference citations:
// kv_cache.hpp, include/fv_sdpa_hip.h).
#include "kv_cache.hpp"

#include <limits.h>

#include "../../include/fv_sdpa_hip.h"
#include "fv_common.h"
#include "fv_internal.h"

namespace fv {
namespace {

// dst[r, dst_off + i] = src[r, src_off + i] for r < rows, i < units (16-byte units; plane strides
// in units). Source and destination ranges of one launch never overlap.
__global__ __launch_bounds__(256) void kv_copy_rows_kernel(u32x4* __restrict__ dst, const u32x4* __restrict__ src,
                                                           size_t units, size_t dst_plane, size_t src_plane,
                                                           size_t dst_off, size_t src_off, size_t total) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
        const size_t r = i / units, u = i - r * units;
        dst[r * dst_plane + dst_off + u] = src[r * src_plane + src_off + u];
    }
}

// The same copy for a K and a V tensor in one launch (blockIdx.y picks the tensor): a cache write or a
// roll chunk moves both, and at these sizes a launch costs about what its copy does.
struct KvCopyArgs {
    u32x4* dst;
    const u32x4* src;
    size_t units, dst_plane, src_plane, dst_off, src_off, total;
};
__global__ __launch_bounds__(256) void kv_copy_rows_pair_kernel(KvCopyArgs a, KvCopyArgs b) {
    const KvCopyArgs& c = blockIdx.y == 0 ? a : b;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < c.total; i += (size_t)gridDim.x * 256) {
        const size_t r = i / c.units, u = i - r * c.units;
        c.dst[r * c.dst_plane + c.dst_off + u] = c.src[r * c.src_plane + c.src_off + u];
    }
}

// Interleaved RoPE on BHSD rows (kernels/core.cu:1933-1955 `apply_rotary_bshd` through
// wan/causal.rs:250-262 `rope_bhsd_f32`): pair (2i, 2i+1) of row r turns by the angle whose cos / sin
// sit in the EVEN slot 2i of the [s, d] tables; f32 arithmetic, products unfused, as the reference.
// One thread per 8 elements. Planes of x and out may be row windows of longer planes.
template <bool IN16, bool OUT16>
__global__ __launch_bounds__(256) void rope_bhsd_kernel(const void* __restrict__ x, size_t x_plane,
                                                        const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                        float sin_sign, void* __restrict__ out, size_t out_plane,
                                                        size_t s, size_t d, size_t total) {
#pragma clang fp contract(off)
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const size_t du = d >> 3, u = i % du, row = (i / du) % s, bh = i / (du * s);
    float v[8];
    if constexpr (IN16) {
        const u32x4 t = *reinterpret_cast<const u32x4*>((const uint16_t*)x + bh * x_plane + row * d + 8 * u);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[2 * j] = __builtin_bit_cast(float, t[j] << 16);
            v[2 * j + 1] = __builtin_bit_cast(float, t[j] & 0xffff0000u);
        }
    } else {
        const float* p = (const float*)x + bh * x_plane + row * d + 8 * u;
        const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
        for (int j = 0; j < 4; j++) v[j] = a[j], v[4 + j] = b[j];
    }
    const float* cp = cos_t + row * d + 8 * u;
    const float* sp = sin_t + row * d + 8 * u;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(cp), c1 = *reinterpret_cast<const f32x4*>(cp + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(sp), s1 = *reinterpret_cast<const f32x4*>(sp + 4);
    const float cs[4] = {c0[0], c0[2], c1[0], c1[2]};
    const float sn[4] = {s0[0] * sin_sign, s0[2] * sin_sign, s1[0] * sin_sign, s1[2] * sin_sign};
    float r[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float x1 = v[2 * j], x2 = v[2 * j + 1];
        r[2 * j] = x1 * cs[j] - x2 * sn[j];
        r[2 * j + 1] = x1 * sn[j] + x2 * cs[j];
    }
    if constexpr (OUT16) {
        u32x4 t;
#pragma unroll
        for (int j = 0; j < 4; j++) t[j] = bf16_rne_bits(r[2 * j]) | ((unsigned)bf16_rne_bits(r[2 * j + 1]) << 16);
        *reinterpret_cast<u32x4*>((uint16_t*)out + bh * out_plane + row * d + 8 * u) = t;
    } else {
        float* p = (float*)out + bh * out_plane + row * d + 8 * u;
        *reinterpret_cast<f32x4*>(p) = f32x4{r[0], r[1], r[2], r[3]};
        *reinterpret_cast<f32x4*>(p + 4) = f32x4{r[4], r[5], r[6], r[7]};
    }
}

}  // namespace
}  // namespace fv

namespace fv::rt {

namespace {
TensorError kv_msg(std::string s) { return TensorError{std::move(s)}; }
size_t esize(DType t) { return t == DType::F32 ? 4 : 2; }
}  // namespace

Result<KvMove> kv_plan(const KvSpec& s, size_t global_end, size_t local_end_prev, size_t current_start, size_t n) {
    const size_t current_end = current_start + n;
    if (!s.rolling && current_end > s.max_attention) {
        const size_t ft = s.frame_tokens ? s.frame_tokens : 1;
        return kv_msg("causal Wan local_attn_size=-1 keeps a " + std::to_string(s.max_attention / ft) +
                      "-frame KV window; got current_end=" + std::to_string(current_end) +
                      " tokens with frame_seqlen=" + std::to_string(s.frame_tokens) +
                      " (set local_attn_size for longer rollouts)");
    }
    if (current_end < global_end && current_end + local_end_prev < global_end)
        return kv_msg("causal kv: block before the cache start");
    const size_t advance = current_end > global_end ? current_end - global_end : 0;
    const size_t evicted =
        (s.rolling && current_end > global_end && n + local_end_prev > s.capacity) ? n + local_end_prev - s.capacity : 0;
    const size_t back = global_end > current_end ? global_end - current_end : 0;
    const size_t grown = local_end_prev + advance;
    if (grown < back || grown - back < evicted) return kv_msg("causal kv: pointer underflow");
    const size_t local_end = grown - back - evicted;
    if (local_end < n) return kv_msg("causal kv: block longer than the cache");
    if (local_end > (s.capacity > n ? s.capacity : n))
        return kv_msg("causal kv: write end " + std::to_string(local_end) + " past the cache (" +
                      std::to_string(s.capacity) + " tokens)");
    KvMove m;
    m.evicted = evicted;
    m.local_start = local_end - n;
    m.local_end = local_end;
    m.window_start = local_end > s.max_attention ? local_end - s.max_attention : 0;
    return m;
}

int kv_copy_tokens(void* dst, size_t dst_rows, size_t dst_off, const void* src, size_t src_rows, size_t src_off,
                   size_t len, size_t bh, size_t d, DType dtype, hipStream_t st) {
    if (!dst || !src) return fv_invalid("kv copy: null operand");
    if (dst_off + len > dst_rows || src_off + len > src_rows) return fv_invalid("kv copy: rows outside the buffers");
    if (len == 0 || bh == 0) return FV_OK;
    const size_t row_bytes = d * esize(dtype);
    if (row_bytes == 0 || row_bytes % 16 != 0 || (((uintptr_t)dst | (uintptr_t)src) & 15) != 0)
        return fv_decline("kv copy: rows must be 16-byte multiples at 16-byte aligned addresses");
    const size_t ru = row_bytes / 16, units = len * ru, total = units * bh;
    if (bh > (size_t)LONG_MAX / (units ? units : 1)) return fv_decline("kv copy: too large");
    const size_t blocks = std::min<size_t>((total + 255) / 256, 1u << 20);
    hipLaunchKernelGGL(fv::kv_copy_rows_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (fv::u32x4*)dst,
                       (const fv::u32x4*)src, units, dst_rows * ru, src_rows * ru, dst_off * ru, src_off * ru, total);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "kv_copy_rows");
}

namespace {
// Arguments of one tensor's copy, checked as kv_copy_tokens checks them. 0 = nothing to move.
int kv_copy_args(void* dst, size_t dst_rows, size_t dst_off, const void* src, size_t src_rows, size_t src_off,
                 size_t len, size_t bh, size_t d, DType dtype, fv::KvCopyArgs& out) {
    out = fv::KvCopyArgs{nullptr, nullptr, 1, 0, 0, 0, 0, 0};
    if (!dst || !src) return fv_invalid("kv copy: null operand");
    if (dst_off + len > dst_rows || src_off + len > src_rows) return fv_invalid("kv copy: rows outside the buffers");
    if (len == 0 || bh == 0) return FV_OK;
    const size_t row_bytes = d * esize(dtype);
    if (row_bytes == 0 || row_bytes % 16 != 0 || (((uintptr_t)dst | (uintptr_t)src) & 15) != 0)
        return fv_decline("kv copy: rows must be 16-byte multiples at 16-byte aligned addresses");
    const size_t ru = row_bytes / 16, units = len * ru;
    if (bh > (size_t)LONG_MAX / (units ? units : 1)) return fv_decline("kv copy: too large");
    out = fv::KvCopyArgs{(fv::u32x4*)dst, (const fv::u32x4*)src, units, dst_rows * ru, src_rows * ru, dst_off * ru,
                         src_off * ru, units * bh};
    return FV_OK;
}

// K and V of one cache write (or one roll chunk) in a single launch.
int kv_copy_tokens_pair(const fv::KvCopyArgs& a, const fv::KvCopyArgs& b, hipStream_t st) {
    const size_t most = std::max(a.total, b.total);
    if (most == 0) return FV_OK;
    const size_t blocks = std::min<size_t>((most + 255) / 256, 1u << 20);
    hipLaunchKernelGGL(fv::kv_copy_rows_pair_kernel, dim3((unsigned)blocks, 2), dim3(256), 0, st, a, b);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "kv_copy_rows_pair");
}

// The roll of K and V together: chunks no longer than the shift, so that no launch reads what it writes.
int kv_shift_pair_down(void* k, void* v, size_t rows, size_t from, size_t to, size_t len, size_t bh, size_t d, size_t dv,
                       DType kd, DType vd, hipStream_t st) {
    if (to >= from) return len == 0 || to == from ? FV_OK : fv_invalid("kv shift: tokens only move down");
    const size_t shift = from - to;
    for (size_t done = 0; done < len;) {
        const size_t n = std::min(shift, len - done);
        fv::KvCopyArgs a, b;
        int rc = kv_copy_args(k, rows, to + done, k, rows, from + done, n, bh, d, kd, a);
        if (rc == FV_OK) rc = kv_copy_args(v, rows, to + done, v, rows, from + done, n, bh, dv, vd, b);
        if (rc == FV_OK) rc = kv_copy_tokens_pair(a, b, st);
        if (rc != FV_OK) return rc;
        done += n;
    }
    return FV_OK;
}
}  // namespace

int kv_shift_tokens_down(void* t, size_t rows, size_t from, size_t to, size_t len, size_t bh, size_t d, DType dtype,
                         hipStream_t st) {
    if (to >= from) return len == 0 || to == from ? FV_OK : fv_invalid("kv shift: tokens only move down");
    const size_t shift = from - to;
    for (size_t done = 0; done < len;) {
        const size_t n = std::min(shift, len - done);
        const int rc = kv_copy_tokens(t, rows, to + done, t, rows, from + done, n, bh, d, dtype, st);
        if (rc != FV_OK) return rc;
        done += n;
    }
    return FV_OK;
}

int kv_rope_bhsd(const void* x, DType x_dtype, size_t x_rows, const float* cos_t, const float* sin_t,
                 bool negate_sin, void* out, DType out_dtype, size_t out_rows, size_t bh, size_t s, size_t d,
                 hipStream_t st) {
    if (!x || !cos_t || !sin_t || !out) return fv_invalid("rope_bhsd: null operand");
    if (x_rows < s || out_rows < s) return fv_invalid("rope_bhsd: plane rows below the row count");
    if (bh == 0 || s == 0) return FV_OK;
    if (d == 0 || d % 8 != 0) return fv_decline("rope_bhsd: head dim must be a multiple of 8");
    if ((((uintptr_t)x | (uintptr_t)out | (uintptr_t)cos_t | (uintptr_t)sin_t) & 15) != 0)
        return fv_invalid("rope_bhsd: operands must be 16-byte aligned");
    const size_t total = bh * s * (d / 8), blocks = (total + 255) / 256;
    if (blocks > (size_t)INT_MAX) return fv_decline("rope_bhsd: too large for one launch");
    const float sign = negate_sin ? -1.0f : 1.0f;
    const dim3 grid((unsigned)blocks), block(256);
    const bool i16 = x_dtype == DType::Bf16, o16 = out_dtype == DType::Bf16;
#define FV_ROPE(I, O)                                                                                             \
    hipLaunchKernelGGL((fv::rope_bhsd_kernel<I, O>), grid, block, 0, st, x, x_rows * d, cos_t, sin_t, sign, out, \
                       out_rows * d, s, d, total)
    if (i16 && o16) FV_ROPE(true, true);
    else if (i16) FV_ROPE(true, false);
    else if (o16) FV_ROPE(false, true);
    else FV_ROPE(false, false);
#undef FV_ROPE
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "rope_bhsd");
}

CausalKvCache::CausalKvCache(KvSpec s, size_t num_layers, bool static_mode)
    : spec(s), layers_(num_layers), static_mode_(static_mode) {}

CausalKvCache::~CausalKvCache() {
    for (auto& l : layers_) {
        if (l.k) (void)hipFree(l.k);
        if (l.v) (void)hipFree(l.v);
        if (l.raw_sink) (void)hipFree(l.raw_sink);
    }
}

void CausalKvCache::reset() {
    std::lock_guard<std::mutex> g(mu_);
    for (auto& l : layers_) {
        l.global_end = l.local_end = l.sink_at = 0;
        l.raw_valid = false;
    }
}

std::vector<KvPointers> CausalKvCache::pointers() const {
    std::lock_guard<std::mutex> g(mu_);
    std::vector<KvPointers> out;
    for (const auto& l : layers_) out.push_back(KvPointers{l.global_end, l.local_end, l.sink_at, l.raw_valid});
    return out;
}

Result<bool> CausalKvCache::set_pointers(const std::vector<KvPointers>& p) {
    std::lock_guard<std::mutex> g(mu_);
    if (!static_mode_ || p.size() != layers_.size())
        return kv_msg("causal kv: set_pointers needs a static cache and one entry per layer");
    for (size_t i = 0; i < p.size(); i++) {
        layers_[i].global_end = p[i].global_end;
        layers_[i].local_end = p[i].local_end;
        layers_[i].sink_at = p[i].sink_at;
        layers_[i].raw_valid = p[i].raw_valid;
    }
    return true;
}

Result<bool> CausalKvCache::advance(size_t current_start, size_t n, size_t sink_target) {
    std::lock_guard<std::mutex> g(mu_);
    if (!static_mode_) return kv_msg("causal kv: advance needs a static cache");
    // plan every layer first, so that an error leaves no layer moved
    std::vector<KvMove> moves;
    for (const Layer& L : layers_) {
        auto mv = kv_plan(spec, L.global_end, L.local_end, current_start, n);
        if (!is_ok(mv)) return std::get<TensorError>(mv);
        if (!L.k) return kv_msg("causal kv: advance over an unwritten cache");
        moves.push_back(std::get<KvMove>(mv));
    }
    for (size_t i = 0; i < layers_.size(); i++) {
        Layer& L = layers_[i];
        if (spec.rebase_sink && spec.sink > 0 && sink_target > 0 && L.sink_at != sink_target && L.local_end >= spec.sink) {
            L.raw_valid = true;
            L.sink_at = sink_target;
        }
        L.global_end = current_start + n;
        L.local_end = moves[i].local_end;
    }
    return true;
}

Result<CausalKvCache::BlockKey> CausalKvCache::block_key(size_t current_start, size_t n, size_t sink_target) const {
    std::lock_guard<std::mutex> g(mu_);
    KvPointers p{0, 0, 0, false};
    if (!layers_.empty()) p = KvPointers{layers_[0].global_end, layers_[0].local_end, layers_[0].sink_at, layers_[0].raw_valid};
    auto mv = kv_plan(spec, p.global_end, p.local_end, current_start, n);
    if (!is_ok(mv)) return std::get<TensorError>(mv);
    const bool rebase = spec.rebase_sink && spec.sink > 0 && sink_target > 0 && p.sink_at != sink_target &&
                        p.local_end >= spec.sink;
    return BlockKey{p.local_end, current_start + n > p.global_end, std::get<KvMove>(mv).evicted, rebase,
                    rebase && !p.raw_valid};
}

size_t CausalKvCache::bytes() const {
    std::lock_guard<std::mutex> g(mu_);
    size_t n = 0;
    for (const auto& l : layers_)
        if (l.k) n += l.b * l.h * (l.cap * (l.d * esize(l.kd) + l.dv * esize(l.vd)) + (l.raw_sink ? spec.sink * l.d * 4 : 0));
    return n;
}

// wan/causal.rs:540-560 `update` + 628-706 `update_static`
Result<std::pair<Tensor, Tensor>> CausalKvCache::update(size_t layer, const Tensor& k, const Tensor& v,
                                                        size_t current_start, hipStream_t st) {
    std::lock_guard<std::mutex> g(mu_);
    if (layer >= layers_.size()) return kv_msg("causal kv: no layer " + std::to_string(layer));
    if (k.rank() != 4) return kv_msg("causal kv: keys must be [b, h, n, d]");
    if (v.rank() != 4 || v.shape[0] != k.shape[0] || v.shape[1] != k.shape[1] || v.shape[2] != k.shape[2])
        return kv_msg("causal kv: keys and values differ in batch, heads or tokens");
    if (k.strided() || v.strided()) return kv_msg("causal kv: the block's keys and values must be contiguous");
    Layer& L = layers_[layer];
    const size_t b = k.shape[0], h = k.shape[1], n = k.shape[2], d = k.shape[3], dv = v.shape[3];
    auto plan = kv_plan(spec, L.global_end, L.local_end, current_start, n);
    if (!is_ok(plan)) return std::get<TensorError>(plan);
    const KvMove mv = std::get<KvMove>(plan);
    // wan/causal.rs:410-418 `guarded`: a recompute of cached frames leaves the sink slots alone
    size_t skip = 0;
    if (sink_guard_ && current_start > 0 && current_start + n <= L.global_end) {
        skip = spec.sink > mv.local_start ? spec.sink - mv.local_start : 0;
        if (skip > n) skip = n;
    }
    if (!static_mode_) return update_dynamic(L, mv, skip, k, v, current_start, st);
    if (!L.k) {
        const size_t cap = spec.capacity > n ? spec.capacity : n;
        if (b * h == 0 || cap == 0 || d == 0 || dv == 0) return kv_msg("causal kv: empty keys");
        hipError_t e = hipMalloc(&L.k, b * h * cap * d * esize(k.dtype));
        if (e == hipSuccess) e = hipMalloc(&L.v, b * h * cap * dv * esize(v.dtype));
        if (e == hipSuccess && spec.rebase_sink && spec.sink > 0)
            e = hipMalloc(&L.raw_sink, b * h * spec.sink * d * 4);   // f32, wan/causal.rs:650-655
        if (e != hipSuccess) {
            if (L.k) (void)hipFree(L.k);
            if (L.v) (void)hipFree(L.v);
            L.k = L.v = L.raw_sink = nullptr;
            return kv_msg(std::string("causal kv: allocating the layer's buffers: ") + hipGetErrorString(e));
        }
        L.b = b, L.h = h, L.cap = cap, L.d = d, L.dv = dv, L.kd = k.dtype, L.vd = v.dtype;
    }
    if (L.b != b || L.h != h || L.d != d || L.dv != dv || L.cap < n || L.kd != k.dtype || L.vd != v.dtype)
        return kv_msg("causal kv: static buffers [" + std::to_string(L.b) + ", " + std::to_string(L.h) + ", " +
                      std::to_string(L.cap) + ", " + std::to_string(L.d) + "] do not fit these keys");
    const size_t prev = L.local_end, bh = b * h;
    // roll: [0, sink) stays, [sink + evicted, prev) moves down to sink
    size_t valid = prev;
    if (mv.evicted > 0) {
        const size_t sink = std::min(spec.sink, prev);
        const size_t tail_start = std::min(sink + mv.evicted, prev), tail = prev - tail_start;
        if (tail > 0) {
            const int rc = kv_shift_pair_down(L.k, L.v, L.cap, tail_start, sink, tail, bh, d, dv, L.kd, L.vd, st);
            if (rc != FV_OK) return kv_msg(std::string("causal kv: roll: ") + fv_sdpa_last_error());
        }
        valid = sink + tail;
    }
    if (mv.local_start + skip > valid)
        return kv_msg("causal kv: write at " + std::to_string(mv.local_start + skip) + " leaves a gap after " +
                      std::to_string(valid) + " cached tokens");
    fv::KvCopyArgs ca, cb;
    int rc = kv_copy_args(L.k, L.cap, mv.local_start + skip, k.data, n, skip, n - skip, bh, d, L.kd, ca);
    if (rc == FV_OK) rc = kv_copy_args(L.v, L.cap, mv.local_start + skip, v.data, n, skip, n - skip, bh, dv, L.vd, cb);
    if (rc == FV_OK) rc = kv_copy_tokens_pair(ca, cb, st);
    if (rc != FV_OK) return kv_msg(std::string("causal kv: write: ") + fv_sdpa_last_error());
    L.global_end = current_start + n;
    L.local_end = mv.local_end;
    const size_t len = mv.local_end - mv.window_start;
    Tensor kw = Tensor::window((char*)L.k + mv.window_start * d * esize(L.kd), {b, h, len, d}, L.kd, L.cap);
    Tensor vw = Tensor::window((char*)L.v + mv.window_start * dv * esize(L.vd), {b, h, len, dv}, L.vd, L.cap);
    return std::make_pair(std::move(kw), std::move(vw));
}

// wan/causal.rs:556-624, the `new` (non-static) mode of `update`: the layer's K / V become
// cat(kept prefix, block) in new buffers of exactly local_end tokens; the roll is part of the copy
// ([0, sink) and [sink + evicted, prev) land back to back), everything after the block is dropped.
Result<std::pair<Tensor, Tensor>> CausalKvCache::update_dynamic(Layer& L, const KvMove& mv, size_t skip, const Tensor& k,
                                                                const Tensor& v, size_t current_start, hipStream_t st) {
    const size_t b = k.shape[0], h = k.shape[1], n = k.shape[2], d = k.shape[3], dv = v.shape[3], bh = b * h;
    if (bh == 0 || d == 0 || dv == 0 || mv.local_end == 0) return kv_msg("causal kv: empty keys");
    if (L.k && (L.b != b || L.h != h || L.d != d || L.dv != dv || L.kd != k.dtype || L.vd != v.dtype))
        return kv_msg("causal kv: keys [" + std::to_string(b) + ", " + std::to_string(h) + ", .., " + std::to_string(d) +
                      "] do not continue the cached [" + std::to_string(L.b) + ", " + std::to_string(L.h) + ", .., " +
                      std::to_string(L.d) + "]");
    const size_t prev = L.k ? L.local_end : 0, at = mv.local_start + skip, len_new = mv.local_end;
    // what survives of the old tokens, as (source start, count) pieces laid back to back from 0
    size_t piece_from[2] = {0, 0}, piece_len[2] = {prev, 0};
    if (mv.evicted > 0) {
        const size_t sink = std::min(spec.sink, prev), tail_start = std::min(sink + mv.evicted, prev);
        piece_len[0] = sink;
        piece_from[1] = tail_start;
        piece_len[1] = prev - tail_start;
    }
    if (at > piece_len[0] + piece_len[1]) {
        if (prev == 0) return kv_msg("causal kv: write past an empty cache");
        return kv_msg("causal kv: write at " + std::to_string(at) + " leaves a gap after " +
                      std::to_string(piece_len[0] + piece_len[1]) + " cached tokens");
    }
    void *nk = nullptr, *nv = nullptr;
    hipError_t e = hipMallocAsync(&nk, bh * len_new * d * esize(k.dtype), st);
    if (e == hipSuccess) e = hipMallocAsync(&nv, bh * len_new * dv * esize(v.dtype), st);
    if (e == hipSuccess && spec.rebase_sink && spec.sink > 0 && !L.raw_sink) e = hipMalloc(&L.raw_sink, bh * spec.sink * d * 4);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        if (nk) (void)hipFreeAsync(nk, st);
        if (nv) (void)hipFreeAsync(nv, st);
        return kv_msg(std::string("causal kv: allocating the layer's buffers: ") + hipGetErrorString(e));
    }
    int rc = FV_OK;
    size_t dst = 0;
    for (int p = 0; p < 2 && rc == FV_OK; p++) {
        const size_t take = std::min(piece_len[p], at - std::min(at, dst));   // the prefix ends at the write position
        if (take > 0) {
            rc = kv_copy_tokens(nk, len_new, dst, L.k, L.cap, piece_from[p], take, bh, d, k.dtype, st);
            if (rc == FV_OK) rc = kv_copy_tokens(nv, len_new, dst, L.v, L.cap, piece_from[p], take, bh, dv, v.dtype, st);
        }
        dst += take;
    }
    if (rc == FV_OK && n > skip) {
        rc = kv_copy_tokens(nk, len_new, at, k.data, n, skip, n - skip, bh, d, k.dtype, st);
        if (rc == FV_OK) rc = kv_copy_tokens(nv, len_new, at, v.data, n, skip, n - skip, bh, dv, v.dtype, st);
    }
    if (rc != FV_OK) {
        (void)hipFreeAsync(nk, st);
        (void)hipFreeAsync(nv, st);
        return kv_msg(std::string("causal kv: write: ") + fv_sdpa_last_error());
    }
    if (L.k) (void)hipFreeAsync(L.k, st);   // stream-ordered: the copies above have read them by then
    if (L.v) (void)hipFreeAsync(L.v, st);
    L.k = nk, L.v = nv;
    L.b = b, L.h = h, L.cap = len_new, L.d = d, L.dv = dv, L.kd = k.dtype, L.vd = v.dtype;
    L.global_end = current_start + n;
    L.local_end = len_new;
    const size_t len = len_new - mv.window_start;
    Tensor kw = Tensor::window((char*)L.k + mv.window_start * d * esize(L.kd), {b, h, len, d}, L.kd, L.cap);
    Tensor vw = Tensor::window((char*)L.v + mv.window_start * dv * esize(L.vd), {b, h, len, dv}, L.vd, L.cap);
    return std::make_pair(std::move(kw), std::move(vw));
}

// wan/causal.rs:739-776 `rebase_sink`, static mode
Result<bool> CausalKvCache::rebase_sink(size_t target, const float* orig_cos, const float* orig_sin,
                                        const float* new_cos, const float* new_sin, hipStream_t st) {
    std::lock_guard<std::mutex> g(mu_);
    const size_t sink = spec.sink;
    if (sink == 0) return false;
    if (!spec.rebase_sink) return kv_msg("causal kv: rebase_sink needs the rebased-sink RoPE policy");
    if (!orig_cos || !orig_sin || !new_cos || !new_sin) return kv_msg("causal kv: rebase_sink needs both table pairs");
    bool any = false;
    for (Layer& L : layers_) {
        if (L.sink_at == target || !L.k || L.local_end < sink) continue;
        if (!L.raw_sink) return kv_msg("causal kv: static rebased sink without its buffer");
        const size_t bh = L.b * L.h;
        int rc = FV_OK;
        if (!L.raw_valid)   // rotating back by the sink's own positions recovers the un-roped keys, kept f32
            rc = kv_rope_bhsd(L.k, L.kd, L.cap, orig_cos, orig_sin, true, L.raw_sink, DType::F32, sink, bh, sink, L.d, st);
        if (rc == FV_OK)
            rc = kv_rope_bhsd(L.raw_sink, DType::F32, sink, new_cos, new_sin, false, L.k, L.kd, L.cap, bh, sink, L.d, st);
        if (rc != FV_OK) return kv_msg(std::string("causal kv: rebase_sink: ") + fv_sdpa_last_error());
        L.raw_valid = true;
        L.sink_at = target;
        any = true;
    }
    return any;
}

}  // namespace fv::rt

// ---- flat C ABI -------------------------------------------------------------------------------

struct fv_kv_cache {
    fv::rt::CausalKvCache cache;
    fv_kv_cache(fv::rt::KvSpec s, size_t layers, bool static_mode) : cache(s, layers, static_mode) {}
};

extern "C" {

int fv_kv_plan(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens, int rolling,
               size_t global_end, size_t local_end_prev, size_t current_start, size_t n, size_t move_out[4]) {
    using namespace fv::rt;
    KvSpec s;
    s.capacity = capacity, s.sink = sink, s.max_attention = max_attention, s.frame_tokens = frame_tokens;
    s.rolling = rolling != 0;
    auto r = kv_plan(s, global_end, local_end_prev, current_start, n);
    if (!is_ok(r)) return fv_invalid(std::get<TensorError>(r).message.c_str());
    const KvMove m = std::get<KvMove>(r);
    if (move_out) move_out[0] = m.evicted, move_out[1] = m.local_start, move_out[2] = m.local_end, move_out[3] = m.window_start;
    return FV_OK;
}

int fv_kv_copy_tokens(void* dst, size_t dst_rows, size_t dst_off, const void* src, size_t src_rows, size_t src_off,
                      size_t len, size_t bh, size_t d, int is_bf16, void* stream) {
    return fv::rt::kv_copy_tokens(dst, dst_rows, dst_off, src, src_rows, src_off, len, bh, d,
                                  is_bf16 ? fv::rt::DType::Bf16 : fv::rt::DType::F32, (hipStream_t)stream);
}

int fv_kv_shift_tokens_down(void* t, size_t rows, size_t from, size_t to, size_t len, size_t bh, size_t d,
                            int is_bf16, void* stream) {
    if (!t) return fv_invalid("kv shift: null operand");
    if (from + len > rows) return fv_invalid("kv shift: rows outside the buffer");
    return fv::rt::kv_shift_tokens_down(t, rows, from, to, len, bh, d,
                                        is_bf16 ? fv::rt::DType::Bf16 : fv::rt::DType::F32, (hipStream_t)stream);
}

static fv_kv_cache* kv_cache_make(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens, int rolling,
                                  int rope_policy, size_t layers, bool static_mode) {
    fv::rt::KvSpec s;
    s.capacity = capacity, s.sink = sink, s.max_attention = max_attention, s.frame_tokens = frame_tokens;
    s.rolling = rolling != 0;
    s.relativistic = rope_policy == FV_KV_ROPE_RELATIVISTIC;
    s.rebase_sink = rope_policy == FV_KV_ROPE_REBASED_SINK && sink > 0;
    return new fv_kv_cache(s, layers, static_mode);
}
fv_kv_cache* fv_kv_cache_new(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens, int rolling,
                             int rope_policy, size_t layers) {
    return kv_cache_make(capacity, sink, max_attention, frame_tokens, rolling, rope_policy, layers, true);
}
fv_kv_cache* fv_kv_cache_new_dynamic(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens, int rolling,
                                     int rope_policy, size_t layers) {
    return kv_cache_make(capacity, sink, max_attention, frame_tokens, rolling, rope_policy, layers, false);
}
int fv_kv_cache_is_static(const fv_kv_cache* c) { return c && c->cache.is_static() ? 1 : 0; }

int fv_rope_bhsd(const void* x, int x_is_bf16, size_t x_rows, const float* cos_t, const float* sin_t, int negate_sin,
                 void* out, int out_is_bf16, size_t out_rows, size_t bh, size_t s, size_t d, void* stream) {
    using fv::rt::DType;
    return fv::rt::kv_rope_bhsd(x, x_is_bf16 ? DType::Bf16 : DType::F32, x_rows ? x_rows : s, cos_t, sin_t,
                                negate_sin != 0, out, out_is_bf16 ? DType::Bf16 : DType::F32, out_rows ? out_rows : s,
                                bh, s, d, (hipStream_t)stream);
}

int fv_kv_cache_rebase_sink(fv_kv_cache* c, size_t target, const float* orig_cos, const float* orig_sin,
                            const float* new_cos, const float* new_sin, void* stream) {
    if (!c) return fv_invalid("kv cache: null argument");
    auto r = c->cache.rebase_sink(target, orig_cos, orig_sin, new_cos, new_sin, (hipStream_t)stream);
    if (!fv::rt::is_ok(r)) return fv_invalid(std::get<fv::rt::TensorError>(r).message.c_str());
    return FV_OK;
}

void fv_kv_cache_free(fv_kv_cache* c) { delete c; }

void fv_kv_cache_reset(fv_kv_cache* c) {
    if (c) c->cache.reset();
}

void fv_kv_cache_set_sink_guard(fv_kv_cache* c, int on) {
    if (c) c->cache.set_sink_guard(on != 0);
}

int fv_kv_cache_pointers(const fv_kv_cache* c, size_t layer, size_t out4[4]) {
    if (!c || !out4) return fv_invalid("kv cache: null argument");
    const auto p = c->cache.pointers();
    if (layer >= p.size()) return fv_invalid("causal kv: no such layer");
    out4[0] = p[layer].global_end, out4[1] = p[layer].local_end, out4[2] = p[layer].sink_at;
    out4[3] = p[layer].raw_valid ? 1 : 0;
    return FV_OK;
}

int fv_kv_cache_set_pointers(fv_kv_cache* c, const size_t* in4, size_t layers) {
    if (!c || !in4) return fv_invalid("kv cache: null argument");
    std::vector<fv::rt::KvPointers> p(layers);
    for (size_t i = 0; i < layers; i++)
        p[i] = fv::rt::KvPointers{in4[4 * i], in4[4 * i + 1], in4[4 * i + 2], in4[4 * i + 3] != 0};
    auto r = c->cache.set_pointers(p);
    if (!fv::rt::is_ok(r)) return fv_invalid(std::get<fv::rt::TensorError>(r).message.c_str());
    return FV_OK;
}

int fv_kv_cache_advance(fv_kv_cache* c, size_t current_start, size_t n, size_t sink_target) {
    if (!c) return fv_invalid("kv cache: null argument");
    auto r = c->cache.advance(current_start, n, sink_target);
    if (!fv::rt::is_ok(r)) return fv_invalid(std::get<fv::rt::TensorError>(r).message.c_str());
    return FV_OK;
}

int fv_kv_cache_block_key(const fv_kv_cache* c, size_t current_start, size_t n, size_t sink_target, size_t out5[5]) {
    if (!c || !out5) return fv_invalid("kv cache: null argument");
    auto r = c->cache.block_key(current_start, n, sink_target);
    if (!fv::rt::is_ok(r)) return fv_invalid(std::get<fv::rt::TensorError>(r).message.c_str());
    const auto& k = std::get<fv::rt::CausalKvCache::BlockKey>(r);
    out5[0] = k.local_end, out5[1] = k.appends, out5[2] = k.evicted, out5[3] = k.rebase, out5[4] = k.take_raw;
    return FV_OK;
}

size_t fv_kv_cache_bytes(const fv_kv_cache* c) { return c ? c->cache.bytes() : 0; }

int fv_kv_cache_update(fv_kv_cache* c, size_t layer, const fv_tensor* k, const fv_tensor* v, size_t current_start,
                       fv_tensor* k_window, fv_tensor* v_window, void* stream) {
    using namespace fv::rt;
    if (!c || !k || !v || !k_window || !v_window) return fv_invalid("kv cache: null argument");
    auto wrap = [](const fv_tensor* t) {
        std::vector<size_t> shape(t->shape, t->shape + (t->rank < 0 ? 0 : (t->rank > 8 ? 8 : t->rank)));
        return Tensor::window(t->data, std::move(shape), t->dtype ? DType::Bf16 : DType::F32, t->plane_rows);
    };
    const Tensor tk = wrap(k), tv = wrap(v);
    auto r = c->cache.update(layer, tk, tv, current_start, (hipStream_t)stream);
    if (!is_ok(r)) return fv_invalid(std::get<TensorError>(r).message.c_str());
    auto& kv = std::get<std::pair<Tensor, Tensor>>(r);
    auto put = [](const Tensor& t, fv_tensor* o) {
        o->data = t.data;
        o->dtype = t.dtype == DType::Bf16 ? 1 : 0;
        o->rank = (int)t.rank();
        for (size_t i = 0; i < t.rank() && i < 8; i++) o->shape[i] = t.shape[i];
        o->plane_rows = t.plane_rows;
    };
    put(kv.first, k_window);
    put(kv.second, v_window);
    return FV_OK;
}

}  // extern "C"
