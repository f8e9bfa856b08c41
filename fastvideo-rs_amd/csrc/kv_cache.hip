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

CausalKvCache::CausalKvCache(KvSpec s, size_t num_layers) : spec(s), layers_(num_layers) {}

CausalKvCache::~CausalKvCache() {
    for (auto& l : layers_) {
        if (l.k) (void)hipFree(l.k);
        if (l.v) (void)hipFree(l.v);
    }
}

void CausalKvCache::reset() {
    std::lock_guard<std::mutex> g(mu_);
    for (auto& l : layers_) l.global_end = l.local_end = 0;
}

std::vector<KvPointers> CausalKvCache::pointers() const {
    std::lock_guard<std::mutex> g(mu_);
    std::vector<KvPointers> out;
    for (const auto& l : layers_) out.push_back(KvPointers{l.global_end, l.local_end});
    return out;
}

size_t CausalKvCache::bytes() const {
    std::lock_guard<std::mutex> g(mu_);
    size_t n = 0;
    for (const auto& l : layers_)
        if (l.k) n += l.b * l.h * l.cap * (l.d * esize(l.kd) + l.dv * esize(l.vd));
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
    if (!L.k) {
        const size_t cap = spec.capacity > n ? spec.capacity : n;
        if (b * h == 0 || cap == 0 || d == 0 || dv == 0) return kv_msg("causal kv: empty keys");
        hipError_t e = hipMalloc(&L.k, b * h * cap * d * esize(k.dtype));
        if (e == hipSuccess) e = hipMalloc(&L.v, b * h * cap * dv * esize(v.dtype));
        if (e != hipSuccess) {
            if (L.k) (void)hipFree(L.k);
            L.k = L.v = nullptr;
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
            int rc = kv_shift_tokens_down(L.k, L.cap, tail_start, sink, tail, bh, d, L.kd, st);
            if (rc == FV_OK) rc = kv_shift_tokens_down(L.v, L.cap, tail_start, sink, tail, bh, dv, L.vd, st);
            if (rc != FV_OK) return kv_msg(std::string("causal kv: roll: ") + fv_sdpa_last_error());
        }
        valid = sink + tail;
    }
    if (mv.local_start + skip > valid)
        return kv_msg("causal kv: write at " + std::to_string(mv.local_start + skip) + " leaves a gap after " +
                      std::to_string(valid) + " cached tokens");
    int rc = kv_copy_tokens(L.k, L.cap, mv.local_start + skip, k.data, n, skip, n - skip, bh, d, L.kd, st);
    if (rc == FV_OK) rc = kv_copy_tokens(L.v, L.cap, mv.local_start + skip, v.data, n, skip, n - skip, bh, dv, L.vd, st);
    if (rc != FV_OK) return kv_msg(std::string("causal kv: write: ") + fv_sdpa_last_error());
    L.global_end = current_start + n;
    L.local_end = mv.local_end;
    const size_t len = mv.local_end - mv.window_start;
    Tensor kw = Tensor::window((char*)L.k + mv.window_start * d * esize(L.kd), {b, h, len, d}, L.kd, L.cap);
    Tensor vw = Tensor::window((char*)L.v + mv.window_start * dv * esize(L.vd), {b, h, len, dv}, L.vd, L.cap);
    return std::make_pair(std::move(kw), std::move(vw));
}

}  // namespace fv::rt

// ---- flat C ABI -------------------------------------------------------------------------------

struct fv_kv_cache {
    fv::rt::CausalKvCache cache;
    fv_kv_cache(fv::rt::KvSpec s, size_t layers) : cache(s, layers) {}
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

fv_kv_cache* fv_kv_cache_new(size_t capacity, size_t sink, size_t max_attention, size_t frame_tokens, int rolling,
                             size_t layers) {
    fv::rt::KvSpec s;
    s.capacity = capacity, s.sink = sink, s.max_attention = max_attention, s.frame_tokens = frame_tokens;
    s.rolling = rolling != 0;
    return new fv_kv_cache(s, layers);
}

void fv_kv_cache_free(fv_kv_cache* c) { delete c; }

void fv_kv_cache_reset(fv_kv_cache* c) {
    if (c) c->cache.reset();
}

void fv_kv_cache_set_sink_guard(fv_kv_cache* c, int on) {
    if (c) c->cache.set_sink_guard(on != 0);
}

int fv_kv_cache_pointers(const fv_kv_cache* c, size_t layer, size_t out2[2]) {
    if (!c || !out2) return fv_invalid("kv cache: null argument");
    const auto p = c->cache.pointers();
    if (layer >= p.size()) return fv_invalid("causal kv: no such layer");
    out2[0] = p[layer].global_end, out2[1] = p[layer].local_end;
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
