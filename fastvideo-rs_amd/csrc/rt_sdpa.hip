// rt::sdpa host layer over the gfx950 kernels + the device composed SDPA.
// See rt_sdpa.hpp for the reference citations.
#include "rt_sdpa.hpp"

#include <ctype.h>
#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <stdio.h>

#include <atomic>
#include <mutex>
#include <set>
#include <string>
#include <tuple>

#include "../../include/fv_sdpa_hip.h"
#include "fv_common.h"
#include "fv_internal.h"

// ---- composed SDPA on the device (rt/sdpa.rs:328-342) ----------------------------------
// softmax(scale * q k^T + mask) v in f32, one workgroup per query row, online
// softmax over chunks of 256 keys: the scalar form, for the head dims the f32 matrix-core kernel
// (composed_fwd.hip: 32 / 64 / 96 / 128) does not take.
namespace fv {

constexpr int kCompThreads = 256;

__global__ __launch_bounds__(kCompThreads) void sdpa_composed_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ mask, long mask_bh_stride, float* __restrict__ out, int sq, int sk,
    int d, float scale) {
#pragma clang fp contract(off)
    __shared__ float qs[256];
    __shared__ float ps[kCompThreads];
    __shared__ float red[4];
    __shared__ float accs[kCompThreads];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int qi = blockIdx.x;
    const long bh = blockIdx.y;
    const float* qr = q + (bh * sq + qi) * (long)d;
    const float* kb = k + bh * sk * (long)d;
    const float* vb = v + bh * sk * (long)d;
    const float* mr = mask ? mask + bh * mask_bh_stride + (long)qi * sk : nullptr;
    for (int c = tid; c < d; c += kCompThreads) qs[c] = qr[c];
    __syncthreads();
    const int parts = kCompThreads / d;       // threads per output column (d <= 256)
    const int col = tid % d, part = tid / d;
    const bool worker = part < parts;
    float m = neg_inf(), l = 0.f, acc = 0.f;
    for (int j0 = 0; j0 < sk; j0 += kCompThreads) {
        const int j = j0 + tid;
        float s = neg_inf();
        if (j < sk) {
            const float* kr = kb + (long)j * d;
            float dot = 0.f;
            for (int c = 0; c < d; c++) dot = dot + qs[c] * kr[c];
            s = dot * scale;
            if (mr) s = s + mr[j];
        }
        float cm = s;
        for (int off = 32; off > 0; off >>= 1) cm = fmaxf(cm, __shfl_xor(cm, off));
        if (lane == 0) red[wave] = cm;
        __syncthreads();
        const float m_new = fmaxf(m, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
        __syncthreads();
        const float alpha = (m == neg_inf()) ? 0.f : expf(m - m_new);
        const float p = (j < sk && m_new != neg_inf()) ? expf(s - m_new) : 0.f;
        ps[tid] = p;
        float cs = p;
        for (int off = 32; off > 0; off >>= 1) cs += __shfl_xor(cs, off);
        if (lane == 0) red[wave] = cs;
        __syncthreads();
        l = l * alpha + (red[0] + red[1] + red[2] + red[3]);
        m = m_new;
        acc *= alpha;
        if (worker) {
            const int n = min(kCompThreads, sk - j0);
            for (int jj = part; jj < n; jj += parts) acc += ps[jj] * vb[(long)(j0 + jj) * d + col];
        }
        __syncthreads();
    }
    accs[tid] = worker ? acc : 0.f;
    __syncthreads();
    if (tid < d) {
        float t = 0.f;
        for (int pt = 0; pt < parts; pt++) t += accs[pt * d + tid];
        out[(bh * sq + qi) * (long)d + tid] = l > 0.f ? t / l : 0.f;
    }
}

}  // namespace fv

extern "C" int fv_sdpa_composed_f32(const float* q, const float* k, const float* v, const float* mask,
                                    int mask_per_bh, float* out, size_t bh, size_t sq, size_t sk,
                                    size_t d, float scale, void* stream) {
    if (!q || !k || !v || !out) return fv_invalid("sdpa_composed: null operand");
    if (bh == 0 || sq == 0) return FV_OK;
    if (sk == 0) return fv_invalid("sdpa_composed: no keys");
    if (d == 0 || d > 256 || bh > 65535 || sq > (size_t)INT_MAX || sk > (size_t)INT_MAX)
        return fv_decline("sdpa_composed: needs 1 <= d <= 256, bh <= 65535, lengths < 2^31");
    // head dims 32 / 64 / 96 / 128: the f32 matrix-core kernel (composed_fwd.hip)
    const int rc = fv_internal_launch_composed_mfma(q, k, v, mask, mask_per_bh ? (long)(sq * sk) : 0L, out, bh, (int)sq,
                                                    (int)sk, (int)d, scale, (hipStream_t)stream);
    if (rc < 0) return fv_fail_hip((hipError_t)(-rc), "sdpa_composed_mfma_f32");
    if (rc == 1) return FV_OK;
    hipLaunchKernelGGL(fv::sdpa_composed_f32_kernel, dim3((unsigned)sq, (unsigned)bh), dim3(fv::kCompThreads), 0,
                       (hipStream_t)stream, q, k, v, mask, mask_per_bh ? (long)(sq * sk) : 0L, out, (int)sq,
                       (int)sk, (int)d, scale);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "sdpa_composed_f32");
}

// ---- rt layer -----------------------------------------------------------------------------
namespace fv::rt {

namespace {

TensorError msg(std::string s) { return TensorError{std::move(s)}; }

std::atomic<uint64_t> g_fused{0}, g_causal{0}, g_composed{0}, g_cast{0}, g_masks{0};
thread_local std::optional<bool> g_bf16_override;
thread_local std::optional<Backend> g_backend_override;
thread_local std::optional<bool> g_fold_override;

// rt/sdpa.rs:234-246 `retired`
std::string retired(Backend b) {
    if (b == Backend::Sparse)
        return "FASTVIDEO_SDPA=sparse (the host block-sparse window prototype) is retired: "
               "FASTVIDEO_VSA=1 selects video sparse attention on the device; unset FASTVIDEO_SDPA for "
               "dense attention";
    return "FASTVIDEO_SDPA=host (the host online-softmax attention) is retired: unset FASTVIDEO_SDPA "
           "for the dense default";
}

bool env_flag(const char* name, bool dflt) {
    const char* v = getenv(name);
    if (!v || !*v) return dflt;
    return !(strcmp(v, "0") == 0 || strcasecmp(v, "false") == 0 || strcasecmp(v, "off") == 0 ||
             strcasecmp(v, "no") == 0);
}

// rt/log.rs: FASTVIDEO_LOG unset / "1" / "info" = info, "2" / "debug" / "trace" / "verbose" = debug,
// "0" / "off" / "false" / "quiet" / "error" = quiet (trimmed, case-insensitive); read once.
int log_level_from(const char* v) {
    if (!v) return 1;
    std::string s(v);
    const size_t a = s.find_first_not_of(" \t\r\n"), b = s.find_last_not_of(" \t\r\n");
    s = a == std::string::npos ? std::string() : s.substr(a, b - a + 1);
    for (char& c : s) c = (char)tolower((unsigned char)c);
    if (s == "0" || s == "off" || s == "false" || s == "quiet" || s == "error") return 0;
    if (s == "2" || s == "debug" || s == "trace" || s == "verbose") return 2;
    return 1;
}
int log_level() {
    static const int level = log_level_from(getenv("FASTVIDEO_LOG"));
    return level;
}

// One "[fastvideo] sdpa: <kernel> B= H= Sq= Sk= D=" line on stderr the first time a (kernel, shape) pair
// runs (rt/attn.rs:306-310 logs its fused launches once; a shape is part of the key here so that a
// run's log shows every attention geometry it used). At most 256 distinct lines per process.
void log_first_use(const char* kernel, size_t b, size_t h, size_t sq, size_t sk, size_t d) {
    if (log_level() < 1) return;
    static std::mutex mu;
    static std::set<std::tuple<std::string, size_t, size_t, size_t, size_t, size_t>> seen;
    std::lock_guard<std::mutex> lock(mu);
    if (seen.size() >= 256 || !seen.emplace(kernel, b, h, sq, sk, d).second) return;
    fprintf(stderr, "[fastvideo] sdpa: %s B=%zu H=%zu Sq=%zu Sk=%zu D=%zu\n", kernel, b, h, sq, sk, d);
}

size_t elem_size(DType t) { return t == DType::F32 ? 4 : 2; }

std::string rc_message(int rc) {
    return std::string(fv_sdpa_last_error()) + " (rc " + std::to_string(rc) + ")";
}

// A bf16 view of `x`: `x` itself when it already is bf16, else a rounded copy in `tmp` (of x * mul: the
// product in f32, one rounding).
Result<const Tensor*> as_bf16(const Tensor& x, Tensor& tmp, hipStream_t st, float mul = 1.0f) {
    if (x.dtype == DType::Bf16) return &x;
    auto r = Tensor::alloc(x.shape, DType::Bf16, st);
    if (!is_ok(r)) return std::get<TensorError>(r);
    tmp = std::move(std::get<Tensor>(r));
    const int rc = fv_cast_f32_bf16_scaled((const float*)x.data, (uint16_t*)tmp.data, x.numel(), mul, st);
    if (rc != FV_OK) return TensorError{"cast_f32_bf16: " + rc_message(rc), rc < 0 ? -rc : 0};
    g_cast++;
    return &tmp;
}

Result<const Tensor*> as_f32(const Tensor& x, Tensor& tmp, hipStream_t st) {
    if (x.dtype == DType::F32) return &x;
    auto r = Tensor::alloc(x.shape, DType::F32, st);
    if (!is_ok(r)) return std::get<TensorError>(r);
    tmp = std::move(std::get<Tensor>(r));
    const int rc = fv_cast_bf16_f32((const uint16_t*)x.data, (float*)tmp.data, x.numel(), st);
    if (rc != FV_OK) return TensorError{"cast_bf16_f32: " + rc_message(rc), rc < 0 ? -rc : 0};
    g_cast++;
    return &tmp;
}

// rt/tensor.rs:428-443 `quantize_bf16` on a result.
Result<Tensor> quantized(Tensor&& x, hipStream_t st) {
    if (x.dtype == DType::Bf16) return std::move(x);
    Tensor tmp;
    auto r = as_bf16(x, tmp, st);
    if (!is_ok(r)) return std::get<TensorError>(r);
    return std::move(tmp);
}

struct Bhsd {
    size_t b, h, sq, sk, d;
};
// rt/attn.rs:44-54: k and v must be [b, h, sk, d] for the fused kernels.
std::optional<Bhsd> bhsd(const Tensor& q, const Tensor& k, const Tensor& v) {
    if (q.rank() != 4 || k.rank() != 4 || v.rank() != 4) return std::nullopt;
    const Bhsd s{q.shape[0], q.shape[1], q.shape[2], k.shape[2], q.shape[3]};
    const std::vector<size_t> want{s.b, s.h, s.sk, s.d};
    if (k.shape != want || v.shape != want) return std::nullopt;
    return s;
}

float default_scale(std::optional<float> scale, size_t d) {
    return scale ? *scale : 1.0f / sqrtf((float)d);
}

// A contiguous copy of a row window (what the reference's `narrow` always makes).
Result<Tensor> compact(const Tensor& x, hipStream_t st) {
    auto r = Tensor::alloc(x.shape, x.dtype, st);
    if (!is_ok(r)) return r;
    Tensor t = std::move(std::get<Tensor>(r));
    const size_t row = x.shape[3] * elem_size(x.dtype), planes = x.shape[0] * x.shape[1];
    if (planes && x.shape[2] && row) {
        const hipError_t e = hipMemcpy2DAsync(t.data, x.shape[2] * row, x.data, x.plane_rows * row, x.shape[2] * row,
                                              planes, hipMemcpyDeviceToDevice, st);
        if (e != hipSuccess)
            return TensorError{std::string("sdpa: compacting a row window: ") + hipGetErrorString(e), (int)e};
    }
    return std::move(t);
}

// One fused launch (dense, block-causal or VDN window); nullopt = the kernel declined.
Result<std::optional<Tensor>> fused(const Tensor& q, const Tensor& k, const Tensor& v,
                                    std::optional<float> scale, bool out_bf16,
                                    const BlockCausal* causal, hipStream_t st,
                                    const VdnWindow* window = nullptr) {
    const auto s = bhsd(q, k, v);
    if (!s || !fv_sdpa_supported(s->b, s->h, s->sq, s->sk, s->d)) return std::optional<Tensor>{};
    // f32 queries are rounded to bf16 here, once: with the fold switch on (off by default: the result then differs
    // from the reference's round-then-scale order by one rounding of q), of q * (scale * log2(e)), and the
    // kernel then runs at scale = ln 2, its form without the per-score multiply
    float sc = default_scale(scale, s->d);
    float q_mul = 1.0f;
    if (q.dtype == DType::F32 && fold_scale()) {
        const float c = sc * 1.4426950408889634f;
        if (c > 0.0f && c < 3.0e38f && !fv_sdpa_is_log2_domain_scale(sc)) {
            q_mul = c;
            sc = FV_SDPA_SCALE_LOG2_DOMAIN;
        }
    }
    Tensor tq, tk, tv;
    auto rq = as_bf16(q, tq, st, q_mul);
    if (!is_ok(rq)) return std::get<TensorError>(rq);
    auto rk = as_bf16(k, tk, st);
    if (!is_ok(rk)) return std::get<TensorError>(rk);
    auto rv = as_bf16(v, tv, st);
    if (!is_ok(rv)) return std::get<TensorError>(rv);
    auto ro = Tensor::alloc({s->b, s->h, s->sq, s->d}, out_bf16 ? DType::Bf16 : DType::F32, st);
    if (!is_ok(ro)) return std::get<TensorError>(ro);
    Tensor out = std::move(std::get<Tensor>(ro));
    const auto* pq = (const uint16_t*)std::get<const Tensor*>(rq)->data;
    const auto* pk = (const uint16_t*)std::get<const Tensor*>(rk)->data;
    const auto* pv = (const uint16_t*)std::get<const Tensor*>(rv)->data;
    int rc;
    if (causal)
        rc = fv_sdpa_block_causal_bf16(pq, pk, pv, out.data, out_bf16, s->b * s->h, s->sq, s->sk, s->d, sc,
                                       causal->block_tokens, causal->window, causal->sink, st);
    else if (window)
        rc = fv_sdpa_vdn_window_bf16(pq, pk, pv, out.data, out_bf16, s->b * s->h, s->sq, s->sk, s->d, sc,
                                     window->video_start, window->frame_tokens, window->frames, window->chunk,
                                     window->radius, st);
    else {
        // few query tiles against many keys: split the keys over more workgroups (fv_sdpa_splitkv_choose)
        const size_t splits = fv_sdpa_splitkv_choose(s->b * s->h, s->sq, s->sk);
        Tensor ws;
        if (splits > 1) {
            auto rw = Tensor::alloc({fv_sdpa_splitkv_workspace_bytes(s->b * s->h, s->sq, s->d, splits) / 4}, DType::F32, st);
            if (!is_ok(rw)) return std::get<TensorError>(rw);
            ws = std::move(std::get<Tensor>(rw));
            rc = fv_sdpa_dense_bf16_splitkv(pq, pk, pv, out.data, out_bf16, s->b * s->h, s->sq, s->sk, s->d, sc,
                                            q.plane_rows, k.plane_rows, v.plane_rows, splits, ws.data, ws.numel() * 4, st);
        } else if (q.strided() || k.strided() || v.strided()) {
            rc = fv_sdpa_dense_bf16_strided(pq, pk, pv, out.data, out_bf16, s->b * s->h, s->sq, s->sk, s->d, sc,
                                            q.plane_rows, k.plane_rows, v.plane_rows, st);
        } else {
            rc = fv_sdpa_dense_bf16(pq, pk, pv, out.data, out_bf16, s->b * s->h, s->sq, s->sk, s->d, sc, st);
        }
    }
    if (rc == FV_DECLINED) return std::optional<Tensor>{};
    if (rc != FV_OK) return TensorError{"sdpa: " + rc_message(rc), rc < 0 ? -rc : 0};
    ((causal || window) ? g_causal : g_fused)++;
    log_first_use(causal ? "fused mma block-causal" : window ? "fused mma vdn-window" : "fused mma", s->b, s->h, s->sq, s->sk,
                  s->d);
    return std::optional<Tensor>{std::move(out)};
}

// rt/sdpa.rs:184-233 `dense` / `run_step` over the collapsed route.
Result<Tensor> dense(const Tensor& q, const Tensor& k, const Tensor& v, std::optional<float> scale,
                     const Tensor* mask, hipStream_t st) {
    const bool act16 = bf16_activations();
    const Backend be = backend();
    bool composed_step = false;
    for (Step step : dense_route(Shape::of(q.shape, k.shape, v.shape), mask != nullptr, be)) {
        if (step == Step::Retired) return msg(retired(be));
        if (step == Step::Fused) {
            auto r = fused(q, k, v, scale, act16, nullptr, st);
            if (!is_ok(r)) return std::get<TensorError>(r);
            auto& o = std::get<std::optional<Tensor>>(r);
            if (o) return std::move(*o);
        }
        if (step == Step::Composed) composed_step = true;
    }
    if (!composed_step) return msg("sdpa: every kernel of the route declined");
    // Step::Composed on the bf16-rounded operands under bf16 activations
    Tensor tq, tk, tv;
    const Tensor *pq = &q, *pk = &k, *pv = &v;
    if (act16) {
        auto rq = as_bf16(q, tq, st);
        if (!is_ok(rq)) return std::get<TensorError>(rq);
        auto rk = as_bf16(k, tk, st);
        if (!is_ok(rk)) return std::get<TensorError>(rk);
        auto rv = as_bf16(v, tv, st);
        if (!is_ok(rv)) return std::get<TensorError>(rv);
        pq = std::get<const Tensor*>(rq);
        pk = std::get<const Tensor*>(rk);
        pv = std::get<const Tensor*>(rv);
    }
    auto out = sdpa_composed(*pq, *pk, *pv, scale, mask, st);
    if (!is_ok(out)) return out;
    if (act16) return quantized(std::move(std::get<Tensor>(out)), st);
    return out;
}

Result<Tensor> upload_mask(const std::vector<float>& host, size_t sq, size_t sk, hipStream_t st) {
    auto r = Tensor::alloc({1, 1, sq, sk}, DType::F32, st);
    if (!is_ok(r)) return r;
    Tensor t = std::move(std::get<Tensor>(r));
    hipError_t e = hipMemcpyAsync(t.data, host.data(), host.size() * 4, hipMemcpyHostToDevice, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);   // `host` dies with the caller's frame
    if (e != hipSuccess) return msg(std::string("sdpa: mask upload: ") + hipGetErrorString(e));
    g_masks++;
    return std::move(t);
}

// rt/sdpa.rs:248-269
Result<Tensor> block_causal(const Tensor& q, const Tensor& k, const Tensor& v, std::optional<float> scale,
                            BlockCausal mask, hipStream_t st) {
    const size_t sq = q.shape[2], sk = k.shape[2];
    if (causal_flash_enabled()) {
        auto r = fused(q, k, v, scale, bf16_activations(), &mask, st);
        if (!is_ok(r)) return std::get<TensorError>(r);
        auto& o = std::get<std::optional<Tensor>>(r);
        if (o) return std::move(*o);
    }
    auto m = upload_mask(mask.dense_mask(sq, sk), sq, sk, st);
    if (!is_ok(m)) return m;
    return dense(q, k, v, scale, &std::get<Tensor>(m), st);
}

// rt/sdpa.rs:271-298
Result<Tensor> vdn_window(const Tensor& q, const Tensor& k, const Tensor& v, std::optional<float> scale,
                          VdnWindow mask, hipStream_t st) {
    const size_t sq = q.shape[2], sk = k.shape[2];
    auto r = fused(q, k, v, scale, bf16_activations(), nullptr, st, &mask);
    if (!is_ok(r)) return std::get<TensorError>(r);
    auto& o = std::get<std::optional<Tensor>>(r);
    if (o) return std::move(*o);
    // The masked fallback materialises [sq, sk]: small (test) shapes only.
    if (sq != 0 && sk > ((size_t)1 << 26) / sq)
        return msg("sdpa_vdn_window: the window kernel cannot run this " + std::to_string(sq) + "x" +
                   std::to_string(sk) + " call and the dense mask is too large");
    auto m = upload_mask(mask.dense_mask(sq, sk), sq, sk, st);
    if (!is_ok(m)) return m;
    return dense(q, k, v, scale, &std::get<Tensor>(m), st);
}

// rt/sdpa.rs:300-324
Result<Tensor> kv_window(const Tensor& q, const Tensor& k, const Tensor& v, bool flash, hipStream_t st) {
    if (flash) return dense(q, k, v, std::nullopt, nullptr, st);
    const bool act16 = bf16_activations();
    Tensor tq, tk, tv;
    const Tensor *pq = &q, *pk = &k, *pv = &v;
    if (act16) {
        auto rq = as_bf16(q, tq, st);
        if (!is_ok(rq)) return std::get<TensorError>(rq);
        auto rk = as_bf16(k, tk, st);
        if (!is_ok(rk)) return std::get<TensorError>(rk);
        auto rv = as_bf16(v, tv, st);
        if (!is_ok(rv)) return std::get<TensorError>(rv);
        pq = std::get<const Tensor*>(rq);
        pk = std::get<const Tensor*>(rk);
        pv = std::get<const Tensor*>(rv);
    }
    auto out = sdpa_composed(*pq, *pk, *pv, std::nullopt, nullptr, st);
    if (!is_ok(out)) return out;
    if (act16) return quantized(std::move(std::get<Tensor>(out)), st);
    return out;
}

}  // namespace

// ---- Tensor --------------------------------------------------------------------------------

Tensor::Tensor(Tensor&& o) noexcept { *this = std::move(o); }
Tensor& Tensor::operator=(Tensor&& o) noexcept {
    if (this != &o) {
        if (owned_ && data) (void)hipFreeAsync(data, stream_);
        shape = std::move(o.shape);
        dtype = o.dtype;
        data = o.data;
        plane_rows = o.plane_rows;
        owned_ = o.owned_;
        stream_ = o.stream_;
        o.data = nullptr;
        o.owned_ = false;
    }
    return *this;
}
Tensor::~Tensor() {
    if (owned_ && data) (void)hipFreeAsync(data, stream_);
}
Tensor Tensor::borrowed(void* data, std::vector<size_t> shape, DType dtype) {
    Tensor t;
    t.data = data;
    t.shape = std::move(shape);
    t.dtype = dtype;
    return t;
}
Tensor Tensor::window(void* data, std::vector<size_t> shape, DType dtype, size_t plane_rows) {
    Tensor t = borrowed(data, std::move(shape), dtype);
    t.plane_rows = t.shape.size() == 4 && plane_rows != t.shape[2] ? plane_rows : 0;
    return t;
}
Result<Tensor> Tensor::alloc(std::vector<size_t> shape, DType dtype, hipStream_t stream) {
    Tensor t;
    t.shape = std::move(shape);
    t.dtype = dtype;
    const size_t bytes = (t.numel() ? t.numel() : 1) * elem_size(dtype);
    hipError_t e = hipMallocAsync(&t.data, bytes, stream);
    if (e != hipSuccess) {
        (void)hipGetLastError();   // the failed allocation is reported here, not by the next launch
        return TensorError{std::string("sdpa: device allocation failed: ") + hipGetErrorString(e), (int)e};
    }
    t.owned_ = true;
    t.stream_ = stream;
    return std::move(t);
}
size_t Tensor::numel() const {
    size_t n = 1;
    for (size_t s : shape) n *= s;
    return n;
}
void* Tensor::release() {
    void* p = data;
    data = nullptr;
    owned_ = false;
    return p;
}

// ---- BlockCausal ---------------------------------------------------------------------------

bool BlockCausal::allows(size_t q, size_t k) const {
    return fv_block_causal_allows(block_tokens, window, sink, q, k) != 0;
}
std::vector<float> BlockCausal::dense_mask(size_t sq, size_t sk) const {
    std::vector<float> m(sq * sk);
    fv_block_causal_dense_mask(block_tokens, window, sink, sq, sk, m.data());
    return m;
}

bool VdnWindow::allows(size_t q, size_t k) const {
    return fv_vdn_window_allows(video_start, frame_tokens, frames, chunk, radius, q, k) != 0;
}
std::vector<float> VdnWindow::dense_mask(size_t sq, size_t sk) const {
    std::vector<float> m(sq * sk);
    fv_vdn_window_dense_mask(video_start, frame_tokens, frames, chunk, radius, sq, sk, m.data());
    return m;
}

// ---- Plan ----------------------------------------------------------------------------------

Plan Plan::dense(std::optional<float> scale) { return masked(scale, nullptr); }
Plan Plan::masked(std::optional<float> scale, const Tensor* mask) {
    Plan p;
    p.kind = Kind::Dense;
    p.scale = scale;
    p.mask = mask;
    return p;
}
Plan Plan::fp8_first() const {
    Plan p = *this;
    if (p.kind == Kind::Dense && p.mask == nullptr) p.fp8_first_flag = true;
    return p;
}
Plan Plan::composed(std::optional<float> scale, const Tensor* mask) {
    Plan p;
    p.kind = Kind::Composed;
    p.scale = scale;
    p.mask = mask;
    return p;
}
Plan Plan::block_causal(std::optional<float> scale, BlockCausal mask) {
    Plan p;
    p.kind = Kind::BlockCausalK;
    p.scale = scale;
    p.causal = mask;
    return p;
}
Plan Plan::vdn_window(std::optional<float> scale, VdnWindow mask) {
    Plan p;
    p.kind = Kind::VdnWindowK;
    p.scale = scale;
    p.window = mask;
    return p;
}
Plan Plan::kv_window() {
    Plan p;
    p.kind = Kind::KvWindow;
    return p;
}
Plan Plan::kv_window_with(bool flash) {
    Plan p = kv_window();
    p.kv_flash = flash;
    return p;
}

// ---- settings --------------------------------------------------------------------------------

bool bf16_activations() {
    if (g_bf16_override) return *g_bf16_override;
    static const bool env = env_flag("FASTVIDEO_BF16_ACT", true);
    return env;
}
void set_bf16_activations_override(std::optional<bool> v) { g_bf16_override = v; }
bool causal_flash_enabled() {
    static const bool env = env_flag("FASTVIDEO_WAN_CAUSAL_FLASH", true);
    return env;
}
bool fold_scale() {
    if (g_fold_override) return *g_fold_override;
    static const bool env = env_flag("FASTVIDEO_SDPA_FOLD_SCALE", false);
    return env;
}
void set_fold_scale_override(std::optional<bool> v) { g_fold_override = v; }

Backend parse_backend(const std::string& v) {
    if (v == "cublas") return Backend::Cublas;
    if (v == "flash") return Backend::Flash;
    if (v == "host") return Backend::Host;
    if (v == "sparse") return Backend::Sparse;
    return Backend::Dense;
}
Backend backend() {
    if (g_backend_override) return *g_backend_override;
    static const Backend env = [] {
        const char* v = getenv("FASTVIDEO_SDPA");
        std::string s = v ? v : "dense";
        for (char& c : s) c = (char)tolower((unsigned char)c);
        return parse_backend(s);
    }();
    return env;
}
void set_backend_override(std::optional<Backend> v) { g_backend_override = v; }

Shape Shape::of(const std::vector<size_t>& q, const std::vector<size_t>& k, const std::vector<size_t>& v) {
    Shape s;
    s.sq = q.size() > 2 ? q[2] : 0;
    s.sk = k.size() > 2 ? k[2] : 0;
    if (q.size() == 4 && k.size() == 4 && k == std::vector<size_t>{q[0], q[1], k[2], q[3]} && v == k)
        s.dims = Dims{q[0], q[1], q[2], k[2], q[3]};
    return s;
}

std::vector<Step> dense_route(const Shape&, bool masked, Backend be) {
    std::vector<Step> route;
    if (!masked) {
        if (be == Backend::Host || be == Backend::Sparse) return {Step::Retired};
        if (be == Backend::Dense) route.push_back(Step::Fused);
    }
    route.push_back(Step::Composed);
    return route;
}

Stats stats_snapshot() {
    Stats s;
    s.fused_launches = g_fused;
    s.causal_launches = g_causal;
    s.composed_launches = g_composed;
    s.cast_launches = g_cast;
    s.masks_materialised = g_masks;
    return s;
}

// ---- entry points ----------------------------------------------------------------------------

Result<Tensor> sdpa_composed(const Tensor& q, const Tensor& k, const Tensor& v, std::optional<float> scale,
                             const Tensor* mask, hipStream_t st) {
    if (q.rank() != 4 || k.rank() != 4 || v.rank() != 4) return msg("sdpa expects BHSD");
    const size_t b = q.shape[0], h = q.shape[1], sq = q.shape[2], d = q.shape[3], sk = k.shape[2];
    // rt/tensor.rs:1655-1667: the matmuls need matching batch and inner dims
    if (k.shape[0] != b || k.shape[1] != h || k.shape[3] != d)
        return msg("matmul inner " + std::to_string(d) + " vs " + std::to_string(k.shape[3]));
    if (v.shape[0] != b || v.shape[1] != h || v.shape[2] != sk)
        return msg("matmul inner " + std::to_string(sk) + " vs " + std::to_string(v.shape[2]));
    if (v.shape[3] != d) return msg("sdpa: value head dim differs from the query head dim");
    int mask_per_bh = 0;
    Tensor tm;
    const Tensor* pm = nullptr;
    if (mask) {
        // additive [.., sq, sk], broadcast over batch*heads or one mask per (batch, head)
        const size_t r = mask->rank();
        if (r < 2 || mask->shape[r - 2] != sq || mask->shape[r - 1] != sk)
            return msg("sdpa: mask must be [.., sq, sk]");
        if (sq == 0) return Tensor::alloc({b, h, 0, d}, DType::F32, st);   // no query rows: an empty result
        if (sk == 0) return msg("sdpa: no keys");
        const size_t lead = mask->numel() / (sq * sk);
        if (lead == b * h && lead != 1) mask_per_bh = 1;
        else if (lead != 1) return msg("sdpa: mask batch must be 1 or batch*heads");
        auto rm = as_f32(*mask, tm, st);
        if (!is_ok(rm)) return std::get<TensorError>(rm);
        pm = std::get<const Tensor*>(rm);
    }
    Tensor tq, tk, tv;
    auto rq = as_f32(q, tq, st);
    if (!is_ok(rq)) return std::get<TensorError>(rq);
    auto rk = as_f32(k, tk, st);
    if (!is_ok(rk)) return std::get<TensorError>(rk);
    auto rv = as_f32(v, tv, st);
    if (!is_ok(rv)) return std::get<TensorError>(rv);
    auto ro = Tensor::alloc({b, h, sq, d}, DType::F32, st);
    if (!is_ok(ro)) return ro;
    Tensor out = std::move(std::get<Tensor>(ro));
    const int rc = fv_sdpa_composed_f32((const float*)std::get<const Tensor*>(rq)->data,
                                        (const float*)std::get<const Tensor*>(rk)->data,
                                        (const float*)std::get<const Tensor*>(rv)->data,
                                        pm ? (const float*)pm->data : nullptr, mask_per_bh, (float*)out.data, b * h,
                                        sq, sk, d, default_scale(scale, d), st);
    if (rc == FV_DECLINED) return msg("sdpa: every kernel of the route declined");
    if (rc != FV_OK) return TensorError{"sdpa: " + rc_message(rc), -rc};
    g_composed++;
    log_first_use(mask ? "composed f32 (masked)" : "composed f32", b, h, sq, sk, d);
    return std::move(out);
}

Result<Tensor> sdpa(const Tensor& q, const Tensor& k, const Tensor& v, const Plan& plan, hipStream_t st) {
    if (q.rank() != 4 || k.rank() != 4 || v.rank() != 4) return msg("sdpa expects BHSD");
    if (q.strided() || k.strided() || v.strided()) {
        // Row windows of longer planes (a KV cache read in place). The fused dense kernel takes bf16
        // windows as they are; every other path gets contiguous copies.
        const bool dense_like = (plan.kind == Plan::Kind::Dense && !plan.mask) ||
                                (plan.kind == Plan::Kind::KvWindow && plan.kv_flash.value_or(causal_flash_enabled()));
        const bool all16 = q.dtype == DType::Bf16 && k.dtype == DType::Bf16 && v.dtype == DType::Bf16;
        if (dense_like && all16 && backend() == Backend::Dense) {
            auto r = fused(q, k, v, plan.scale, bf16_activations(), nullptr, st);
            if (!is_ok(r)) return std::get<TensorError>(r);
            auto& o = std::get<std::optional<Tensor>>(r);
            if (o) return std::move(*o);
        }
        Tensor cq, ck, cv;
        const Tensor *pq = &q, *pk = &k, *pv = &v;
        for (auto [src, tmp, dst] : {std::tuple{&q, &cq, &pq}, std::tuple{&k, &ck, &pk}, std::tuple{&v, &cv, &pv}}) {
            if (!src->strided()) continue;
            auto r = compact(*src, st);
            if (!is_ok(r)) return std::get<TensorError>(r);
            *tmp = std::move(std::get<Tensor>(r));
            *dst = tmp;
        }
        return sdpa(*pq, *pk, *pv, plan, st);
    }
    switch (plan.kind) {
        case Plan::Kind::Dense:
            // fp8_first marks H3's FP8 QK^T attempt (rt/sdpa.rs:148-158); this library is bf16 only
            return dense(q, k, v, plan.scale, plan.mask, st);
        case Plan::Kind::Composed:
            return sdpa_composed(q, k, v, plan.scale, plan.mask, st);
        case Plan::Kind::BlockCausalK:
            return block_causal(q, k, v, plan.scale, plan.causal, st);
        case Plan::Kind::VdnWindowK:
            return vdn_window(q, k, v, plan.scale, plan.window, st);
        case Plan::Kind::KvWindow:
            return kv_window(q, k, v, plan.kv_flash.value_or(causal_flash_enabled()), st);
    }
    return msg("sdpa: unknown plan");
}

}  // namespace fv::rt

// ---- flat C ABI over the rt layer ---------------------------------------------------------------

extern "C" {

int fv_rt_sdpa(const fv_tensor* q, const fv_tensor* k, const fv_tensor* v, const fv_plan* plan, fv_tensor* out,
               void* stream) {
    using namespace fv::rt;
    if (!q || !k || !v || !plan || !out) return fv_invalid("fv_rt_sdpa: null argument");
    auto wrap = [](const fv_tensor* t) {
        std::vector<size_t> shape(t->shape, t->shape + (t->rank < 0 ? 0 : (t->rank > 8 ? 8 : t->rank)));
        return Tensor::window(t->data, std::move(shape), t->dtype ? DType::Bf16 : DType::F32, t->plane_rows);
    };
    for (const fv_tensor* t : {q, k, v})
        if (t->plane_rows != 0 && (t->rank != 4 || t->plane_rows < t->shape[2]))
            return fv_invalid("fv_rt_sdpa: plane_rows needs a rank-4 operand and plane_rows >= shape[2]");
    const Tensor tq = wrap(q), tk = wrap(k), tv = wrap(v);
    Tensor tmask;
    if (plan->mask) tmask = wrap(plan->mask);
    const std::optional<float> scale = plan->has_scale ? std::optional<float>(plan->scale) : std::nullopt;
    Plan p;
    switch (plan->kind) {
        case FV_PLAN_DENSE:
            p = Plan::masked(scale, plan->mask ? &tmask : nullptr);
            if (plan->fp8_first) p = p.fp8_first();
            break;
        case FV_PLAN_COMPOSED:
            p = Plan::composed(scale, plan->mask ? &tmask : nullptr);
            break;
        case FV_PLAN_BLOCK_CAUSAL:
            p = Plan::block_causal(scale, BlockCausal{plan->block_tokens, plan->window, plan->sink});
            break;
        case FV_PLAN_VDN_WINDOW:
            p = Plan::vdn_window(scale, VdnWindow{plan->video_start, plan->frame_tokens, plan->frames, plan->chunk,
                                                  plan->radius});
            break;
        case FV_PLAN_KV_WINDOW:
            p = plan->kv_flash < 0 ? Plan::kv_window() : Plan::kv_window_with(plan->kv_flash != 0);
            break;
        default:
            return fv_invalid("fv_rt_sdpa: unknown plan kind");
    }
    auto r = sdpa(tq, tk, tv, p, (hipStream_t)stream);
    if (!is_ok(r)) {
        // a refused argument is -hipErrorInvalidValue; an allocation or launch failure keeps its own code
        const TensorError& err = std::get<TensorError>(r);
        const int rc = fv_invalid(err.message.c_str());
        return err.hip_code > 0 ? -err.hip_code : rc;
    }
    Tensor& t = std::get<Tensor>(r);
    out->rank = (int)t.rank();
    for (size_t i = 0; i < t.rank() && i < 8; i++) out->shape[i] = t.shape[i];
    out->dtype = t.dtype == DType::Bf16 ? 1 : 0;
    out->plane_rows = 0;
    out->data = t.release();
    return FV_OK;
}

int fv_rt_free(void* p, void* stream) {
    if (!p) return FV_OK;
    hipError_t e = hipFreeAsync(p, (hipStream_t)stream);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "fv_rt_free");
}

void fv_rt_set_bf16_activations(int v) {
    fv::rt::set_bf16_activations_override(v < 0 ? std::nullopt : std::optional<bool>(v != 0));
}
int fv_rt_bf16_activations(void) { return fv::rt::bf16_activations() ? 1 : 0; }
void fv_rt_set_fold_scale(int v) {
    fv::rt::set_fold_scale_override(v < 0 ? std::nullopt : std::optional<bool>(v != 0));
}
int fv_rt_fold_scale(void) { return fv::rt::fold_scale() ? 1 : 0; }

int fv_rt_log_level(void) { return fv::rt::log_level(); }
int fv_rt_parse_log_level(const char* v) { return fv::rt::log_level_from(v); }

int fv_rt_parse_backend(const char* v) { return (int)fv::rt::parse_backend(v ? v : ""); }
int fv_rt_backend(void) { return (int)fv::rt::backend(); }
void fv_rt_set_backend(int v) {
    fv::rt::set_backend_override(v < 0 || v > 4 ? std::nullopt
                                                : std::optional<fv::rt::Backend>((fv::rt::Backend)v));
}
int fv_rt_dense_route(const size_t* q_shape, const size_t* k_shape, const size_t* v_shape, int masked,
                      int backend, int steps_out[4], size_t dims_out[5]) {
    using namespace fv::rt;
    if (!q_shape || !k_shape || !v_shape || !steps_out || backend < 0 || backend > 4) return -1;
    const Shape s = Shape::of({q_shape, q_shape + 4}, {k_shape, k_shape + 4}, {v_shape, v_shape + 4});
    if (dims_out) {
        const Dims d = s.dims.value_or(Dims{0, 0, 0, 0, 0});
        dims_out[0] = d.b, dims_out[1] = d.h, dims_out[2] = d.sq, dims_out[3] = d.sk, dims_out[4] = d.d;
    }
    const auto route = dense_route(s, masked != 0, (Backend)backend);
    for (size_t i = 0; i < route.size() && i < 4; i++) steps_out[i] = (int)route[i];
    return (int)route.size();
}

void fv_rt_stats(uint64_t out5[5]) {
    const auto s = fv::rt::stats_snapshot();
    out5[0] = s.fused_launches;
    out5[1] = s.causal_launches;
    out5[2] = s.composed_launches;
    out5[3] = s.cast_launches;
    out5[4] = s.masks_materialised;
}

}  // extern "C"
