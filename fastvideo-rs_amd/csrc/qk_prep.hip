// Producer and consumer either side of the SDPA call, for gfx950: q/k RMSNorm
// (+ interleaved RoPE) straight into BHSD, the value-head split, and the merge of
// the attention output back to [batch, seq, heads*d].
//
// Replaces the reference's qk_norm_rope_bhsd / split_heads_bhsd / merge_heads
// kernels (crates/fastvideo-cudarc/src/rt/kernels/core.cu:373-443, launched from
// rt/ops.rs:528-620) and its bf16 q/k kernel wan_qk_norm_rope16
// (wan/fuse.rs:527-561, rounding points rt/fuse/policy.rs:404-412).
//
// All three are HBM-bound scans. One wave owns one projection row: the row is read
// once from HBM in 16-byte lane chunks for the sum of squares (lane-strided partial
// sums, then a butterfly), read again from cache for the normalise / rotate pass and
// written as 16-byte chunks into its heads' planes. No LDS, no barriers.
#include <limits.h>

#include "../../include/fv_sdpa_hip.h"
#include "fv_common.h"
#include "fv_internal.h"

namespace fv {
namespace {

constexpr int kRowsPerBlock = 4;   // 256 threads = 4 waves = 4 rows

// 8 values to bf16 (RNE, v_cvt_pk_bf16_f32) as 4 packed words
FV_DEV u32x4 pack_bf16x8(const float (&r)[8]) {
    f32x8 f;
#pragma unroll
    for (int i = 0; i < 8; i++) f[i] = r[i];
    return __builtin_bit_cast(u32x4, __builtin_convertvector(f, bf16x8));
}
// round 8 values to bf16 and back to f32
FV_DEV void round_bf16x8(float (&r)[8]) {
    const u32x4 t = pack_bf16x8(r);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        r[2 * i] = __builtin_bit_cast(float, t[i] << 16);
        r[2 * i + 1] = __builtin_bit_cast(float, t[i] & 0xffff0000u);
    }
}

// 8 consecutive elements starting at element index j (multiple of 8) of a bf16 or f32 row
template <bool IS16>
FV_DEV void load8(const void* row, size_t j, float (&v)[8]) {
    if constexpr (IS16) {
        const u32x4 t = *reinterpret_cast<const u32x4*>((const unsigned short*)row + j);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = __builtin_bit_cast(float, t[i] << 16);
            v[2 * i + 1] = __builtin_bit_cast(float, t[i] & 0xffff0000u);
        }
    } else {
        const f32x4 a = *reinterpret_cast<const f32x4*>((const float*)row + j);
        const f32x4 b = *reinterpret_cast<const f32x4*>((const float*)row + j + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[i] = a[i];
            v[4 + i] = b[i];
        }
    }
}

FV_DEV float wave_sum(float x) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
    return x;
}

// ROUND16: the bf16 rounding points of the reference's bf16 q/k kernel,
// bf16(bf16(x*inv)*w), rotation in f32, one rounding, bf16 out. Otherwise the f32 op:
// x*inv*w, rotation, f32 out, no intermediate rounding. Products and sums are kept
// unfused so that every value is the one the host formula gives.
// NC > 0: the row fits NC 16-byte chunks per lane and stays in registers between the two
// passes (all loads of a row are in flight together). NC == 0: any width, second pass
// re-reads the row from cache.
template <bool X16, bool W16, bool ROUND16, int NC>
__global__ __launch_bounds__(256) void qk_norm_rope_bhsd_kernel(
    const void* __restrict__ src, const void* __restrict__ w, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, void* __restrict__ out, long rows, int seq, int heads, int d,
    long src_width, long col_off, float eps, float out_mul, const unsigned* __restrict__ row_map, long out_rows) {
#pragma clang fp contract(off)
    const int lane = threadIdx.x & 63;
    const long row = (long)blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;
    const long b = row / seq;
    const int s = (int)(row - b * seq);
    const int width = heads * d;
    const int chunks = width >> 3;
    const char* x = (const char*)src + (row * src_width + col_off) * (X16 ? 2 : 4);
    constexpr int NR = NC > 0 ? NC : 1;
    float xr[NR][8];

    float ss = 0.f;
    if constexpr (NC > 0) {
#pragma unroll
        for (int k = 0; k < NC; k++) {
            const int c = lane + 64 * k;
            if (c < chunks) load8<X16>(x, (size_t)c * 8, xr[k]);
        }
#pragma unroll
        for (int k = 0; k < NC; k++) {
            if (lane + 64 * k < chunks) {
#pragma unroll
                for (int i = 0; i < 8; i++) ss += xr[k][i] * xr[k][i];
            }
        }
    } else {
        for (int c = lane; c < chunks; c += 64) {
            load8<X16>(x, (size_t)c * 8, xr[0]);
#pragma unroll
            for (int i = 0; i < 8; i++) ss += xr[0][i] * xr[0][i];
        }
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / __builtin_sqrtf(ss / (float)width + eps);

    // row_map: the head planes are [out_rows, d] and token s lands in row row_map[s] (the VSA
    // tile-slot order); without it the planes are [seq, d] in token order.
    const size_t orow = row_map ? row_map[s] : (unsigned)s;
    if (orow >= (size_t)out_rows) return;   // a slot outside the plane: nothing is written
    const bool rope = cos_t != nullptr;
    // With d/8 dividing 64 every chunk of a lane sits at the same offset p inside its head,
    // so the lane's 8 cos / 8 sin values are loaded once per row instead of once per head.
    const bool same_p = (64 % (d >> 3)) == 0;
    float cs0[8], sn0[8];
    if (rope && same_p) {
        const int p0 = (lane * 8) % d;
        load8<false>(cos_t, (size_t)s * d + p0, cs0);
        load8<false>(sin_t, (size_t)s * d + p0, sn0);
    }
    auto emit = [&](int c, const float (&v)[8]) {
        const int j = c * 8;
        const int h = j / d, p = j - h * d;
        float wv[8], r[8];
        load8<W16>(w, (size_t)j, wv);
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = v[i] * inv;
        if (ROUND16) round_bf16x8(r);
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = r[i] * wv[i];
        if (ROUND16) round_bf16x8(r);
        if (rope) {
            float cs[8], sn[8];
            if (same_p) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    cs[i] = cs0[i];
                    sn[i] = sn0[i];
                }
            } else {
                load8<false>(cos_t, (size_t)s * d + p, cs);
                load8<false>(sin_t, (size_t)s * d + p, sn);
            }
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const float x1 = r[i], x2 = r[i + 1], cv = cs[i], sv = sn[i + 1];
                // f32 op: odd = x1*sn + x2*c (rt/ops.rs:2338); bf16 twin: odd = x2*c + x1*sn
                // (rt/fuse/host.rs:262): the same sum, operands in the order of the form restated
                r[i] = x1 * cv - x2 * sv;
                r[i + 1] = ROUND16 ? (x2 * cv + x1 * sv) : (x1 * sv + x2 * cv);
            }
        }
        // the caller's output factor (1 = none: x * 1.0f is x), before the one rounding of the rotated values
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = r[i] * out_mul;
        const size_t o = (((size_t)b * heads + h) * out_rows + orow) * d + p;
        if constexpr (ROUND16) {
            *reinterpret_cast<u32x4*>((unsigned short*)out + o) = pack_bf16x8(r);
        } else {
            f32x4 a = {r[0], r[1], r[2], r[3]}, bb = {r[4], r[5], r[6], r[7]};
            *reinterpret_cast<f32x4*>((float*)out + o) = a;
            *reinterpret_cast<f32x4*>((float*)out + o + 4) = bb;
        }
    };
    if constexpr (NC > 0) {
#pragma unroll
        for (int k = 0; k < NC; k++)
            if (lane + 64 * k < chunks) emit(lane + 64 * k, xr[k]);
    } else {
        for (int c = lane; c < chunks; c += 64) {
            load8<X16>(x, (size_t)c * 8, xr[0]);
            emit(c, xr[0]);
        }
    }
}

// Both permutes move 16-byte units; `du` = units per head row (d * elem / 16).
// split: out[((b*heads + h)*seq + s)*du + u] = src[(b*seq + s)*wu + cu + h*du + u]; with a row map
// the planes are [out_rows, du] and token s lands in row row_map[s].
__global__ __launch_bounds__(256) void split_heads_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ out,
                                                          size_t n, size_t seq, size_t heads, size_t du,
                                                          size_t wu, size_t cu,
                                                          const unsigned* __restrict__ row_map, size_t out_rows) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const size_t u = i % du;
    size_t t = i / du;
    const size_t s = t % seq;
    t /= seq;
    const size_t h = t % heads, b = t / heads;
    size_t o = i;
    if (row_map) {
        const size_t r = row_map[s];
        if (r >= out_rows) return;   // a slot outside the plane: nothing is written
        o = ((b * heads + h) * out_rows + r) * du + u;
    }
    out[o] = src[(b * seq + s) * wu + cu + h * du + u];
}

// merge: out[(b*seq + s)*heads*du + h*du + u] = src[((b*heads + h)*seq + s)*du + u]
__global__ __launch_bounds__(256) void merge_heads_kernel(const u32x4* __restrict__ src, u32x4* __restrict__ out,
                                                          size_t n, size_t seq, size_t heads, size_t du) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const size_t hd = heads * du;
    const size_t j = i % hd, row = i / hd;
    const size_t s = row % seq, b = row / seq;
    const size_t h = j / du, u = j - h * du;
    out[i] = src[((b * heads + h) * seq + s) * du + u];
}

template <bool X16, bool W16, bool R16, int NC>
void launch_qk_nc(dim3 grid, hipStream_t st, const void* src, const void* w, const float* cos_t,
                  const float* sin_t, void* out, long rows, int seq, int heads, int d, long src_width,
                  long col_off, float eps, float out_mul, const unsigned* row_map, long out_rows) {
    hipLaunchKernelGGL((qk_norm_rope_bhsd_kernel<X16, W16, R16, NC>), grid, dim3(256), 0, st, src, w, cos_t, sin_t,
                       out, rows, seq, heads, d, src_width, col_off, eps, out_mul, row_map, out_rows);
}

template <bool X16, bool W16, bool R16>
void launch_qk_r(const void* src, const void* w, const float* cos_t, const float* sin_t, void* out, long rows,
                 int seq, int heads, int d, long src_width, long col_off, float eps, float out_mul,
                 const unsigned* row_map, long out_rows, hipStream_t st) {
    const dim3 grid((unsigned)((rows + kRowsPerBlock - 1) / kRowsPerBlock));
    const int per_lane = (heads * d / 8 + 63) / 64;   // 16-byte chunks per lane
#define FV_QK_ARGS grid, st, src, w, cos_t, sin_t, out, rows, seq, heads, d, src_width, col_off, eps, out_mul, row_map, out_rows
    if (per_lane <= 2) launch_qk_nc<X16, W16, R16, 2>(FV_QK_ARGS);
    else if (per_lane <= 3) launch_qk_nc<X16, W16, R16, 3>(FV_QK_ARGS);        // 12 heads x 128
    else if (per_lane <= 6) launch_qk_nc<X16, W16, R16, 6>(FV_QK_ARGS);
    else if (per_lane <= 10) launch_qk_nc<X16, W16, R16, 10>(FV_QK_ARGS);      // 40 heads x 128
    else launch_qk_nc<X16, W16, R16, 0>(FV_QK_ARGS);
#undef FV_QK_ARGS
}

template <bool X16, bool W16>
hipError_t launch_qk(int round16, const void* src, const void* w, const float* cos_t, const float* sin_t,
                     void* out, long rows, int seq, int heads, int d, long src_width, long col_off,
                     float eps, float out_mul, const unsigned* row_map, long out_rows, hipStream_t st) {
    if (round16)
        launch_qk_r<X16, W16, true>(src, w, cos_t, sin_t, out, rows, seq, heads, d, src_width, col_off, eps, out_mul,
                                    row_map, out_rows, st);
    else
        launch_qk_r<X16, W16, false>(src, w, cos_t, sin_t, out, rows, seq, heads, d, src_width, col_off, eps, out_mul,
                                     row_map, out_rows, st);
    return hipGetLastError();
}

}  // namespace
}  // namespace fv

extern "C" {

static int qk_norm_rope_common(const void* src, int src_is_bf16, const void* w, int w_is_bf16,
                               const float* cos_t, const float* sin_t, void* out, int out_is_bf16,
                               size_t batch, size_t seq, size_t heads, size_t d, size_t src_width,
                               size_t col_off, float eps, float out_mul, const uint32_t* row_map, size_t out_rows,
                               void* stream) {
    if (!src || !w || !out) return fv_invalid("qk_norm_rope: null operand");
    if (!(out_mul == out_mul) || out_mul - out_mul != 0.0f) return fv_invalid("qk_norm_rope: out_mul must be finite");
    if ((cos_t == nullptr) != (sin_t == nullptr)) return fv_invalid("qk_norm_rope: one rope table without the other");
    if (batch == 0 || seq == 0) return FV_OK;
    if (heads == 0 || d == 0 || col_off + heads * d > src_width)
        return fv_invalid("qk_norm_rope: columns outside the projection");
    // 16-byte lane chunks: 8 elements, never straddling a head, aligned in the source row
    if (d % 8 != 0 || col_off % 8 != 0 || src_width % 8 != 0)
        return fv_decline("qk_norm_rope: d, col_off and src_width must be multiples of 8");
    if (batch * seq > (size_t)INT_MAX || seq > (size_t)INT_MAX || heads * d > (size_t)INT_MAX / 2 ||
        out_rows > (size_t)INT_MAX)
        return fv_decline("qk_norm_rope: too large for one launch");
    const long rows = (long)(batch * seq);
    hipStream_t st = (hipStream_t)stream;
    hipError_t e;
#define FV_QK_CALL(X16, W16)                                                                                  \
    fv::launch_qk<X16, W16>(out_is_bf16, src, w, cos_t, sin_t, out, rows, (int)seq, (int)heads, (int)d,        \
                            (long)src_width, (long)col_off, eps, out_mul, row_map, (long)out_rows, st)
    if (src_is_bf16 && w_is_bf16) e = FV_QK_CALL(true, true);
    else if (src_is_bf16) e = FV_QK_CALL(true, false);
    else if (w_is_bf16) e = FV_QK_CALL(false, true);
    else e = FV_QK_CALL(false, false);
#undef FV_QK_CALL
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "qk_norm_rope_bhsd");
}

int fv_qk_norm_rope_bhsd(const void* src, int src_is_bf16, const void* w, int w_is_bf16,
                         const float* cos_t, const float* sin_t, void* out, int out_is_bf16,
                         size_t batch, size_t seq, size_t heads, size_t d, size_t src_width,
                         size_t col_off, float eps, float out_mul, void* stream) {
    return qk_norm_rope_common(src, src_is_bf16, w, w_is_bf16, cos_t, sin_t, out, out_is_bf16, batch, seq, heads, d,
                               src_width, col_off, eps, out_mul, nullptr, seq, stream);
}

int fv_qk_norm_rope_tiles(const void* src, int src_is_bf16, const void* w, int w_is_bf16,
                          const float* cos_t, const float* sin_t, void* out, int out_is_bf16,
                          size_t batch, size_t seq, size_t heads, size_t d, size_t src_width,
                          size_t col_off, float eps, float out_mul, const uint32_t* token_slot, size_t padded,
                          void* stream) {
    if (!token_slot) return fv_invalid("qk_norm_rope_tiles: null token_slot");
    if (padded < seq) return fv_invalid("qk_norm_rope_tiles: padded < seq");
    return qk_norm_rope_common(src, src_is_bf16, w, w_is_bf16, cos_t, sin_t, out, out_is_bf16, batch, seq, heads, d,
                               src_width, col_off, eps, out_mul, token_slot, padded, stream);
}

static int split_heads_common(const void* src, void* out, int is_bf16, size_t batch, size_t seq, size_t heads,
                              size_t d, size_t src_width, size_t col_off, const uint32_t* row_map,
                              size_t out_rows, void* stream) {
    if (!src || !out) return fv_invalid("split_heads: null operand");
    if (col_off + heads * d > src_width) return fv_invalid("split_heads: columns outside the projection");
    const size_t per16 = is_bf16 ? 8 : 4;
    if (d % per16 != 0 || col_off % per16 != 0 || src_width % per16 != 0)
        return fv_decline("split_heads: d, col_off and src_width must be multiples of 16 bytes");
    const size_t du = d / per16, n = batch * heads * seq * du;
    if (n == 0) return FV_OK;
    const size_t blocks = (n + 255) / 256;
    if (blocks > (size_t)INT_MAX) return fv_decline("split_heads: too large for one launch");
    hipLaunchKernelGGL(fv::split_heads_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const fv::u32x4*)src, (fv::u32x4*)out, n, seq, heads, du, src_width / per16,
                       col_off / per16, row_map, out_rows);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "split_heads_bhsd");
}

int fv_split_heads_bhsd(const void* src, void* out, int is_bf16, size_t batch, size_t seq, size_t heads,
                        size_t d, size_t src_width, size_t col_off, void* stream) {
    return split_heads_common(src, out, is_bf16, batch, seq, heads, d, src_width, col_off, nullptr, seq, stream);
}

int fv_split_heads_tiles(const void* src, void* out, int is_bf16, size_t batch, size_t seq, size_t heads,
                         size_t d, size_t src_width, size_t col_off, const uint32_t* token_slot, size_t padded,
                         void* stream) {
    if (!token_slot) return fv_invalid("split_heads_tiles: null token_slot");
    if (padded < seq) return fv_invalid("split_heads_tiles: padded < seq");
    return split_heads_common(src, out, is_bf16, batch, seq, heads, d, src_width, col_off, token_slot, padded,
                              stream);
}

int fv_merge_heads(const void* src, void* out, int is_bf16, size_t batch, size_t heads, size_t seq, size_t d,
                   void* stream) {
    if (!src || !out) return fv_invalid("merge_heads: null operand");
    const size_t per16 = is_bf16 ? 8 : 4;
    if (d % per16 != 0) return fv_decline("merge_heads: d must be a multiple of 16 bytes");
    const size_t du = d / per16, n = batch * heads * seq * du;
    if (n == 0) return FV_OK;
    const size_t blocks = (n + 255) / 256;
    if (blocks > (size_t)INT_MAX) return fv_decline("merge_heads: too large for one launch");
    hipLaunchKernelGGL(fv::merge_heads_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                       (const fv::u32x4*)src, (fv::u32x4*)out, n, seq, heads, du);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "merge_heads");
}

}  // extern "C"
