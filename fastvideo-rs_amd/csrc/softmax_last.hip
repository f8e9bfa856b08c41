// Row softmax over a contiguous trailing axis: the reference's `softmax_last` / `softmax_last_bf16`
// (kernels/core.cu:177-252, launched from rt/ops.rs:377-401; host form rt/ops.rs:2178-2193), the
// step between the two GEMMs of its materialised-score attention (rt/attn.rs:748-865) and of the VSA
// coarse stage (rt/vsa.rs:385-394). The fused kernels of this library never materialise scores; this
// entry serves callers that hold a score matrix of their own.
//
// out[r, j] = exp(x[r, j] - max_j x[r, :]) * (1 / sum_j exp(x[r, j] - max)), f32 or bf16 (RNE) out.
//
// One row per group of WAVES waves: 1 wave for rows up to 1024 wide (4 rows per workgroup), the 4
// waves of a workgroup up to 16384, 16 waves (one 1024-thread workgroup) above. The first
// KEEP * 64 * WAVES elements of a row stay in registers between the three passes (KEEP = 16, or
// 64 for the 4-wave form above 4096, 32 for 16 waves), so rows up to 32768 wide are read from
// memory once; the tail of a wider row is re-read.
#include <limits.h>

#include "../../include/fv_sdpa_hip.h"
#include "fv_common.h"
#include "fv_internal.h"

namespace fv {
namespace {

FV_DEV float wave_max(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x = __builtin_fmaxf(x, __shfl_xor(x, o, 64));
    return x;
}
FV_DEV float wave_sum(float x) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) x += __shfl_xor(x, o, 64);
    return x;
}

// KEEP = row elements per thread held in registers
template <int WAVES, int KEEP, bool OUT16>
__global__ __launch_bounds__(WAVES == 16 ? 1024 : 256) void softmax_last_kernel(const float* x, void* out,
                                                                                 size_t rows, size_t width) {
    constexpr int NT = 64 * WAVES;                 // threads per row
    constexpr int RPB = WAVES == 1 ? 4 : 1;        // rows per workgroup
    __shared__ float red[2][WAVES];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rt = WAVES == 1 ? lane : tid;        // thread index within the row's group
    const size_t row = (size_t)blockIdx.x * RPB + (WAVES == 1 ? wave : 0);
    const bool row_ok = row < rows;                // whole waves only: no barrier is skipped below
    const float* src = x + (row_ok ? row : 0) * width;

    float keep[KEEP];
    float mx = neg_inf();
    if (row_ok) {
#pragma unroll
        for (int i = 0; i < KEEP; i++) {
            const size_t j = (size_t)rt + (size_t)i * NT;
            keep[i] = j < width ? src[j] : neg_inf();
            mx = __builtin_fmaxf(mx, keep[i]);
        }
        for (size_t j = (size_t)rt + (size_t)KEEP * NT; j < width; j += NT) mx = __builtin_fmaxf(mx, src[j]);
    }
    mx = wave_max(mx);
    if (WAVES > 1) {
        if (lane == 0) red[0][wave] = mx;
        __syncthreads();
        mx = red[0][0];
#pragma unroll
        for (int w = 1; w < WAVES; w++) mx = __builtin_fmaxf(mx, red[0][w]);
    }

    float sum = 0.f;
    if (row_ok) {
#pragma unroll
        for (int i = 0; i < KEEP; i++) {
            const size_t j = (size_t)rt + (size_t)i * NT;
            keep[i] = j < width ? expf(keep[i] - mx) : 0.f;
            sum += keep[i];
        }
        for (size_t j = (size_t)rt + (size_t)KEEP * NT; j < width; j += NT) sum += expf(src[j] - mx);
    }
    sum = wave_sum(sum);
    if (WAVES > 1) {
        if (lane == 0) red[1][wave] = sum;
        __syncthreads();
        float part[WAVES];
#pragma unroll
        for (int w = 0; w < WAVES; w++) part[w] = red[1][w];
#pragma unroll
        for (int n = WAVES / 2; n > 0; n >>= 1)
#pragma unroll
            for (int w = 0; w < n; w++) part[w] += part[w + n];
        sum = part[0];
    }
    if (!row_ok) return;

    const float inv = 1.0f / sum;
    float* o32 = (float*)out + row * width;
    unsigned short* o16 = (unsigned short*)out + row * width;
#pragma unroll
    for (int i = 0; i < KEEP; i++) {
        const size_t j = (size_t)rt + (size_t)i * NT;
        if (j < width) {
            const float p = keep[i] * inv;
            if (OUT16) o16[j] = bf16_rne_bits(p);
            else o32[j] = p;
        }
    }
    for (size_t j = (size_t)rt + (size_t)KEEP * NT; j < width; j += NT) {
        const float p = expf(src[j] - mx) * inv;
        if (OUT16) o16[j] = bf16_rne_bits(p);
        else o32[j] = p;
    }
}

template <int WAVES, int KEEP>
hipError_t launch_softmax(const float* x, void* out, int out_is_bf16, size_t rows, size_t width, hipStream_t st) {
    constexpr int RPB = WAVES == 1 ? 4 : 1;
    const dim3 block(WAVES == 16 ? 1024 : 256);
    const dim3 grid((unsigned)((rows + RPB - 1) / RPB));
    if (out_is_bf16)
        hipLaunchKernelGGL((softmax_last_kernel<WAVES, KEEP, true>), grid, block, 0, st, x, out, rows, width);
    else
        hipLaunchKernelGGL((softmax_last_kernel<WAVES, KEEP, false>), grid, block, 0, st, x, out, rows, width);
    return hipGetLastError();
}

}  // namespace
}  // namespace fv

extern "C" int fv_softmax_last(const float* x, void* out, int out_is_bf16, size_t rows, size_t width, void* stream) {
    if (rows == 0 || width == 0) return FV_OK;
    if (!x || !out) return fv_invalid("softmax_last: null operand");
    if (rows > (size_t)INT_MAX) return fv_decline("softmax_last: too many rows for one launch");
    if (x == out && out_is_bf16) return fv_invalid("softmax_last: the bf16 form cannot run in place");
    const hipStream_t st = (hipStream_t)stream;
    const hipError_t e = width <= 1024   ? fv::launch_softmax<1, 16>(x, out, out_is_bf16, rows, width, st)
                         : width <= 4096 ? fv::launch_softmax<4, 16>(x, out, out_is_bf16, rows, width, st)
                         : width <= 16384 ? fv::launch_softmax<4, 64>(x, out, out_is_bf16, rows, width, st)
                                         : fv::launch_softmax<16, 32>(x, out, out_is_bf16, rows, width, st);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "softmax_last");
}
