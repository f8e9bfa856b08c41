// Measurement probes for the benchmark driver; not part of the product library and not linked into it.
//
// fv_probe_mfma_bf16: every wave issues v_mfma_f32_32x32x16_bf16 back to back on four independent
// accumulators with register operands (no LDS, no memory, no VALU work in the loop), two waves per
// SIMD: the rate the matrix pipes sustain on this machine with nothing else in their way. Run for
// a few microseconds it shows the pipe's issue rate at the clock the chip starts at; run for tens of
// milliseconds it shows the clock the chip holds under matrix load (power), which is the ceiling
// any MFMA-bound kernel of the library sees. pattern 0 feeds every MFMA the same small operands
// (few bits toggle between instructions); pattern 1 cycles four operand pairs of random sign,
// mantissa and exponent (2^-2 .. 2^0, the bit activity of N(0,1) data), which costs more power.
//
// fv_probe_copy_f32x4: out[i] = in[i] in 16-byte units, grid-stride: the HBM rate a plain stream gets.
//
// fv_probe_tile_dma: the load side of the block-sparse fine kernel alone. Workgroups of 2 waves with
// two 16 KB LDS buffers (4 workgroups per CU, as that kernel) stream 64-row x 256-byte tiles through
// global_load_lds_dwordx4, always one tile in flight behind the one being waited for, no arithmetic.
// The tiles come from the first `region_tiles` tiles of the source in a scattered order, so a small
// region measures the L2 -> LDS path and a large one the path from HBM.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../fv_common.h"
#include "../attn_core.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace {

constexpr int kMfmaPerIter = 16;

typedef __attribute__((ext_vector_type(8))) unsigned short u16x8;

__device__ __forceinline__ unsigned short random_bf16_bits(unsigned x) {
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    const unsigned sign = x & 1u, expo = 125u + ((x >> 1) % 3u), mant = (x >> 8) & 0x7fu;
    return (unsigned short)((sign << 15) | (expo << 7) | mant);
}

__global__ __launch_bounds__(256) void probe_mfma_bf16_kernel(float* sink, int iters) {
    const int l = threadIdx.x & 63;
    bf16x8 a, b;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        a[j] = (__bf16)(0.001f * (float)(l + j));
        b[j] = (__bf16)(0.002f * (float)(l - j));
    }
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; i++) c0[i] = c1[i] = c2[i] = c3[i] = 0.f;
#pragma unroll 1
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int u = 0; u < kMfmaPerIter / 4; u++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void probe_mfma_bf16_random_kernel(float* sink, int iters) {
    const unsigned t = blockIdx.x * 256 + threadIdx.x;
    bf16x8 a[4], b[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        u16x8 ua, ub;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            ua[j] = random_bf16_bits(t * 64u + s * 16u + j);
            ub[j] = random_bf16_bits(t * 64u + s * 16u + 8u + j);
        }
        a[s] = __builtin_bit_cast(bf16x8, ua);
        b[s] = __builtin_bit_cast(bf16x8, ub);
    }
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int i = 0; i < 16; i++) c0[i] = c1[i] = c2[i] = c3[i] = 0.f;
#pragma unroll 1
    for (int i = 0; i < iters; i++) {
#pragma unroll
        for (int u = 0; u < kMfmaPerIter / 4; u++) {
            c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u], b[u], c0, 0, 0, 0);
            c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + 1) & 3], b[(u + 2) & 3], c1, 0, 0, 0);
            c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + 2) & 3], b[(u + 3) & 3], c2, 0, 0, 0);
            c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[(u + 3) & 3], b[(u + 1) & 3], c3, 0, 0, 0);
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) s += c0[i] + c1[i] + c2[i] + c3[i];
    sink[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

__global__ __launch_bounds__(256) void probe_copy_kernel(const f32x4* __restrict__ in, f32x4* __restrict__ out, size_t n16) {
    const size_t stride = (size_t)gridDim.x * 256;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) out[i] = in[i];
}

__global__ __launch_bounds__(128, 2) void probe_tile_dma_kernel(const uint16_t* src, unsigned region_tiles, int iters,
                                                                float* sink) {
    using namespace fv;
    extern __shared__ __attribute__((aligned(16))) unsigned char probe_smem[];
    lds_u8* kbuf = (lds_u8*)probe_smem;
    lds_u8* vbuf = kbuf + kTileBytes;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    TileDma<2, 128> dma;
    dma.init(wave, lane);
    unsigned t = (blockIdx.x * 2654435761u) % region_tiles;
    const unsigned step = 40503u % region_tiles + 1u;
    dma.template issue<false>(kbuf, src + (size_t)t * kTileRows * 128, kTileRows, wave);
#pragma unroll 1
    for (int i = 0; i < iters; i++) {
        t = (t + step) % region_tiles;
        dma.template issue<true>(vbuf, src + (size_t)t * kTileRows * 128, kTileRows, wave);
        wait_vmcnt<8>();    // the K tile landed; the V tile is in flight
        t = (t + step) % region_tiles;
        dma.template issue<false>(kbuf, src + (size_t)t * kTileRows * 128, kTileRows, wave);
        wait_vmcnt<8>();    // the V tile landed
    }
    wait_vmcnt<0>();
    __syncthreads();
    if (sink) sink[(size_t)blockIdx.x * 128 + tid] = (float)kbuf[16 * tid] + (float)vbuf[16 * tid];
}

}  // namespace

extern "C" {

// `blocks` workgroups, each streaming 2 * iters + 1 tiles of 16 KB out of the first region_tiles tiles
// of src (region_tiles * 16 KB readable bytes). Returns the bytes loaded through *bytes.
int fv_probe_tile_dma(const void* src, unsigned region_tiles, int blocks, int iters, float* sink, double* bytes,
                      void* stream) {
    if (!src || region_tiles == 0 || blocks <= 0 || iters <= 0) return -(int)hipErrorInvalidValue;
    if (((uintptr_t)src & 15) != 0) return -(int)hipErrorInvalidValue;
    hipLaunchKernelGGL(probe_tile_dma_kernel, dim3((unsigned)blocks), dim3(128), 40 * 1024 /* 4 workgroups per CU */, (hipStream_t)stream,
                       (const uint16_t*)src, region_tiles, iters, sink);
    if (bytes) *bytes = (double)fv::kTileBytes * (2.0 * iters + 1.0) * (double)blocks;
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : -(int)e;
}

// Launches `blocks` workgroups of 4 waves, each wave issuing 16 * iters MFMAs (32768 FLOP each).
// `sink` holds blocks * 256 floats; pattern 0 = constant operands, 1 = random. Returns the FLOP count of the launch through *flops, 0 or a
// negative hipError_t.
int fv_probe_mfma_bf16(float* sink, int blocks, int iters, int pattern, double* flops, void* stream) {
    if (!sink || blocks <= 0 || iters <= 0) return -(int)hipErrorInvalidValue;
    if (pattern)
        hipLaunchKernelGGL(probe_mfma_bf16_random_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, sink,
                           iters);
    else
        hipLaunchKernelGGL(probe_mfma_bf16_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, sink, iters);
    if (flops) *flops = 32768.0 * kMfmaPerIter * (double)iters * 4.0 * (double)blocks;
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : -(int)e;
}

// Copies n16 16-byte units with `blocks` workgroups.
int fv_probe_copy_f32x4(const void* in, void* out, size_t n16, int blocks, void* stream) {
    if (!in || !out || blocks <= 0) return -(int)hipErrorInvalidValue;
    if ((((uintptr_t)in | (uintptr_t)out) & 15) != 0) return -(int)hipErrorInvalidValue;
    hipLaunchKernelGGL(probe_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const f32x4*)in,
                       (f32x4*)out, n16);
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : -(int)e;
}

}  // extern "C"
