// Composed SDPA in f32 on the matrix cores: softmax(scale * q k^T + mask) v with every operand,
// product and accumulation in fp32 (v_mfma_f32_32x32x2_f32), the path of the plans the reference
// runs through its composed tensor ops (rt/sdpa.rs:328-342: masked calls, Plan::composed, the
// block-causal / KV-window fallbacks, FASTVIDEO_SDPA=cublas) — there materialised scores through
// cuBLAS f32 (rt/attn.rs:748-865), here an online softmax over 32-key tiles, so no [bh, sq, sk]
// buffer exists. Head dims 32 / 64 / 96 / 128; other head dims keep the scalar kernel of rt_sdpa.hip.
//
// One workgroup = 4 waves x 32 queries. K and V tiles of 32 keys go global -> registers -> LDS
// (double buffered: the loads of tile t+1 are in flight under the arithmetic of tile t, one barrier
// per tile); 2 workgroups share a CU, so one wave's softmax runs under the other's MFMAs.
//
//   S^T (32 keys x 32 queries) = K Q^T     A = K[key = l%32][k], B = Q[query = l%32][k]; the MFMA's
//                                          two k slots (lane halves) take d = j and d = j + D/2, so a
//                                          lane's K operands of 4 consecutive steps are one 16-byte read
//   C layout                               lane l, register i: query l%32, key 8*(i/4) + 4*(l/32) + i%4
//   O^T (D x 32 queries) += V^T P^T        step i takes register i of both halves as the two key slots;
//                                          A = V[that key][32*db + l%32]
//
// LDS rows are padded (K: D + 4 floats, V: D + 8) so that both read patterns spread over all banks.
#include <limits.h>

#include "../../include/fv_sdpa_hip.h"
#include "fv_common.h"
#include "fv_internal.h"

namespace fv {
namespace {

constexpr int kCQ = 128;   // queries per workgroup
constexpr int kCK = 32;    // keys per tile

FV_DEV f32x16 mfma32_f32(float a, float b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

template <int D>
__global__ __launch_bounds__(256, 2) void sdpa_composed_mfma_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ mask, long mask_bh_stride, float* __restrict__ out, int sq, int sk, float scale) {
    constexpr int RK = D + 4, RV = D + 8;          // padded LDS row lengths (floats)
    constexpr int kUnits = D / 32;                  // 16-byte units per thread and tile
    constexpr int kNO = D / 32;
    extern __shared__ __attribute__((aligned(16))) float csm[];
    // buffers b = 0, 1: K at csm + b * kKT, V at csm + 2 * kKT + b * kVT (offsets, so that the compiler
    // keeps every access in the LDS address space)
    constexpr int kKT = kCK * RK, kVT = kCK * RV;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h = lane >> 5, c32 = lane & 31;
    const long bh = blockIdx.y;
    const int q0 = blockIdx.x * kCQ;
    const int qi = q0 + wave * 32 + c32;            // this lane's query
    const bool q_ok = qi < sq;
    const float NEG = neg_inf();
    const float* kb = k + bh * sk * (long)D;
    const float* vb = v + bh * sk * (long)D;
    const float* mr = mask ? mask + bh * mask_bh_stride + (long)(q_ok ? qi : 0) * sk : nullptr;

    // Q operand: this lane's query, d = h*D/2 + j for step j
    float qr[D / 2];
    {
        const float* src = q + (bh * sq + (q_ok ? qi : 0)) * (long)D + h * (D / 2);
#pragma unroll
        for (int j = 0; j < D / 2; j += 4) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (q_ok) t = *reinterpret_cast<const f32x4*>(src + j);
#pragma unroll
            for (int x = 0; x < 4; x++) qr[j + x] = t[x];
        }
    }

    // tile loads: thread t owns 16-byte units t + 256 r of the [32][D] tile
    f32x4 kreg[kUnits], vreg[kUnits];
    auto load_tile = [&](int kv0) {
#pragma unroll
        for (int r = 0; r < kUnits; r++) {
            const int u = tid + 256 * r, row = u / (D / 4), c4 = u % (D / 4);
            const f32x4 z = {0.f, 0.f, 0.f, 0.f};
            kreg[r] = vreg[r] = z;
            if (kv0 + row < sk) {
                kreg[r] = *reinterpret_cast<const f32x4*>(kb + (long)(kv0 + row) * D + 4 * c4);
                vreg[r] = *reinterpret_cast<const f32x4*>(vb + (long)(kv0 + row) * D + 4 * c4);
            }
        }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
        for (int r = 0; r < kUnits; r++) {
            const int u = tid + 256 * r, row = u / (D / 4), c4 = u % (D / 4);
            *reinterpret_cast<f32x4*>(csm + buf * kKT + row * RK + 4 * c4) = kreg[r];
            *reinterpret_cast<f32x4*>(csm + 2 * kKT + buf * kVT + row * RV + 4 * c4) = vreg[r];
        }
    };

    f32x16 o[kNO];
#pragma unroll
    for (int db = 0; db < kNO; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    float m_run = NEG, l_run = 0.f;

    const int nt = (sk + kCK - 1) / kCK;
    load_tile(0);
    store_tile(0);
    __syncthreads();
#pragma unroll 1
    for (int t = 0; t < nt; t++) {
        const int kv0 = t * kCK, buf = t & 1;
        if (t + 1 < nt) load_tile(kv0 + kCK);      // in flight under this tile's arithmetic
        // ---- S^T = K Q^T ----
        f32x16 s;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.f;
        const float* krow = csm + buf * kKT + c32 * RK + h * (D / 2);
#pragma unroll
        for (int j = 0; j < D / 2; j += 4) {
            const f32x4 a = *reinterpret_cast<const f32x4*>(krow + j);
#pragma unroll
            for (int x = 0; x < 4; x++) s = mfma32_f32(a[x], qr[j + x], s);
        }
        // ---- scale, mask, online softmax (per lane = per query; halves exchange max and sum) ----
        {
#pragma clang fp contract(off)
            float mx = NEG;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const int key = kv0 + 8 * (i >> 2) + 4 * h + (i & 3);
                float sv = s[i] * scale;
                if (mr && key < sk) sv = sv + mr[key];
                if (key >= sk) sv = NEG;
                s[i] = sv;
                mx = __builtin_fmaxf(mx, sv);
            }
            mx = pair_max(mx);
            const float m_new = __builtin_fmaxf(m_run, mx);
            const float alpha = (m_run == NEG) ? 0.f : fast_exp2((m_run - m_new) * 1.4426950408889634f);
            float ls = 0.f;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float p = (m_new == NEG) ? 0.f : fast_exp2((s[i] - m_new) * 1.4426950408889634f);
                s[i] = p;
                ls += p;
            }
            l_run = l_run * alpha + pair_sum(ls);
            m_run = m_new;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
                for (int db = 0; db < kNO; db++)
#pragma unroll
                    for (int i = 0; i < 16; i++) o[db][i] *= alpha;
            }
        }
        // ---- O^T += V^T P^T ----
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const float* vrow = csm + 2 * kKT + buf * kVT + (8 * (i >> 2) + 4 * h + (i & 3)) * RV + c32;
#pragma unroll
            for (int db = 0; db < kNO; db++) o[db] = mfma32_f32(vrow[32 * db], s[i], o[db]);
        }
        if (t + 1 < nt) store_tile(buf ^ 1);        // the other buffer: its readers passed the last barrier
        __syncthreads();
    }

    if (q_ok) {
#pragma clang fp contract(off)
        float* dst = out + (bh * sq + qi) * (long)D;
#pragma unroll
        for (int db = 0; db < kNO; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                f32x4 r;
#pragma unroll
                for (int x = 0; x < 4; x++) r[x] = l_run > 0.f ? o[db][4 * g + x] / l_run : 0.f;
                *reinterpret_cast<f32x4*>(dst + 32 * db + 8 * g + 4 * h) = r;
            }
    }
}

template <int D>
hipError_t launch_composed(const float* q, const float* k, const float* v, const float* mask, long mask_bh_stride,
                           float* out, size_t bh, int sq, int sk, float scale, hipStream_t st) {
    constexpr int lds = (2 * kCK * (D + 4) + 2 * kCK * (D + 8)) * (int)sizeof(float);   // 67 KB at D = 128
    if (lds > 64 * 1024) {
        static std::atomic<unsigned long long> attr_done;
        const hipError_t e = fv_set_max_lds_once((const void*)sdpa_composed_mfma_f32_kernel<D>, lds, attr_done);
        if (e != hipSuccess) return e;
    }
    const dim3 grid((unsigned)((sq + kCQ - 1) / kCQ), (unsigned)bh);
    hipLaunchKernelGGL((sdpa_composed_mfma_f32_kernel<D>), grid, dim3(256), lds, st, q, k, v, mask, mask_bh_stride, out,
                       sq, sk, scale);
    return hipGetLastError();
}

}  // namespace
}  // namespace fv

// 1 = launched, 0 = this head dim / alignment is the scalar kernel's, < 0 = -(hipError_t)
extern "C" int fv_internal_launch_composed_mfma(const float* q, const float* k, const float* v, const float* mask,
                                                long mask_bh_stride, float* out, size_t bh, int sq, int sk, int d,
                                                float scale, hipStream_t st) {
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0) return 0;
    if (sk > INT_MAX - 2 * fv::kCK || sq > INT_MAX - fv::kCQ) return 0;   // tile indices stay in int range
    hipError_t e;
    switch (d) {
        case 32: e = fv::launch_composed<32>(q, k, v, mask, mask_bh_stride, out, bh, sq, sk, scale, st); break;
        case 64: e = fv::launch_composed<64>(q, k, v, mask, mask_bh_stride, out, bh, sq, sk, scale, st); break;
        case 96: e = fv::launch_composed<96>(q, k, v, mask, mask_bh_stride, out, bh, sq, sk, scale, st); break;
        case 128: e = fv::launch_composed<128>(q, k, v, mask, mask_bh_stride, out, bh, sq, sk, scale, st); break;
        default: return 0;
    }
    return e == hipSuccess ? 1 : -(int)e;
}
