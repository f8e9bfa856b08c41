// Video Sparse Attention stages for gfx950: tile mean, coarse scores, coarse
// softmax x V, bitwise-descent top-k, tile permute, block-sparse fine attention,
// gated combine. Reference stages: crates/fastvideo-cudarc/src/rt/vsa.rs:358-470
// and the kernels cited per function below (kernels/core.cu, kernels/attn3.cu).
#include "attn_core.h"
#include "fv_internal.h"

namespace fv {

constexpr int kTileElems = 64;   // VSA cube = 4x4x4 tokens (rt/vsa.rs:29-31)

// ---- tile mean (kernels/core.cu:550-570, kernels/attn3.cu:208-226) --------------
// One 32-lane group per tile, 4 consecutive d per lane; the sum runs over the
// tile's real tokens in slot order with one f32 add per token, then / n — the
// same order and operations as the reference, so the result is bit-identical
// to its host restatement.
template <bool IN_BF16>
FV_DEV void tile_mean_body(const void* __restrict__ x, const int* __restrict__ slot_src,
                           const int* __restrict__ block_sizes, float* __restrict__ out, long seq, int dim,
                           int num_tiles, int round16) {
    const int grp = threadIdx.x >> 5, ln = threadIdx.x & 31;
    const int tile = blockIdx.x * 8 + grp;
    const long bh = blockIdx.y;
    if (tile >= num_tiles) return;
    const int n = block_sizes[tile];
    // slot_src == null: x is already tile-ordered, slot j of the tile is row tile*64 + j
    const int* src = slot_src ? slot_src + (long)tile * kTileElems : nullptr;
    const long row0 = (long)tile * kTileElems;
    float* ob = out + (bh * num_tiles + tile) * (long)dim;
    auto load_tok = [&](long tok, int d0) -> f32x4 {
        f32x4 v;
        if constexpr (IN_BF16) {
            const u32x2 raw = *reinterpret_cast<const u32x2*>(
                (const uint16_t*)x + (bh * seq + tok) * dim + d0);
            v[0] = __builtin_bit_cast(float, raw[0] << 16);
            v[1] = __builtin_bit_cast(float, raw[0] & 0xffff0000u);
            v[2] = __builtin_bit_cast(float, raw[1] << 16);
            v[3] = __builtin_bit_cast(float, raw[1] & 0xffff0000u);
        } else {
            v = *reinterpret_cast<const f32x4*>((const float*)x + (bh * seq + tok) * dim + d0);
            if (round16) {
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = bf16_bits_to_f32(bf16_rne_bits(v[e]));
            }
        }
        return v;
    };
    for (int d0 = ln * 4; d0 < dim; d0 += 128) {
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        int j = 0;
        // eight loads in flight, then their adds in slot order (the order is the contract)
        for (; j + 8 <= n; j += 8) {
            f32x4 v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = load_tok(src ? src[j + u] : row0 + j + u, d0);
#pragma unroll
            for (int u = 0; u < 8; u++)
#pragma unroll
                for (int e = 0; e < 4; e++) acc[e] = __fadd_rn(acc[e], v[u][e]);
        }
        for (; j < n; j++) {
            const f32x4 v = load_tok(src ? src[j] : row0 + j, d0);
#pragma unroll
            for (int e = 0; e < 4; e++) acc[e] = __fadd_rn(acc[e], v[e]);
        }
        f32x4 r;
#pragma unroll
        for (int e = 0; e < 4; e++) r[e] = n > 0 ? __fdiv_rn(acc[e], (float)n) : 0.0f;
        *reinterpret_cast<f32x4*>(ob + d0) = r;
    }
}

template <bool IN_BF16>
__global__ __launch_bounds__(256) void vsa_tile_mean_kernel(
    const void* __restrict__ x, const int* __restrict__ slot_src,
    const int* __restrict__ block_sizes, float* __restrict__ out, long seq, int dim,
    int num_tiles, int round16) {
    tile_mean_body<IN_BF16>(x, slot_src, block_sizes, out, seq, dim, num_tiles, round16);
}
// ---- tile pass and tile means in one scan (the whole op; rt/vsa.rs:378-384 and 406-414) ----------------
// dim == 128. 16 lanes per tile, a lane owns 8 consecutive d of every slot: it reads the slot's 16 (bf16) or 32
// (f32) bytes, writes them as bf16 (RNE) to the tile-ordered copy if there is one (zeros for padding slots), and adds
// them in f32, in slot order over the tile's real tokens, to its share of the mean: the same values in the same
// order as vsa_tile_mean_kernel, so the means (and the selection that follows from them) are bit-identical.
// slot_src == null: x is already tile-ordered. Eight slots in flight per lane. (Measured and not kept: the tile's 64
// slot indices fetched once and handed round the 16-lane row, the next batch's rows requested before a batch is
// stored and added: 124 registers and 10 % slower.)
struct ThreeScan {
    const void* in[3];
    uint16_t* tiles[3];   // null: no copy wanted
    float* means[3];
    float mul[3];         // f32 operands: factor on the values of the copy before their one rounding (1 = none);
                          // the means pool the operand as it is
};
template <bool IN_BF16>
__global__ __launch_bounds__(256) void vsa_tile_scan3_kernel(ThreeScan t, const int* __restrict__ slot_src,
                                                             const int* __restrict__ block_sizes, long seq, long padded,
                                                             int num_tiles) {
    constexpr int kDim = 128;
    const int grp = threadIdx.x >> 4, c = threadIdx.x & 15;
    const int tile = blockIdx.x * 16 + grp;
    if (tile >= num_tiles) return;
    const long bh = blockIdx.y;
    const void* __restrict__ x = t.in[blockIdx.z];
    uint16_t* __restrict__ xt = t.tiles[blockIdx.z];
    const int n = block_sizes[tile];
    const long row0 = (long)tile * kTileElems;
    const int* src = slot_src ? slot_src + row0 : nullptr;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.f;
    for (int j = 0; j < kTileElems; j += 8) {
        float v[8][8];
        u32x4 packed[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const long tok = src ? (long)src[j + u] : row0 + j + u;
            const bool real = tok >= 0;
            if constexpr (IN_BF16) {
                u32x4 raw = {0u, 0u, 0u, 0u};
                if (real) raw = *reinterpret_cast<const u32x4*>((const uint16_t*)x + (bh * seq + tok) * kDim + c * 8);
                packed[u] = raw;
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    v[u][2 * w] = __builtin_bit_cast(float, raw[w] << 16);
                    v[u][2 * w + 1] = __builtin_bit_cast(float, raw[w] & 0xffff0000u);
                }
            } else {
                f32x4 a = {0.f, 0.f, 0.f, 0.f}, b = a;
                if (real) {
                    const float* px = (const float*)x + (bh * seq + tok) * kDim + c * 8;
                    a = *reinterpret_cast<const f32x4*>(px);
                    b = *reinterpret_cast<const f32x4*>(px + 4);
                }
#pragma unroll
                for (int w = 0; w < 4; w++) v[u][w] = a[w], v[u][4 + w] = b[w];
                if (xt) {
                    const float m = t.mul[blockIdx.z];
#pragma unroll
                    for (int w = 0; w < 4; w++)
                        packed[u][w] = bf16_rne_bits(v[u][2 * w] * m) | ((unsigned)bf16_rne_bits(v[u][2 * w + 1] * m) << 16);
                }
            }
        }
        if (xt) {
#pragma unroll
            for (int u = 0; u < 8; u++)
                *reinterpret_cast<u32x4*>(xt + (bh * padded + row0 + j + u) * kDim + c * 8) = packed[u];
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            if (j + u < n) {   // uniform over the tile's 16 lanes
#pragma unroll
                for (int e = 0; e < 8; e++) acc[e] = __fadd_rn(acc[e], v[u][e]);
            }
        }
    }
    float* ob = t.means[blockIdx.z] + (bh * num_tiles + tile) * (long)kDim + c * 8;
    f32x4 r0, r1;
#pragma unroll
    for (int e = 0; e < 4; e++) {
        r0[e] = n > 0 ? __fdiv_rn(acc[e], (float)n) : 0.0f;
        r1[e] = n > 0 ? __fdiv_rn(acc[4 + e], (float)n) : 0.0f;
    }
    *reinterpret_cast<f32x4*>(ob) = r0;
    *reinterpret_cast<f32x4*>(ob + 4) = r1;
}

// The same scan for bf16 operands that want their tile-ordered copy, one wave per tile: the wave reads the tile's 64
// rows as whole 256-byte rows, four consecutive slots (1 KB, contiguous where the slots' tokens are) per load
// instruction, all 16 in flight; writes them to the copy the same way and to 16 KB of LDS; then lane c adds word c
// (two d) of every real slot in slot order. Same values, same order: means bit-identical to the kernel above.
// 99 - 108 us at 12 x 32768 / 32760 tokens x 3 operands where the 16-lanes-per-tile form takes 126 - 136 (its loads
// touch four tiles, 256 bytes each, per instruction); for pooling alone (no copy) that form is the faster one.
__global__ __launch_bounds__(64) void vsa_tile_scan3_staged_kernel(ThreeScan t, const int* __restrict__ slot_src,
                                                                   const int* __restrict__ block_sizes, long seq,
                                                                   long padded, int num_tiles) {
    __shared__ __attribute__((aligned(16))) unsigned stage[kTileElems * 64];   // 64 rows x 64 words
    const int lane = threadIdx.x;
    const int tile = blockIdx.x;
    const long bh = blockIdx.y;
    const uint16_t* __restrict__ x = (const uint16_t*)t.in[blockIdx.z];
    uint16_t* __restrict__ xt = t.tiles[blockIdx.z];
    const long row0 = (long)tile * kTileElems;
    const int n = block_sizes[tile];
    const int my_tok = slot_src ? slot_src[row0 + lane] : (int)(row0 + lane);   // lane = slot
    const int c = lane & 15;
    u32x4 v[16];
#pragma unroll
    for (int it = 0; it < 16; it++) {
        const int slot = it * 4 + (lane >> 4);
        const int tok = __shfl(my_tok, slot);
        v[it] = u32x4{0u, 0u, 0u, 0u};
        if (tok >= 0) v[it] = *reinterpret_cast<const u32x4*>(x + (bh * seq + tok) * 128 + c * 8);
    }
#pragma unroll
    for (int it = 0; it < 16; it++) {
        const int slot = it * 4 + (lane >> 4);
        *reinterpret_cast<u32x4*>(xt + (bh * padded + row0 + slot) * 128 + c * 8) = v[it];
        *reinterpret_cast<u32x4*>(&stage[slot * 64 + c * 4]) = v[it];
    }
    __syncthreads();   // one wave: orders its LDS writes before the reads below
    float a0 = 0.f, a1 = 0.f;
#pragma unroll 8
    for (int j = 0; j < kTileElems; j++) {
        const unsigned w = stage[j * 64 + lane];
        if (j < n) {
            a0 = __fadd_rn(a0, __builtin_bit_cast(float, w << 16));
            a1 = __fadd_rn(a1, __builtin_bit_cast(float, w & 0xffff0000u));
        }
    }
    float* ob = t.means[blockIdx.z] + (bh * num_tiles + tile) * 128L + lane * 2;
    float2 r;
    r.x = n > 0 ? __fdiv_rn(a0, (float)n) : 0.0f;
    r.y = n > 0 ? __fdiv_rn(a1, (float)n) : 0.0f;
    *reinterpret_cast<float2*>(ob) = r;
}

// ... and for f32 operands: the tile in two halves of 32 slots (16 KB of f32 each), two consecutive slots per load
// instruction; the copy is rounded to bf16 (RNE), the sums take the unrounded values, lane c owning d = c and c + 64.
__global__ __launch_bounds__(64) void vsa_tile_scan3_staged_f32_kernel(ThreeScan t, const int* __restrict__ slot_src,
                                                                       const int* __restrict__ block_sizes, long seq,
                                                                       long padded, int num_tiles) {
    __shared__ __attribute__((aligned(16))) unsigned stage[32 * 128];   // 32 rows x 128 words
    const int lane = threadIdx.x;
    const int tile = blockIdx.x;
    const long bh = blockIdx.y;
    const float* __restrict__ x = (const float*)t.in[blockIdx.z];
    uint16_t* __restrict__ xt = t.tiles[blockIdx.z];
    const long row0 = (long)tile * kTileElems;
    const int n = block_sizes[tile];
    const int my_tok = slot_src ? slot_src[row0 + lane] : (int)(row0 + lane);   // lane = slot
    const int c = lane & 31;
    const float mul = t.mul[blockIdx.z];   // x * 1.0f is x
    float a0 = 0.f, a1 = 0.f;
    u32x4 v[2][16];
    auto load_half = [&](int half, u32x4 (&r)[16]) {
#pragma unroll
        for (int it = 0; it < 16; it++) {
            const int slot = 32 * half + it * 2 + (lane >> 5);
            const int tok = __shfl(my_tok, slot);
            r[it] = u32x4{0u, 0u, 0u, 0u};
            if (tok >= 0) r[it] = *reinterpret_cast<const u32x4*>(x + (bh * seq + tok) * 128 + c * 4);
        }
    };
    load_half(0, v[0]);
#pragma unroll
    for (int half = 0; half < 2; half++) {
        if (half == 0) load_half(1, v[1]);   // in flight while the first half is stored and added
#pragma unroll
        for (int it = 0; it < 16; it++) {
            const int sl = it * 2 + (lane >> 5);
            const u32x4 w = v[half][it];
            // (the vector cast as a whole: __builtin_bit_cast(float, w[i]) read element 0 for every i with hipcc 7.2)
            const f32x4 f = __builtin_bit_cast(f32x4, w);
            u32x2 packed;
            packed[0] = bf16_rne_bits(f[0] * mul) | ((unsigned)bf16_rne_bits(f[1] * mul) << 16);
            packed[1] = bf16_rne_bits(f[2] * mul) | ((unsigned)bf16_rne_bits(f[3] * mul) << 16);
            *reinterpret_cast<u32x2*>(xt + (bh * padded + row0 + 32 * half + sl) * 128 + c * 4) = packed;
            *reinterpret_cast<u32x4*>(&stage[sl * 128 + c * 4]) = w;
        }
        __syncthreads();   // one wave: orders its LDS writes before the reads below
#pragma unroll 8
        for (int j = 0; j < 32; j++) {
            const float w0 = __builtin_bit_cast(float, stage[j * 128 + lane]);
            const float w1 = __builtin_bit_cast(float, stage[j * 128 + 64 + lane]);
            if (32 * half + j < n) {
                a0 = __fadd_rn(a0, w0);
                a1 = __fadd_rn(a1, w1);
            }
        }
        __syncthreads();   // ... and the reads before the next half's writes
    }
    float* ob = t.means[blockIdx.z] + (bh * num_tiles + tile) * 128L;
    ob[lane] = n > 0 ? __fdiv_rn(a0, (float)n) : 0.0f;
    ob[64 + lane] = n > 0 ? __fdiv_rn(a1, (float)n) : 0.0f;
}

// ---- coarse scores (rt/vsa.rs:385-388; arithmetic of the host oracle, rt/vsa.rs:185-189) ----
// scores[bh, qt, kt] = f32( (f64 dot of the tile means, d ascending from -0.0) * f64(scale) ).
// The product of two f32 values is exact in f64, so one v_fma_f64 per term is the oracle's
// multiply-then-add, and the scores (and with them the selected tiles) equal the host oracle's
// bit for bit. (The reference's device path runs cuBLAS f32 here, whose order is unspecified.)
// A 64 x 64 block of scores per workgroup, 4 x 4 per thread, the means staged in LDS as f32.
__global__ __launch_bounds__(256) void vsa_coarse_scores_kernel(
    const float* __restrict__ qc, const float* __restrict__ kc, float* __restrict__ scores,
    int nb, int dim, float scale) {
    __shared__ float qs[32][65];   // [d][tile]: the 4 tiles of a thread are consecutive words
    __shared__ float ks[32][65];
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    const int q0 = blockIdx.y * 64, k0 = blockIdx.x * 64;
    const long bh = blockIdx.z;
    const float* qb = qc + bh * nb * (long)dim;
    const float* kb = kc + bh * nb * (long)dim;
    double acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = -0.0;   // the identity of Rust's f64 Sum
    for (int d0 = 0; d0 < dim; d0 += 32) {
        for (int e = threadIdx.x; e < 64 * 32; e += 256) {
            const int r = e >> 5, c = e & 31;
            qs[c][r] = (q0 + r < nb && d0 + c < dim) ? qb[(long)(q0 + r) * dim + d0 + c] : 0.f;
            ks[c][r] = (k0 + r < nb && d0 + c < dim) ? kb[(long)(k0 + r) * dim + d0 + c] : 0.f;
        }
        __syncthreads();
        const int dn = min(32, dim - d0);
        for (int c = 0; c < dn; c++) {
            double a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; i++) a[i] = (double)qs[c][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; j++) b[j] = (double)ks[c][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = __builtin_fma(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
    const double sc = (double)scale;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int qi = q0 + ty * 4 + i, kj = k0 + tx * 4 + j;
            if (qi < nb && kj < nb) scores[(bh * nb + qi) * (long)nb + kj] = (float)(acc[i][j] * sc);
        }
}

// ---- coarse softmax x V (rt/vsa.rs:389-393, kernels/core.cu:177-252) ---------------
// coarse[bh, qt, :] = softmax(scores[bh, qt, :]) vc[bh]; eight query tiles per block
// share every vc row they read. dim = 128.
constexpr int kCoarseRows = 8;
__global__ __launch_bounds__(256) void vsa_coarse_pv_kernel(
    const float* __restrict__ scores, const float* __restrict__ vc, float* __restrict__ coarse,
    int nb) {
    extern __shared__ __attribute__((aligned(16))) float p_lds[];   // [kCoarseRows][nbp], rows 16-byte aligned
    __shared__ float red[kCoarseRows][4];
    __shared__ float stat[kCoarseRows];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int q0 = blockIdx.x * kCoarseRows;
    const long bh = blockIdx.y;
    const int rows = min(kCoarseRows, nb - q0);
    const int nbp = (nb + 3) & ~3;
    const float* sb = scores + (bh * nb + q0) * (long)nb;
    for (int r = 0; r < rows; r++)
        for (int j = tid; j < nb; j += 256) p_lds[r * nbp + j] = sb[(long)r * nb + j];
    __syncthreads();
    // row max
    for (int r = 0; r < rows; r++) {
        float m = neg_inf();
        for (int j = tid; j < nb; j += 256) m = fmaxf(m, p_lds[r * nbp + j]);
        for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
        if (lane == 0) red[r][wave] = m;
    }
    __syncthreads();
    if (tid < rows) stat[tid] = fmaxf(fmaxf(red[tid][0], red[tid][1]), fmaxf(red[tid][2], red[tid][3]));
    __syncthreads();
    for (int r = 0; r < rows; r++) {
        const float m = stat[r];
        float s = 0.f;
        for (int j = tid; j < nb; j += 256) {
            const float e = expf(p_lds[r * nbp + j] - m);
            p_lds[r * nbp + j] = e;
            s += e;
        }
        for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
        if (lane == 0) red[r][wave] = s;
    }
    __syncthreads();
    if (tid < rows) stat[tid] = 1.0f / (red[tid][0] + red[tid][1] + red[tid][2] + red[tid][3]);
    __syncthreads();
    // each half-block owns four rows; lane d accumulates over all key tiles in ascending order, four
    // vc rows in flight per step and the four weights of a row in one 16-byte LDS read
    constexpr int kOwn = kCoarseRows / 2;
    const int d = tid & 127, rh = tid >> 7;
    const float* vb = vc + bh * nb * 128L + d;
    const float* pr = p_lds + (kOwn * rh) * nbp;
    float a[kOwn];
#pragma unroll
    for (int r = 0; r < kOwn; r++) a[r] = 0.f;
    int kt = 0;
    for (; kt + 4 <= nb; kt += 4) {
        float vv[4];
#pragma unroll
        for (int u = 0; u < 4; u++) vv[u] = vb[(long)(kt + u) * 128];
#pragma unroll
        for (int r = 0; r < kOwn; r++) {
            const f32x4 p4 = *reinterpret_cast<const f32x4*>(pr + r * nbp + kt);
#pragma unroll
            for (int u = 0; u < 4; u++) a[r] += p4[u] * vv[u];
        }
    }
    for (; kt < nb; kt++) {
        const float vv = vb[(long)kt * 128];
#pragma unroll
        for (int r = 0; r < kOwn; r++) a[r] += pr[r * nbp + kt] * vv;
    }
#pragma unroll
    for (int r = 0; r < kOwn; r++)
        if (kOwn * rh + r < rows) coarse[(bh * nb + q0 + kOwn * rh + r) * 128L + d] = a[r] * stat[kOwn * rh + r];
}

// ---- top-k (kernels/core.cu:576-619, kernels/attn3.cu:279-363) ----------------------
// Output contract: T = the k-th largest sortable key of the row; the indices whose key is
// above T in ascending order, then those equal to T in ascending order, k in all, zero padded
// (k > n: every index, then zeros). Integer work, bit-exact.
//
// One wave owns one row and keeps it in registers: lane l holds the keys of indices
// l, 64 + l, 128 + l, ... (KPL of them; slots past n hold key 0 and are never emitted).
// T is built bit by bit from the top: a bit stays set if at least k keys are >= the candidate.
// A count is the sum of the popcounts of KPL wave-wide compare masks, so it lands in a scalar
// register and the decision is a scalar branch: no LDS, no atomics, no barrier. The emit pass
// walks the registers in index order; a lane's output slot is the running total plus the number
// of set mask bits below it.
FV_DEV unsigned sortable_key(float x) {
    const unsigned u = __builtin_bit_cast(unsigned, x);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

constexpr int kTopkMaxN = 4096;
constexpr int kTopkRowsPerBlock = 4;

FV_DEV int lanes_below(unsigned long long m) {
    return (int)__builtin_amdgcn_mbcnt_hi((unsigned)(m >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)m, 0u));
}

template <int KPL>
__global__ __launch_bounds__(64 * kTopkRowsPerBlock) void vsa_topk_kernel(const float* __restrict__ scores,
                                                                          unsigned* __restrict__ out, int rows,
                                                                          int n, int k) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kTopkRowsPerBlock + (threadIdx.x >> 6);
    if (row >= rows) return;   // the whole wave leaves; waves never meet at a barrier
    const float* s = scores + (long)row * n;
    unsigned key[KPL];
#pragma unroll
    for (int j = 0; j < KPL; j++) {
        const int i = 64 * j + lane;
        key[j] = i < n ? sortable_key(s[i]) : 0u;
    }
    unsigned t = 0u;           // k > n: threshold 0 lets every index through
    if (k <= n) {
#pragma unroll 1
        for (unsigned bit = 0x80000000u; bit != 0u; bit >>= 1) {
            const unsigned cand = t | bit;
            int at_least = 0;
#pragma unroll
            for (int j = 0; j < KPL; j++)
                at_least += __builtin_popcountll(__builtin_amdgcn_ballot_w64(key[j] >= cand));
            if (at_least >= k) t = cand;
        }
    }
    unsigned* dst = out + (long)row * k;
    int filled = 0;            // wave-uniform count of slots written so far
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
#pragma unroll
        for (int j = 0; j < KPL; j++) {
            const int i = 64 * j + lane;
            const bool take = i < n && (pass == 0 ? key[j] > t : key[j] == t);
            const unsigned long long m = __builtin_amdgcn_ballot_w64(take);
            const int pos = filled + lanes_below(m);
            if (take && pos < k) dst[pos] = (unsigned)i;
            filled += __builtin_popcountll(m);
        }
    }
    for (int pos = filled + lane; pos < k; pos += 64) dst[pos] = 0u;
}

// ---- tile permute (kernels/core.cu:1659-1672, kernels/attn3.cu:230-244) --------------
// [bh, seq, 128] -> tile-contiguous bf16 [bh, padded, 128]; padding slots are zero.
template <bool IN_BF16>
FV_DEV void tile_qkv_body(const void* __restrict__ x, const int* __restrict__ slot_src, uint16_t* __restrict__ xt,
                          long seq, long padded, int dim) {
    const long chunks = dim / 8;
    const long rem = blockIdx.x * 256L + threadIdx.x;
    if (rem >= padded * chunks) return;
    const long bh = blockIdx.y;
    const long slot = rem / chunks;
    const long c = rem - slot * chunks;
    const int src = slot_src[slot];
    u32x4 v = {0u, 0u, 0u, 0u};
    if (src >= 0) {
        if constexpr (IN_BF16) {
            v = *reinterpret_cast<const u32x4*>((const uint16_t*)x + (bh * seq + src) * dim + c * 8);
        } else {
            const float* px = (const float*)x + (bh * seq + src) * dim + c * 8;
            const f32x4 a = *reinterpret_cast<const f32x4*>(px);
            const f32x4 b = *reinterpret_cast<const f32x4*>(px + 4);
            v[0] = bf16_rne_bits(a[0]) | ((unsigned)bf16_rne_bits(a[1]) << 16);
            v[1] = bf16_rne_bits(a[2]) | ((unsigned)bf16_rne_bits(a[3]) << 16);
            v[2] = bf16_rne_bits(b[0]) | ((unsigned)bf16_rne_bits(b[1]) << 16);
            v[3] = bf16_rne_bits(b[2]) | ((unsigned)bf16_rne_bits(b[3]) << 16);
        }
    }
    *reinterpret_cast<u32x4*>(xt + (bh * padded + slot) * dim + c * 8) = v;
}
template <bool IN_BF16>
__global__ __launch_bounds__(256) void vsa_tile_qkv_kernel(const void* __restrict__ x,
                                                           const int* __restrict__ slot_src,
                                                           uint16_t* __restrict__ xt, long seq,
                                                           long padded, int dim) {
    tile_qkv_body<IN_BF16>(x, slot_src, xt, seq, padded, dim);
}

// ---- fine stage (kernels/core.cu:1029-1179) ---------------------------------------------
// One workgroup (2 waves x 32 queries) per (query tile, batch*head): online
// softmax over the selected key tiles in list order; key columns >=
// block_sizes[tile] are -inf. K and V tiles are separate single LDS buffers fed
// by direct global->LDS loads: K(i+1) streams in under softmax/PV of tile i and
// V(i) under QK/softmax of tile i. 32 KB of LDS per workgroup, so four
// workgroups share a CU.
// The softmax offset rides in the C operand of the K Q^T MFMAs (softmax_tile_side_off). LOG2DOM: the call's
// scale * log2(e) is exactly 1 (the caller folded the softmax scale into Q) and the per-score multiply is gone too.
template <bool LOG2DOM>
__global__ __launch_bounds__(128, 2) void vsa_fine_kernel(const VsaFineParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    lds_u8* kbuf = (lds_u8*)smem_raw;
    lds_u8* vbuf = kbuf + kTileBytes;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h = lane >> 5, c32 = lane & 31;
    const int work = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
    if (work >= p.total) return;
    const int bh = work / p.q_tiles;
    const int qtile = p.q_base + work % p.q_tiles;
    if (qtile >= p.num_tiles) return;
    const int nb = p.num_tiles, topk = p.topk;
    const size_t padded = (size_t)nb * kTileElems;
    const uint16_t* kb = p.kt + (size_t)bh * padded * 128;
    const uint16_t* vb = p.vt + (size_t)bh * padded * 128;
    const unsigned* sel = p.selected + ((size_t)bh * nb + qtile) * topk;
    const float sl2 = p.sl2;
    const float NEG = neg_inf();

    bf16x8 qf[8];
    load_q_frags(p.qt + ((size_t)bh * padded + (size_t)qtile * kTileElems) * 128, wave * 32 + c32,
                 true, lane, qf);
    const TileReadBases rb = tile_read_bases(lane);

    f32x16 o[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    SoftmaxOffState st;
    st.init();
    f32x16 s_init;   // the C operand every S block starts from: minus the lane's softmax offset
#pragma unroll
    for (int i = 0; i < 16; i++) s_init[i] = 0.f;

    // Per-lane DMA offsets are loop-invariant (every tile has 64 rows in the tile-ordered layout), so a
    // tile load is 8 (m0, load) pairs from a scalar base. The tile indices and sizes of the next two
    // list entries are fetched one iteration ahead: no scalar-load latency sits in front of a DMA issue.
    TileDma<2, 128> dma;
    dma.init(wave, lane);
    auto tile_at = [&](int i) -> int { return min((int)sel[min(i, topk - 1)], nb - 1); };
    int tile = tile_at(0), tile_next = tile_at(1);
    int valid = p.block_sizes[tile], valid_next = p.block_sizes[tile_next];
    dma.template issue<false>(kbuf, kb + (size_t)tile * kTileElems * 128, kTileElems, wave);
#pragma unroll 1
    for (int i = 0; i < topk; i++) {
        wait_vmcnt<0>();     // K(i) landed
        block_barrier();     // ... for every wave; PV(i-1) finished everywhere: V buffer free
        const int tile_nn = tile_at(i + 2);          // consumed an iteration from now
        f32x16 s[2];
        // the 8 DMA instructions of V(i) go out one behind every second MFMA of QK(i), those of K(i+1)
        // in three groups through the softmax: issued in one burst they hold the wave (in-order issue)
        // while the CU's address path drains, 4 % of the kernel's time
        const uint16_t* vsrc = vb + (size_t)tile * kTileElems * 128;
        qk_tile_side(kbuf, rb.k, qf, s, s_init, [&](int g) {
            if (g & 1) dma.template issue_one<true>(vbuf, vsrc, wave, g >> 1);
        });
        block_barrier();     // K buffer free
        const bool more = i + 1 < topk;
        const uint16_t* ksrc = kb + (size_t)tile_next * kTileElems * 128;
        if (valid < kTileElems) {
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int e = 0; e < 16; e++) {
                    const int col = 32 * b + 8 * (e >> 2) + 4 * h + (e & 3);
                    if (col >= valid) s[b][e] = NEG;
                }
        }
        bf16x8 pb[4];
        auto k_loads = [&](int part) {
            if (more) {
                const int first = 3 * part, last = part == 2 ? 8 : first + 3;
#pragma unroll
                for (int it = first; it < last; it++) dma.template issue_one<false>(kbuf, ksrc, wave, it);
            }
        };
        softmax_tile_side_off<!LOG2DOM>(s, st, o, s_init, sl2, pb, k_loads);
        if (more) wait_vmcnt<8>(); else wait_vmcnt<0>();   // V(i) landed; K(i+1) may be in flight
        block_barrier();
        pv_tile(vbuf, rb.v, pb, o);
        tile = tile_next;
        tile_next = tile_nn;
        valid = valid_next;
        valid_next = p.block_sizes[tile_nn];
    }

    const float l_tot = pair_sum(st.l_acc);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (p.final_out) {
        // fused combine (kernels/core.cu:803-835): out[token] = coarse[tile] * gate[token] + sparse,
        // the product rounded to f32 before the add as on the host; padding slots write nothing
#pragma clang fp contract(off)
        const int token = p.slot_src[(size_t)qtile * kTileElems + wave * 32 + c32];
        if (token < 0) return;
        const float* co = p.coarse + ((size_t)bh * nb + qtile) * 128;
        const size_t row = ((size_t)bh * p.seq + token) * 128;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = 32 * db + 8 * g + 4 * h;
                const f32x4 c4 = *reinterpret_cast<const f32x4*>(co + d0);
                f32x4 ga = {1.f, 1.f, 1.f, 1.f};
                if (p.gate) {
                    if (p.gate_is_bf16) {
                        const u32x2 raw = *reinterpret_cast<const u32x2*>((const uint16_t*)p.gate + row + d0);
                        ga[0] = __builtin_bit_cast(float, raw[0] << 16);
                        ga[1] = __builtin_bit_cast(float, raw[0] & 0xffff0000u);
                        ga[2] = __builtin_bit_cast(float, raw[1] << 16);
                        ga[3] = __builtin_bit_cast(float, raw[1] & 0xffff0000u);
                    } else {
                        ga = *reinterpret_cast<const f32x4*>((const float*)p.gate + row + d0);
                    }
                }
                f32x4 r;
#pragma unroll
                for (int x = 0; x < 4; x++) {
                    const float sp = o[db][4 * g + x] * inv;
                    r[x] = c4[x] * ga[x] + sp;
                }
                *reinterpret_cast<f32x4*>(p.final_out + row + d0) = r;
            }
        return;
    }
    float* ob = p.out + (((size_t)bh * p.q_tiles + (qtile - p.q_base)) * kTileElems + wave * 32 + c32) * 128;
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            f32x4 r;
#pragma unroll
            for (int x = 0; x < 4; x++) r[x] = o[db][4 * g + x] * inv;
            *reinterpret_cast<f32x4*>(ob + 32 * db + 8 * g + 4 * h) = r;
        }
}

// ---- combine (kernels/core.cu:803-835) -----------------------------------------------------
// out[token] = coarse[tile] * gate[token] + sparse[slot]; gate == null is a gate of one.
// ROUND16 is the bf16 combine of the H3 family (kernels/core.cu:825-830, kernels/attn3.cu:247-270):
// bf16(bf16(sparse) + bf16(bf16(coarse) * bf16(gate))), every step rounded to nearest even and the
// result stored as the f32 of that bf16 value; without a gate the product is bf16(coarse) itself.
template <bool GATE_BF16, bool ROUND16>
__global__ __launch_bounds__(256) void vsa_combine_kernel(
    const float* __restrict__ sparse, const float* __restrict__ coarse,
    const void* __restrict__ gate, const int* __restrict__ slot_src, float* __restrict__ out,
    long seq, int num_tiles, int q_base, int q_tiles, int has_gate) {
#pragma clang fp contract(off)   // coarse * gate rounds to f32 before the add, as on the host
    // one thread per (slot, 4 d): 32 threads per slot, 8 slots per block
    const long slot_lin = blockIdx.x * 8L + (threadIdx.x >> 5);   // over q_tiles * 64
    const int d0 = (threadIdx.x & 31) * 4;
    const long bh = blockIdx.y;
    if (slot_lin >= (long)q_tiles * kTileElems) return;
    const int g = (int)(slot_lin / kTileElems);
    const int tile = q_base + g;
    if (tile >= num_tiles) return;
    const int src = slot_src[(long)tile * kTileElems + (slot_lin - (long)g * kTileElems)];
    if (src < 0) return;
    const f32x4 sp = *reinterpret_cast<const f32x4*>(sparse + (bh * q_tiles * kTileElems + slot_lin) * 128 + d0);
    const f32x4 co = *reinterpret_cast<const f32x4*>(coarse + (bh * num_tiles + tile) * 128L + d0);
    f32x4 ga = {1.f, 1.f, 1.f, 1.f};
    if (has_gate) {
        if constexpr (GATE_BF16) {
            const u32x2 raw = *reinterpret_cast<const u32x2*>((const uint16_t*)gate + (bh * seq + src) * 128 + d0);
            ga[0] = __builtin_bit_cast(float, raw[0] << 16);
            ga[1] = __builtin_bit_cast(float, raw[0] & 0xffff0000u);
            ga[2] = __builtin_bit_cast(float, raw[1] << 16);
            ga[3] = __builtin_bit_cast(float, raw[1] & 0xffff0000u);
        } else {
            ga = *reinterpret_cast<const f32x4*>((const float*)gate + (bh * seq + src) * 128 + d0);
        }
    }
    f32x4 r;
    if constexpr (ROUND16) {
        auto r16 = [](float x) { return bf16_bits_to_f32(bf16_rne_bits(x)); };
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float c = r16(co[e]);
            const float p = has_gate ? r16(c * r16(ga[e])) : c;
            r[e] = r16(r16(sp[e]) + p);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; e++) r[e] = co[e] * ga[e] + sp[e];
    }
    *reinterpret_cast<f32x4*>(out + (bh * seq + src) * 128 + d0) = r;
}

}  // namespace fv

// ---- host launchers -----------------------------------------------------------------------

using namespace fv;

extern "C" hipError_t fv_internal_launch_tile_mean(const void* x, int x_is_bf16, const int* slot_src,
                                                   const int* block_sizes, float* out, size_t bh,
                                                   size_t seq, int dim, int num_tiles, int round16,
                                                   hipStream_t st) {
    const dim3 grid((num_tiles + 7) / 8, (unsigned)bh), block(256);
    if (x_is_bf16)
        hipLaunchKernelGGL(vsa_tile_mean_kernel<true>, grid, block, 0, st, x, slot_src, block_sizes, out,
                           (long)seq, dim, num_tiles, round16);
    else
        hipLaunchKernelGGL(vsa_tile_mean_kernel<false>, grid, block, 0, st, x, slot_src, block_sizes, out,
                           (long)seq, dim, num_tiles, round16);
    return hipGetLastError();
}

// Tile pass (tiles != null) and tile means of q, k and v in one launch; dim == 128. copy_mul (f32 operands only,
// null = none): factors on the values of the three copies before their rounding to bf16.
extern "C" hipError_t fv_internal_launch_tile_scan3(const void* const x[3], int x_is_bf16, const int* slot_src,
                                                    const int* block_sizes, uint16_t* const tiles[3],
                                                    float* const means[3], const float* copy_mul, size_t bh, size_t seq,
                                                    size_t padded, int num_tiles, hipStream_t st) {
    if (copy_mul && x_is_bf16) return hipErrorInvalidValue;   // a second rounding of values already rounded
    ThreeScan t;
    for (int i = 0; i < 3; i++)
        t.in[i] = x[i], t.tiles[i] = tiles ? tiles[i] : nullptr, t.means[i] = means[i], t.mul[i] = copy_mul ? copy_mul[i] : 1.0f;
    const dim3 grid((num_tiles + 15) / 16, (unsigned)bh, 3), block(256);
    if (tiles) {
        if (x_is_bf16)
            hipLaunchKernelGGL(vsa_tile_scan3_staged_kernel, dim3(num_tiles, (unsigned)bh, 3), dim3(64), 0, st, t, slot_src,
                               block_sizes, (long)seq, (long)padded, num_tiles);
        else
            hipLaunchKernelGGL(vsa_tile_scan3_staged_f32_kernel, dim3(num_tiles, (unsigned)bh, 3), dim3(64), 0, st, t,
                               slot_src, block_sizes, (long)seq, (long)padded, num_tiles);
        return hipGetLastError();
    }
    if (x_is_bf16)
        hipLaunchKernelGGL(vsa_tile_scan3_kernel<true>, grid, block, 0, st, t, slot_src, block_sizes, (long)seq, (long)padded, num_tiles);
    else
        hipLaunchKernelGGL(vsa_tile_scan3_kernel<false>, grid, block, 0, st, t, slot_src, block_sizes, (long)seq, (long)padded, num_tiles);
    return hipGetLastError();
}

// The coarse PV kernel's dynamic LDS limit (8 rows of up to 4096 scores), once per device.
extern "C" hipError_t fv_internal_init_vsa(void) {
    static std::atomic<unsigned long long> attr_done;
    return fv_set_max_lds_once((const void*)vsa_coarse_pv_kernel, (int)(sizeof(float) * kCoarseRows * kTopkMaxN),
                               attr_done);
}

extern "C" hipError_t fv_internal_launch_coarse(const float* qc, const float* kc, const float* vc,
                                                float* scores, float* coarse, size_t bh, int nb,
                                                int dim, float scale, hipStream_t st) {
    const dim3 g1((nb + 63) / 64, (nb + 63) / 64, (unsigned)bh);
    hipLaunchKernelGGL(vsa_coarse_scores_kernel, g1, dim3(256), 0, st, qc, kc, scores, nb, dim, scale);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || !coarse) return e;
    const size_t lds = sizeof(float) * kCoarseRows * (size_t)((nb + 3) & ~3);
    e = fv_internal_init_vsa();
    if (e != hipSuccess) return e;
    const dim3 g2((nb + kCoarseRows - 1) / kCoarseRows, (unsigned)bh);
    hipLaunchKernelGGL(vsa_coarse_pv_kernel, g2, dim3(256), lds, st, scores, vc, coarse, nb);
    return hipGetLastError();
}

extern "C" hipError_t fv_internal_launch_topk(const float* scores, unsigned* out, int rows, int n, int k,
                                              hipStream_t st) {
    if (n < 1 || n > kTopkMaxN) return hipErrorInvalidValue;
    const dim3 grid((rows + kTopkRowsPerBlock - 1) / kTopkRowsPerBlock), block(64 * kTopkRowsPerBlock);
    // keys per lane: the smallest instantiated count that holds the row (624 tiles: 10)
    const int need = (n + 63) / 64;
#define FV_TOPK(K) hipLaunchKernelGGL(vsa_topk_kernel<K>, grid, block, 0, st, scores, out, rows, n, k)
    if (need <= 4) FV_TOPK(4);
    else if (need <= 8) FV_TOPK(8);
    else if (need <= 10) FV_TOPK(10);
    else if (need <= 12) FV_TOPK(12);
    else if (need <= 16) FV_TOPK(16);
    else if (need <= 24) FV_TOPK(24);
    else if (need <= 32) FV_TOPK(32);
    else if (need <= 48) FV_TOPK(48);
    else FV_TOPK(64);
#undef FV_TOPK
    return hipGetLastError();
}

extern "C" hipError_t fv_internal_launch_tile_qkv(const void* x, int x_is_bf16, const int* slot_src,
                                                  uint16_t* xt, size_t bh, size_t seq, size_t padded,
                                                  int dim, hipStream_t st) {
    const size_t per = padded * (size_t)(dim / 8);
    const dim3 grid((unsigned)((per + 255) / 256), (unsigned)bh), block(256);
    if (x_is_bf16)
        hipLaunchKernelGGL(vsa_tile_qkv_kernel<true>, grid, block, 0, st, x, slot_src, xt, (long)seq,
                           (long)padded, dim);
    else
        hipLaunchKernelGGL(vsa_tile_qkv_kernel<false>, grid, block, 0, st, x, slot_src, xt, (long)seq,
                           (long)padded, dim);
    return hipGetLastError();
}

extern "C" hipError_t fv_internal_launch_fine(const fv::VsaFineParams* p, hipStream_t st) {
    if (p->sl2 == 1.0f)   // scale = ln 2: the caller folded the softmax scale into Q
        hipLaunchKernelGGL(vsa_fine_kernel<true>, dim3(p->per_xcd * 8), dim3(128), 2 * kTileBytes, st, *p);
    else
        hipLaunchKernelGGL(vsa_fine_kernel<false>, dim3(p->per_xcd * 8), dim3(128), 2 * kTileBytes, st, *p);
    return hipGetLastError();
}

extern "C" hipError_t fv_internal_launch_combine(const float* sparse, const float* coarse,
                                                 const void* gate, int gate_is_bf16,
                                                 const int* slot_src, float* out, size_t bh,
                                                 size_t seq, int num_tiles, int q_base, int q_tiles,
                                                 int round16, hipStream_t st) {
    const dim3 grid((unsigned)(((size_t)q_tiles * kTileElems + 7) / 8), (unsigned)bh), block(256);
    const int has_gate = gate != nullptr;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, grid, block, 0, st, sparse, coarse, gate, slot_src, out, (long)seq, num_tiles,
                           q_base, q_tiles, has_gate);
    };
    if (gate_is_bf16) {
        if (round16) launch(vsa_combine_kernel<true, true>);
        else launch(vsa_combine_kernel<true, false>);
    } else {
        if (round16) launch(vsa_combine_kernel<false, true>);
        else launch(vsa_combine_kernel<false, false>);
    }
    return hipGetLastError();
}
