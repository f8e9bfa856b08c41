// Dense and block-causal flash attention forward for gfx950, head_dim 128, bf16.
//
// Replaces the reference's flash_mma_fwd2_d128 / flash_mma_fwd2_causal_d128
// (crates/fastvideo-cudarc/src/rt/kernels/attn2.cu:40-352) behind
// attn::device_mma_sdpa / device_mma_sdpa_causal (rt/attn.rs:225-421, 652-730).
//
// Schedule (not a translation of the CUDA one):
//   * one workgroup = 4 waves = 128 queries of one (batch, head); each wave
//     owns 32 queries and walks the keys in tiles of 64;
//   * the wave computes S^T = K Q^T with v_mfma_f32_32x32x16_bf16: K rows come
//     from LDS as the A operand, Q^T stays in registers as the B operand for
//     the whole kernel. In the 32x32 accumulator layout every lane then holds
//     32 scores of ONE query, so the row max / row sum are in-lane reductions
//     plus one exchange with lane^32;
//   * P^T (bf16, RNE) is the B operand of O^T = V^T P^T straight from those
//     registers (the contraction index is a fixed permutation of the keys,
//     matched on the V side); V^T fragments are read from the row-major
//     [key][d] LDS tile with ds_read_b64_tr_b16;
//   * online softmax in base 2 with f32 max / sum / accumulators. The
//     accumulator is rescaled only when some row's max grew by more than
//     2^kRescaleLog2 since the last rescale; the final O / l is exact for any
//     such choice because P and l always share the same reference max;
//   * K/V tiles are prefetched global -> registers -> LDS (two LDS stages, one
//     barrier per tile);
//   * workgroup ids are remapped so that the workgroups resident on one XCD
//     walk consecutive query tiles of the same head (their K/V stream hits
//     that XCD's L2).
#include <stdlib.h>

#include "attn_core.h"
#include "fv_internal.h"

namespace fv {

constexpr int kD = 128;          // head dim
constexpr int kBM = 128;         // queries per workgroup
constexpr int kBN = 64;          // keys per tile
constexpr int kKStride = 272;    // bytes per K row in LDS (256 + 16 pad)
constexpr int kVStride = 320;    // bytes per V row in LDS (256 + 64 pad)
constexpr int kKBytes = kBN * kKStride;
constexpr int kVBytes = kBN * kVStride;
constexpr int kStageBytes = kKBytes + kVBytes;
constexpr int kFlashLdsBytes = 2 * kStageBytes;


template <bool CAUSAL>
__global__ __launch_bounds__(256, 2) void flash_fwd_d128(const FlashParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    lds_u8* smem = (lds_u8*)smem_raw;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int h = lane >> 5, c32 = lane & 31;

    // XCD-aware work assignment: workgroup ids go round-robin over the 8 XCDs,
    // so id%8 picks the XCD and id/8 the position in that XCD's contiguous
    // range of (head, query tile) work items.
    const int work = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
    if (work >= p.total) return;
    const int bh = work / p.nqt;
    // causal: heaviest (latest) query tiles first
    const int qt = CAUSAL ? (p.nqt - 1 - work % p.nqt) : (work % p.nqt);
    const int q0 = qt * kBM;
    const int sq = p.sq, sk = p.sk;
    const int qlen = min(kBM, sq - q0);
    const float sl2 = p.sl2;
    const float NEG = neg_inf();

    const uint16_t* Qh = p.q + ((size_t)bh * sq + q0) * kD;
    const uint16_t* Kh = p.k + (size_t)bh * sk * kD;
    const uint16_t* Vh = p.v + (size_t)bh * sk * kD;

    // ---- key-tile walk: [0, ns) then [mlo, mlo + ne - ns) --------------------
    const int nkt = (sk + kBN - 1) / kBN;
    int ns = 0, mlo = 0, ne = nkt;
    int hi_q = 0, lo_q = 0, sink_tok = 0;   // this lane's visible key range
    if constexpr (CAUSAL) {
        const int ft = p.ft, win = p.win;
        const int fq_lo = q0 / ft, fq_hi = (q0 + qlen - 1) / ft;
        const int hi_tok = (int)min((long)sk, (long)(fq_hi + 1) * ft);
        const int lo_tok = min(hi_tok, win > 0 ? max(0, fq_lo - win + 1) * ft : 0);
        sink_tok = (int)min((long)sk, (long)p.sink * ft);
        const int sink_tiles = (sink_tok + kBN - 1) / kBN;
        mlo = lo_tok / kBN;
        // sink blocks are visible to every query, also to those before them
        const int mhi = max((hi_tok + kBN - 1) / kBN, sink_tiles);
        ns = min(sink_tiles, mlo);
        ne = ns + (mhi - mlo);
        const int tq = (q0 + wave * 32 + c32) / ft;
        hi_q = (int)min((long)0x7fffffff, (long)(tq + 1) * ft);
        lo_q = win > 0 ? max(0, tq - win + 1) * ft : 0;
    }
    auto tile_of = [&](int e) -> int {
        if constexpr (CAUSAL) return e < ns ? e : mlo + (e - ns);
        else return e;
    };

    // ---- Q^T fragments (B operand), resident for the whole kernel ------------
    bf16x8 qf[8];
    {
        const int row = wave * 32 + c32;
        const bool ok = row < qlen;
        const uint16_t* src = Qh + (size_t)row * kD + 8 * h;
#pragma unroll
        for (int dk = 0; dk < 8; dk++) {
            u32x4 t = {0u, 0u, 0u, 0u};
            if (ok) t = *reinterpret_cast<const u32x4*>(src + 16 * dk);
            qf[dk] = __builtin_bit_cast(bf16x8, t);
        }
    }

    // ---- global -> register staging of one K/V tile --------------------------
    // 64 rows x 16 chunks of 16 B per tensor; thread t takes chunks t + 256 i.
    u32x4 gk[4], gv[4];
    const int ld_row = tid >> 4, ld_col = tid & 15;
    auto load_tile = [&](int kt) {
        const int kv0 = kt * kBN;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = kv0 + ld_row + 16 * i;
            u32x4 a = {0u, 0u, 0u, 0u}, b = {0u, 0u, 0u, 0u};
            if (row < sk) {
                const size_t off = (size_t)row * kD + ld_col * 8;
                a = *reinterpret_cast<const u32x4*>(Kh + off);
                b = *reinterpret_cast<const u32x4*>(Vh + off);
            }
            gk[i] = a;
            gv[i] = b;
        }
    };
    auto store_tile = [&](int stage) {
        lds_u8* kb = smem + stage * kStageBytes;
        lds_u8* vb = kb + kKBytes;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = ld_row + 16 * i;
            lds_write_b128(kb + row * kKStride + ld_col * 16, gk[i]);
            lds_write_b128(vb + row * kVStride + ld_col * 16, gv[i]);
        }
    };

    // per-lane LDS read offsets
    const int k_rd = c32 * kKStride + h * 16;                       // + kb*32*kKStride + dk*32
    const int b16 = lane >> 4, i16 = lane & 15;
    const int v_rd = (4 * h + (i16 >> 2)) * kVStride + (16 * (b16 & 1) + 4 * (i16 & 3)) * 2;
    // + (16 t + 8 g) * kVStride + db * 64

    f32x16 o[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    float m_run = NEG;     // running row max (raw scores)
    float ms_used = 0.f;   // m_used * sl2, the exponent offset P and l refer to
    float m_used = NEG;
    float l_acc = 0.f;     // this lane's share of the row sum

    if (ne > 0) {
        load_tile(tile_of(0));
        store_tile(0);
    }
    __syncthreads();

#pragma unroll 1
    for (int j = 0; j < ne; j++) {
        const int kt = tile_of(j);
        const int kv0 = kt * kBN;
        const int stage = j & 1;
        if (j + 1 < ne) load_tile(tile_of(j + 1));

        const lds_u8* kb = smem + stage * kStageBytes;
        const lds_u8* vb = kb + kKBytes;

        // S^T = K Q^T : two 32-key blocks
        f32x16 s[2];
#pragma unroll
        for (int b = 0; b < 2; b++) {
#pragma unroll
            for (int i = 0; i < 16; i++) s[b][i] = 0.f;
#pragma unroll
            for (int dk = 0; dk < 8; dk++) {
                const bf16x8 a = lds_read_b128(kb + k_rd + b * 32 * kKStride + dk * 32);
                s[b] = mfma32(a, qf[dk], s[b]);
            }
        }

        // key of s[b][i]: kv0 + 32 b + 8 (i/4) + 4 h + i%4
        if (kv0 + kBN > sk) {
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = kv0 + 32 * b + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (key >= sk) s[b][i] = NEG;
                }
        }
        if constexpr (CAUSAL) {
            const int kend = min(kv0 + kBN, sk);
            const bool lane_all = (kend <= hi_q && kv0 >= lo_q) || kend <= sink_tok;
            if (__builtin_amdgcn_ballot_w64(!lane_all) != 0) {
#pragma unroll
                for (int b = 0; b < 2; b++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int key = kv0 + 32 * b + 8 * (i >> 2) + 4 * h + (i & 3);
                        const bool vis = (key < hi_q && key >= lo_q) || key < sink_tok;
                        if (!vis) s[b][i] = NEG;
                    }
            }
        }

        // row max over this lane's 32 keys, then the other half's
        float mx = s[0][0];
#pragma unroll
        for (int i = 1; i < 16; i++) mx = __builtin_fmaxf(mx, s[0][i]);
#pragma unroll
        for (int i = 0; i < 16; i++) mx = __builtin_fmaxf(mx, s[1][i]);
        mx = pair_max(mx);
        m_run = __builtin_fmaxf(m_run, mx);

        // rescale when some row's max outgrew the offset in use
        const bool need = (m_run * sl2 - ms_used > kRescaleLog2) || (m_used == NEG && m_run != NEG);
        if (__builtin_amdgcn_ballot_w64(need) != 0) {
            const float ms_new = (m_run == NEG) ? 0.f : m_run * sl2;
            const float alpha = (m_used == NEG) ? 0.f : fast_exp2(ms_used - ms_new);
            l_acc *= alpha;
#pragma unroll
            for (int db = 0; db < 4; db++)
#pragma unroll
                for (int i = 0; i < 16; i++) o[db][i] *= alpha;
            m_used = m_run;
            ms_used = ms_new;
        }

        // P = 2^(s*sl2 - ms_used), row-sum share, bf16 pack
        bf16x8 pb[4];
#pragma unroll
        for (int b = 0; b < 2; b++) {
            f32x16 e;
#pragma unroll
            for (int i = 0; i < 16; i++) {
                e[i] = fast_exp2(__builtin_fmaf(s[b][i], sl2, -ms_used));
                l_acc += e[i];
            }
#pragma unroll
            for (int t = 0; t < 2; t++) {
                f32x8 f;
#pragma unroll
                for (int x = 0; x < 8; x++) f[x] = e[8 * t + x];
                pb[2 * b + t] = __builtin_convertvector(f, bf16x8);
            }
        }

        // O^T += V^T P^T
#pragma unroll
        for (int t = 0; t < 4; t++) {
#pragma unroll
            for (int db = 0; db < 4; db++) {
                const s16x4 lo = lds_read_tr16_b64(vb + v_rd + (16 * t) * kVStride + db * 64);
                const s16x4 hi = lds_read_tr16_b64(vb + v_rd + (16 * t + 8) * kVStride + db * 64);
                s16x8 a;
                a.lo = lo;
                a.hi = hi;
                o[db] = mfma32(__builtin_bit_cast(bf16x8, a), pb[t], o[db]);
            }
        }

        if (j + 1 < ne) store_tile(stage ^ 1);
        __syncthreads();
    }

    // ---- epilogue: O / l, written row-major [query][d] -------------------------
    const float l_tot = pair_sum(l_acc);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int row = wave * 32 + c32;
    if (row < qlen) {
        const size_t base = ((size_t)bh * sq + q0 + row) * kD;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = 32 * db + 8 * g + 4 * h;
                f32x4 r;
#pragma unroll
                for (int x = 0; x < 4; x++) r[x] = o[db][4 * g + x] * inv;
                if (p.out_is_bf16) {
                    const bf16x4 rb = __builtin_convertvector(r, bf16x4);
                    *reinterpret_cast<bf16x4*>(p.out_bf16 + base + d0) = rb;
                } else {
                    *reinterpret_cast<f32x4*>(p.out_f32 + base + d0) = r;
                }
            }
    }
}


// ---- ping-pong variant ------------------------------------------------------------------
// One workgroup = 8 waves = 256 queries; waves 0-3 (group 0) and 4-7 (group 1)
// share the SIMDs pairwise and run half an iteration apart: while one group is
// in its MFMA phase (O += P V of the previous tile, S = K Q^T of the current
// one) the other is in its VALU phase (softmax of its current tile), separated
// by workgroup barriers, so each SIMD's matrix pipe and vector ALU are busy at
// the same time by construction instead of by chance.
//
// Time is counted in slots (one phase each). Group 0 runs MFMA(j) in slot 2j and
// VALU(j) in slot 2j+1; group 1 is one slot behind. K and V tiles rotate
// through 3 LDS buffers each (swizzled, LDS-DMA fed). Every wave issues its
// share (2 + 2 instructions) of K(j+2) and V(j+1) from inside its MFMA phase j,
// where the address arithmetic and the issue ride under the matrix pipe, and
// waits for them (vmcnt) at the end of its MFMA phase j+1; both tiles are first
// read in MFMA phase j+2 / j+1's successor, at least three slots after issue.
// The buffers they overwrite held K(j-1) and V(j-2), last read in MFMA phase
// j-1 of either group, which ended at least one barrier before any wave's
// phase j began. Past the last tile the loads re-fetch the last tile into a
// buffer nobody reads, which keeps the issue and wait counts constant.
constexpr int kPpBM = 256;
constexpr int kStages = 3;
constexpr int kPpLdsBytes = 2 * kStages * kTileBytes;   // K[3], V[3] = 96 KB

template <bool CAUSAL>
__global__ __launch_bounds__(512, 2) void flash_fwd_pp_d128(const FlashParams p) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    lds_u8* smem = (lds_u8*)smem_raw;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: branches on it stay scalar
    const int grp = wave >> 2;
    const int h = lane >> 5, c32 = lane & 31;
    const int work = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
    if (work >= p.total) return;
    const int bh = work / p.nqt;
    const int qt = CAUSAL ? (p.nqt - 1 - work % p.nqt) : (work % p.nqt);
    const int q0 = qt * kPpBM;
    const int sq = p.sq, sk = p.sk;
    const int qlen = min(kPpBM, sq - q0);
    const float sl2 = p.sl2;
    const float NEG = neg_inf();
    // Fetch the epilogue's arguments now. Left to the compiler, their scalar loads sit
    // right before the main loop, still pending at its head, and a pending scalar load
    // (out-of-order return) turns every LDS wait count in the loop into a full drain.
    float* out_f32 = p.out_f32;
    uint16_t* out_bf16 = p.out_bf16;
    int out_is_bf16 = p.out_is_bf16;
    asm volatile("" : "+s"(out_f32), "+s"(out_bf16), "+s"(out_is_bf16));

    const uint16_t* Qh = p.q + ((size_t)bh * sq + q0) * kD;
    const uint16_t* Kh = p.k + (size_t)bh * sk * kD;
    const uint16_t* Vh = p.v + (size_t)bh * sk * kD;

    const int nkt = (sk + kBN - 1) / kBN;
    int ns = 0, mlo = 0, ne = nkt;
    int hi_q = 0, lo_q = 0, sink_tok = 0;
    if constexpr (CAUSAL) {
        const int ft = p.ft, win = p.win;
        const int fq_lo = q0 / ft, fq_hi = (q0 + qlen - 1) / ft;
        const int hi_tok = (int)min((long)sk, (long)(fq_hi + 1) * ft);
        const int lo_tok = min(hi_tok, win > 0 ? max(0, fq_lo - win + 1) * ft : 0);
        sink_tok = (int)min((long)sk, (long)p.sink * ft);
        const int sink_tiles = (sink_tok + kBN - 1) / kBN;
        mlo = lo_tok / kBN;
        const int mhi = max((hi_tok + kBN - 1) / kBN, sink_tiles);
        ns = min(sink_tiles, mlo);
        ne = ns + (mhi - mlo);
        const int tq = (q0 + wave * 32 + c32) / ft;
        hi_q = (int)min((long)0x7fffffff, (long)(tq + 1) * ft);
        lo_q = win > 0 ? max(0, tq - win + 1) * ft : 0;
    }
    if (ne <= 0) return;   // cannot happen for sk >= 1 (the walk always holds the query's own block)
    // key-tile index of walk position e; positions past the end repeat the last tile
    auto tile_of = [&](int e) -> int {
        e = min(e, ne - 1);
        if constexpr (CAUSAL) return e < ns ? e : mlo + (e - ns);
        else return e;
    };
    auto kbuf = [&](int st) -> lds_u8* { return smem + st * kTileBytes; };
    auto vbuf = [&](int st) -> lds_u8* { return smem + (kStages + st) * kTileBytes; };
    auto next_stage = [](int st) -> int { return st == kStages - 1 ? 0 : st + 1; };

    TileDma<8> dma;
    dma.init(wave, lane);
    auto issue_k = [&](int e, int st) {
        const int kv0 = tile_of(e) * kBN;
        dma.issue<false>(kbuf(st), Kh + (size_t)kv0 * kD, sk - kv0, wave);
    };
    auto issue_v = [&](int e, int st) {
        const int kv0 = tile_of(e) * kBN;
        dma.issue<true>(vbuf(st), Vh + (size_t)kv0 * kD, sk - kv0, wave);
    };

    issue_k(0, 0);
    issue_k(1, 1);
    issue_v(0, 0);
    bf16x8 qf[8];
    {
        const int row = wave * 32 + c32;
        load_q_frags(Qh, row, row < qlen, lane, qf);   // drains vmcnt: the three tiles have landed too
    }
    const TileReadBases rb = tile_read_bases(lane);

    f32x16 o[4];
#pragma unroll
    for (int db = 0; db < 4; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    SoftmaxState st;
    st.init();
    f32x16 s[2];
    bf16x8 pb[4];     // P of the previous tile; zero before the first one
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int x = 0; x < 8; x++) pb[t][x] = (__bf16)0.0f;

    // the loads a matrix phase issues are prepared (addresses, tail clamp) one VALU phase earlier
    auto prep_k = [&](int e, int st) {
        const int kv0 = tile_of(e) * kBN;
        return dma.prepare<false>(kbuf(st), Kh + (size_t)kv0 * kD, sk - kv0, wave);
    };
    auto prep_v = [&](int e, int st) {
        const int kv0 = tile_of(e) * kBN;
        return dma.prepare<true>(vbuf(st), Vh + (size_t)kv0 * kD, sk - kv0, wave);
    };
    TileDma<8>::Prepared dk = prep_k(2, 2), dv = prep_v(1, 1);

    block_barrier();                 // K(0), K(1), V(0) resident
    if (grp == 1) block_barrier();   // group 1 idles through slot 0

    // LDS stages: K(j) in sk_cur, K(j+2) goes to sk_ld = stage of j-1; V(j-1) in sv_prev, V(j+1)
    // goes to the stage after V(j)
    int sk_cur = 0, sk_ld = 2, sv_prev = 0, sv_ld = 1;
#pragma unroll 1
    for (int j = 0; j < ne; j++) {
        // ---- MFMA phase: group 0 in slot 2j, group 1 in slot 2j+1 ----
        __builtin_amdgcn_s_setprio(1);
        constexpr int kAhead = CAUSAL ? 2 : 3;   // LDS prefetch depth the register budget allows
        // P starts as zero, so the first pass adds 0 * V(0) (finite, resident) and needs no special case
        mfma_phase<true, kAhead>(vbuf(sv_prev), kbuf(sk_cur), rb, pb, o, qf, s, [&](int g) {
            if (g == 1) TileDma<8>::issue_prepared(dk, 0);
            if (g == 2) TileDma<8>::issue_prepared(dk, 1);
            if (g == 4) TileDma<8>::issue_prepared(dv, 0);
            if (g == 5) TileDma<8>::issue_prepared(dv, 1);
        });
        __builtin_amdgcn_s_setprio(0);
        wait_vmcnt<4>();             // this wave's loads of the previous phase have landed
        __builtin_amdgcn_sched_barrier(0);
        block_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // ---- VALU phase: group 0 in slot 2j+1, group 1 in slot 2j+2 ----
        const int kv0 = tile_of(j) * kBN;
        if (kv0 + kBN > sk) {
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = kv0 + 32 * b + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (key >= sk) s[b][i] = NEG;
                }
        }
        if constexpr (CAUSAL) {
            const int kend = min(kv0 + kBN, sk);
            const bool lane_all = (kend <= hi_q && kv0 >= lo_q) || kend <= sink_tok;
            if (__builtin_amdgcn_ballot_w64(!lane_all) != 0) {
#pragma unroll
                for (int b = 0; b < 2; b++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int key = kv0 + 32 * b + 8 * (i >> 2) + 4 * h + (i & 3);
                        const bool vis = (key < hi_q && key >= lo_q) || key < sink_tok;
                        if (!vis) s[b][i] = NEG;
                    }
            }
        }
        softmax_tile(s, st, o, sl2, pb);
        // P and the row sum must be complete before the barrier: without this the
        // compiler sinks the exponentials past it, into the matrix phase
        asm volatile("" ::"v"(pb[0]), "v"(pb[1]), "v"(pb[2]), "v"(pb[3]), "v"(st.l_acc));
        sv_prev = j > 0 ? next_stage(sv_prev) : 0;   // V(j) lives in stage j % 3
        sv_ld = next_stage(sv_ld);
        sk_ld = sk_cur;
        sk_cur = next_stage(sk_cur);
        dk = prep_k(j + 3, sk_ld);   // for matrix phase j+1: K(j+3), V(j+2)
        dv = prep_v(j + 2, sv_ld);
        if (grp == 0 || j + 1 < ne) {
            __builtin_amdgcn_sched_barrier(0);
            block_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // O += P V of the last tile (its V landed before the last barrier both groups passed)
    pv_tile(vbuf(sv_prev), rb.v, pb, o);
    wait_vmcnt<0>();   // the redundant tail loads must not outlive the workgroup's LDS

    const float l_tot = pair_sum(st.l_acc);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int row = wave * 32 + c32;
    if (row < qlen) {
        const size_t base = ((size_t)bh * sq + q0 + row) * kD;
#pragma unroll
        for (int db = 0; db < 4; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = 32 * db + 8 * g + 4 * h;
                f32x4 r;
#pragma unroll
                for (int x = 0; x < 4; x++) r[x] = o[db][4 * g + x] * inv;
                if (out_is_bf16) {
                    const bf16x4 rb4 = __builtin_convertvector(r, bf16x4);
                    *reinterpret_cast<bf16x4*>(out_bf16 + base + d0) = rb4;
                } else {
                    *reinterpret_cast<f32x4*>(out_f32 + base + d0) = r;
                }
            }
    }
}

}  // namespace fv

// ---- host launchers -------------------------------------------------------------

extern "C" int fv_internal_flash_block_m(void) {
    static const int bm = [] {
        const char* e = getenv("FV_FLASH_KERNEL");
        return (e && e[0] == 'v' && e[1] == '1') ? fv::kBM : fv::kPpBM;
    }();
    return bm;
}

extern "C" hipError_t fv_internal_launch_flash(const fv::FlashParams* p, int causal,
                                               hipStream_t stream) {
    const bool pp = fv_internal_flash_block_m() == fv::kPpBM;
    static bool attr_done[4] = {false, false, false, false};
    const void* fn = pp ? (causal ? (const void*)fv::flash_fwd_pp_d128<true> : (const void*)fv::flash_fwd_pp_d128<false>)
                        : (causal ? (const void*)fv::flash_fwd_d128<true> : (const void*)fv::flash_fwd_d128<false>);
    const int lds = pp ? fv::kPpLdsBytes : fv::kFlashLdsBytes;
    const int idx = (pp ? 2 : 0) + causal;
    if (!attr_done[idx]) {
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        attr_done[idx] = true;
    }
    const dim3 grid(p->per_xcd * 8), block(pp ? 512 : 256);
    if (pp) {
        if (causal) hipLaunchKernelGGL(fv::flash_fwd_pp_d128<true>, grid, block, lds, stream, *p);
        else hipLaunchKernelGGL(fv::flash_fwd_pp_d128<false>, grid, block, lds, stream, *p);
    } else {
        if (causal) hipLaunchKernelGGL(fv::flash_fwd_d128<true>, grid, block, lds, stream, *p);
        else hipLaunchKernelGGL(fv::flash_fwd_d128<false>, grid, block, lds, stream, *p);
    }
    return hipGetLastError();
}
