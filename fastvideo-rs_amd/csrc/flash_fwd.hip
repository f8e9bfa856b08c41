// Dense and block-causal flash attention forward for gfx950, head dim 128 or 64, bf16.
//
// Replaces the reference's flash_mma_fwd2_d128 / flash_mma_fwd2_causal_d128
// (crates/fastvideo-cudarc/src/rt/kernels/attn2.cu:40-352) behind
// attn::device_mma_sdpa / device_mma_sdpa_causal (rt/attn.rs:225-421, 652-730), and
// flash_mma_fwd2_window_d128 (attn2.cu:356-578) behind device_mma_sdpa_window
// (rt/attn.rs:526-610).
//
// Schedule (not a translation of the CUDA one):
//   * one workgroup = 8 waves = 256 queries of one (batch, head); each wave
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
//   * waves 0-3 (group 0) and 4-7 (group 1) share the SIMDs pairwise and run
//     half an iteration apart: while one group is in its MFMA phase (O += P V
//     of the previous tile, S = K Q^T of the current one, operands prefetched
//     from LDS a fixed number of MFMAs ahead) the other is in its VALU phase
//     (softmax of its current tile), separated by workgroup barriers, so each
//     SIMD's matrix pipe and vector ALU are busy at the same time by
//     construction. Interleaving the two instruction kinds inside one wave
//     loses on this hardware: a wave issues in order, so its VALU work stalls
//     behind every MFMA that waits for the matrix pipe;
//   * K/V tiles go global -> LDS directly (global_load_lds_dwordx4) into
//     XOR-swizzled unpadded tiles, four buffers each;
//   * dense launches remap workgroup ids so that the workgroups resident on one
//     XCD walk consecutive query tiles of the same head (their K/V stream hits
//     that XCD's L2); block-causal launches run longest tiles first.
//
// Time is counted in slots (one phase each); a phase covers a PAIR of key tiles
// (128 keys): a matrix phase is 64 MFMAs (PV of the previous pair, QK of the
// current pair), a VALU phase the softmax of the pair with one shared max /
// rescale decision. Barriers, the LDS-latency ramp at the head of a matrix phase
// and the per-phase bookkeeping are thus paid once per 128 keys. Group 0 runs
// matrix phase m in slot 2m and VALU phase m in slot 2m+1; group 1 is one slot
// behind. K and V tiles rotate through 4 LDS buffers each (128 KB): matrix phase
// m reads K(2m), K(2m+1), V(2m-2), V(2m-1) and issues K(2m+2), K(2m+3), V(2m),
// V(2m+1) into the buffers phase m-1 read last, all of them during the first tile
// of the pair (a load needs more than a thousand cycles to land), from descriptors
// (addresses, tail clamp) prepared in the VALU phase before, so the matrix phase
// carries bare DMA instructions and no branches (a branch inside the unrolled phase breaks the
// register allocation of the 16-register accumulator tuples: 59 spills measured).
// Every wave waits for its own loads at the end of the same phase, one barrier
// before phase m+1 of either group reads them. Phase 0 has no previous pair and runs its QK half only
// (unrolled apart from the loop). An odd tile count is rounded up: the extra
// tile re-reads the last one and all its scores are masked. Tile indices are walk
// positions: a masked call walks up to three ascending tile ranges (block-causal:
// sink tiles, then the band; VDN window: rows before the video + frame 0, the
// window frames, the last frame + rows after the video).
#include <stdlib.h>
#include <string.h>

#include "attn_core.h"
#include "fv_internal.h"

namespace fv {

constexpr int kBN = 64;          // keys per tile
constexpr int kPpBM = 256;      // queries per workgroup
constexpr int kRing2 = 4;        // K buffers = V buffers: 128 KB of LDS at D = 128, 64 KB at D = 64
constexpr int kVoteBytes = 64;   // behind the rings: one word per wave for the fixed-offset pass's vote

// Workgroups that had to redo their pass with the running max (see flash_item) since the library was loaded on
// this device.
__device__ unsigned long long g_exact_pass_reruns;

// One workgroup's item: the whole pass over its key tiles and the store of its rows. Returns false (FIXED only,
// nothing stored) when the pass has to be made again with the running max.
// FIXED: once the first phase has put every query's offset at the largest score of its first 128 keys, the offset
// stays there: no row max and no rescale decision in the loop (32 three-operand VALU instructions a phase less:
// 2 % of the time of the long launches, 9 % at head dim 64). Exact for any input as long as nothing overflows (P
// and l share the offset), so the pass is checked before anything is stored: if some row's scores grew by more
// than about 2^90 past that first maximum (a row sum of 2^100 or more, whose reciprocal nears the subnormals, or an accumulator not
// finite), the workgroup makes the pass again from the top with the running max. One difference in rounding
// remains: the largest P of a row is exactly 1 under the running max and a rounded bf16 number under the fixed
// offset, so a row that ONE late key dominates can be off by up to 2^-8 relative; the launcher therefore takes
// this form only for results that are rounded to bf16 anyway.
template <bool MASKED, int D, bool LOG2DOM, bool FIXED, class Params>
FV_DEV bool flash_item(const Params& p, const int wave, const int lane, const int block) {
    // (masked launches: only where every query sees key 0, see launch_flash)
    using G = TileGeo<D>;
    constexpr int kD = D;
    constexpr int kTileBytes = G::kTile;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    lds_u8* smem = (lds_u8*)smem_raw;

    const int tid = wave * 64 + lane;   // (wave is scalar: branches on it stay scalar)
    const int grp = wave >> 2;
    const int h = lane >> 5, c32 = lane & 31;
    // Work order. Dense (equal tiles): workgroup i runs on XCD i % 8, and XCD x takes the
    // contiguous range [x, x+1) * per_xcd of (head, query tile) items, so its CUs stream one
    // head's K/V through its L2 together. Masked (tiles differ in length by up to the whole
    // sequence): longest first over the whole launch, tile index major and head minor
    // (block-causal: last tile first; VDN window: the anchor / global tiles at both ends
    // first); measured 9 % faster than the dense order, whose per-XCD ranges hold unequal work.
    int bh, qt, sp = 0;   // sp: this workgroup's key split (dense launches with kv_split > 1)
    if constexpr (MASKED) {
        const int work = block;
        if (work >= p.total) return true;
        const int nbh = p.total / p.nqt;
        bh = work % nbh;
        const int r = work / nbh;
        qt = p.mask_mode == 2 ? ((r & 1) ? (r >> 1) : p.nqt - 1 - (r >> 1)) : p.nqt - 1 - r;
    } else {
        const int work = (block & 7) * p.per_xcd + (block >> 3);
        if (work >= p.total) return true;
        const int per_bh = p.nqt * p.kv_split;
        bh = work / per_bh;
        const int rem = work - bh * per_bh;
        qt = rem / p.kv_split;
        sp = rem - qt * p.kv_split;
    }
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

    const uint16_t* Qh = p.q + (size_t)bh * p.q_plane + (size_t)q0 * kD;
    const uint16_t* Kh = p.k + (size_t)bh * p.k_plane;
    const uint16_t* Vh = p.v + (size_t)bh * p.v_plane;

    const int nkt_all = (sk + kBN - 1) / kBN;
    // a split walks key tiles [t0, t0 + nkt) of the nkt_all tiles (the whole range without split-KV)
    const int t0 = MASKED ? 0 : sp * p.split_tiles;
    const int nkt = MASKED ? nkt_all : min(p.split_tiles, nkt_all - t0);
    // The key-tile walk of this query tile: up to three ascending tile ranges [a_i, a_i + n_i),
    // n0 + n1 + n2 = ne tiles in all. A lane's query sees key x iff
    //   x < a_hi  ||  x >= c_lo  ||  (w_lo <= x && x < w_hi).
    int a1 = 0, a2 = 0, n0 = nkt, n1 = 0, ne = nkt;
    int a_hi = 0, c_lo = 0x7fffffff, w_lo = 0, w_hi = 0;
    if constexpr (MASKED) {
        const int qi = q0 + wave * 32 + c32;   // this lane's query (rows past sq are never stored)
        const TileWalk w = mask_tile_walk(p, q0, qlen, nkt);
        a1 = w.a1;
        a2 = w.a2;
        n0 = w.n0;
        n1 = w.n1;
        ne = w.ne;
        if (p.mask_mode == 1) {
            // block-causal (rt/attn.rs:449-453): keys of blocks (tq - win, tq], plus the sink blocks
            const int ft = p.ft, win = p.win;
            const int tq = qi / ft;
            a_hi = (int)min((long)sk, (long)p.sink * ft);
            w_hi = (int)min((long)0x7fffffff, (long)(tq + 1) * ft);
            w_lo = win > 0 ? max(0, tq - win + 1) * ft : 0;
        } else {
            // VDN window (rt/attn.rs:483-510): rows outside [vs, ve) and the frames 0 and
            // frames-1 are dense both ways; any other frame sees the frames of its window
            const int vs = p.vs, ve = p.ve, t = p.ft, last = p.frames - 1, c = p.chunk, r = p.radius;
            auto lo_frame = [&](int f) { return max(0, c > 0 ? (f / c - r) * c : f - r); };
            auto hi_frame = [&](int f) { return min(last, c > 0 ? (f / c + r + 1) * c - 1 : f + r); };
            const bool inner_q = qi >= vs + t && qi < ve - t;
            if (inner_q) {
                const int qf = (qi - vs) / t;
                a_hi = vs + t;
                c_lo = ve - t;
                w_lo = vs + lo_frame(qf) * t;
                w_hi = vs + (hi_frame(qf) + 1) * t;
            } else {
                a_hi = 0x7fffffff;
            }
        }
    }
    if constexpr (MASKED) {
        // No key tile is visible to any query of this tile (block-causal with more queries than keys
        // and a window that has moved past the last key): rows of zeros, what a query without a
        // visible key gets in a partly visible tile too (l == 0). Workgroup-uniform, before any barrier.
        if (ne <= 0) {
            const int units = kD * (out_is_bf16 ? 2 : 4) / 16;   // 16-byte units per output row
            char* ob = out_is_bf16 ? (char*)(out_bf16 + ((size_t)bh * sq + q0) * kD)
                                   : (char*)(out_f32 + ((size_t)bh * sq + q0) * kD);
            const u32x4 zero = {0u, 0u, 0u, 0u};
            for (int u = tid; u < qlen * units; u += 512) global_store<u32x4>(ob + (size_t)u * 16, zero);
            return true;
        }
    }
    const int np = (ne + 1) / 2;             // phases
    // first key of walk position e; positions past the end repeat the last tile (their scores are masked)
    auto kv0_of = [&](int e) -> int {
        e = min(e, ne - 1);
        if constexpr (MASKED) return (e < n0 ? e : e < n0 + n1 ? a1 + (e - n0) : a2 + (e - n0 - n1)) * kBN;
        else return (t0 + e) * kBN;
    };
    // tile t lives in buffer t mod 4 (t >= -2)
    auto kbuf = [&](int t) -> lds_u8* { return smem + (t & (kRing2 - 1)) * kTileBytes; };
    auto vbuf = [&](int t) -> lds_u8* { return smem + (kRing2 + (t & (kRing2 - 1))) * kTileBytes; };

    TileDma<8, D> dma;
    dma.init(wave, lane);
    // tiles past the end repeat the last one
    auto target_k = [&](int t) {
        const int kv0 = kv0_of(t);
        return dma.template prepare<false>(kbuf(t), Kh + (size_t)kv0 * kD, sk - kv0, wave);
    };
    auto target_v = [&](int t) {
        const int kv0 = kv0_of(t);
        return dma.template prepare<true>(vbuf(t), Vh + (size_t)kv0 * kD, sk - kv0, wave);
    };
    using Dma = TileDma<8, D>;
    constexpr int kIt = Dma::ITER;   // DMA instructions per wave and tile: 2 (D = 128) or 1 (D = 64)
    {
        const typename Dma::Prepared a0 = target_k(0), a1 = target_k(1);
#pragma unroll
        for (int it = 0; it < kIt; it++) {
            Dma::issue_prepared(a0, it);
            Dma::issue_prepared(a1, it);
        }
    }
    bf16x8 qf[D / 16];
    const TileReadBases rb = tile_read_bases<D>(lane);
    // The wave's 32 query rows come through LDS: whole rows by LDS-DMA (1 KB of consecutive global memory per
    // instruction) into the wave's own slice of the V ring (group 0: buffers 0, 1, idle until the first matrix
    // phase requests V(0); group 1: buffers 2, 3, idle a phase longer), in the K tiles' swizzle, then the fragments
    // with the K operand's conflict-free read pattern. (Loading the fragments straight from global memory takes
    // 16-byte pieces of 32 rows per instruction: 2 - 3 % slower on 512-key launches, whose prologue shows.)
    // Group 1, which idles through the first slot anyway, waits for its rows only then: group 0 starts as soon as
    // K(0), K(1) and its own rows are there.
    lds_u8* qs = smem + kRing2 * kTileBytes + wave * (32 * G::kRow);
    auto q_request = [&]() {
        const unsigned qlds = __builtin_amdgcn_readfirstlane((unsigned)(size_t)qs);
        constexpr int kQIt = 32 * G::kRow / 1024;
#pragma unroll
        for (int it = 0; it < kQIt; it++) {
            const int r = it * G::kRowsPerDma + lane / G::kChunks, pch = lane % G::kChunks;
            const int rg = min(wave * 32 + r, qlen - 1);   // rows past the end re-read the last one (zeroed below)
            lds_dma16_s(qlds + it * 1024, Qh, (unsigned)(rg * G::kRow + ((pch ^ G::kswz(r)) << 4)));
        }
    };
    auto q_read = [&]() {
        wait_vmcnt<0>();   // this wave's rows (and its parts of K(0), K(1)) have landed
        const bool ok = wave * 32 + c32 < qlen;
#pragma unroll
        for (int dk = 0; dk < D / 16; dk++) {
            bf16x8 t = lds_read_b128(qs + (rb.k ^ (dk << 5)));
            if (!ok) t = __builtin_bit_cast(bf16x8, u32x4{0u, 0u, 0u, 0u});
            qf[dk] = t;
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the slice is read before the wave passes its next barrier
    };
    if (grp == 0) {
        q_request();
        q_read();
    } else {
        q_request();
        wait_vmcnt<32 * G::kRow / 1024>();   // this wave's parts of K(0), K(1); its query rows are still in flight
    }

    constexpr int kNO = D / 32;   // 32-wide d blocks of the accumulator
    f32x16 o[kNO];
#pragma unroll
    for (int db = 0; db < kNO; db++)
#pragma unroll
        for (int i = 0; i < 16; i++) o[db][i] = 0.f;
    SoftmaxOffState st;
    st.init();
    // the C operand every S block starts from: minus the lane's softmax offset (zero until the first rescale)
    f32x16 s_init;
#pragma unroll
    for (int i = 0; i < 16; i++) s_init[i] = 0.f;
    f32x16 s0[2], s1[2];
    bf16x8 pb0[4], pb1[4];     // P of the previous pair of tiles (first read in phase 1; defined from the start)
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int x = 0; x < 8; x++) {
            pb0[t][x] = (__bf16)0.0f;
            pb1[t][x] = (__bf16)0.0f;
        }

    typename Dma::Prepared dk0 = target_k(2), dk1 = target_k(3), dv0 = target_v(0), dv1 = target_v(1);
    // Per-lane LDS addresses of the operand fragments of the first tile of the pair a matrix phase reads: K tiles
    // 2m, 2m+1 sit in buffers 2 (m & 1) + {0, 1}, V tiles 2m-2, 2m-1 in buffers 2 (1 - m & 1) + {0, 1}, so every
    // phase flips one bit (two tiles' worth) in each register instead of adding a buffer base to every read.
    const lds_u8* ka[D / 16];
    const lds_u8* va[D / 32];
#pragma unroll
    for (int dk = 0; dk < D / 16; dk++) ka[dk] = smem + (rb.k ^ (dk << 5));
#pragma unroll
    for (int db = 0; db < D / 32; db++) va[db] = smem + ((rb.v ^ (db << 6)) + (kRing2 + 2) * kTileBytes);
    // (the ring starts at LDS address 0 and spans a power of two, so flipping an address bit moves between buffers)
    auto flip = [](const lds_u8* q, unsigned bit) -> const lds_u8* {
        return (const lds_u8*)(__attribute__((address_space(3))) void*)(size_t)((unsigned)(size_t)q ^ bit);
    };

    block_barrier();                 // K(0), K(1) resident
    if (grp == 1) {                  // group 1 takes its query rows in slot 0, in which it has nothing else to do
        q_read();
        block_barrier();
    }

    // scores of walk position e: keys past the end (or a position past the walk) to -inf;
    // masked launches: keys this lane's query may not see to -inf, skipped when the whole
    // wave sees the whole tile
    auto mask_tile = [&](f32x16 (&s)[2], int e) {
        const int kv0 = kv0_of(e);
        if (e >= ne || kv0 + kBN > sk) {
            const int lim = e >= ne ? 0 : sk;
#pragma unroll
            for (int b = 0; b < 2; b++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int key = kv0 + 32 * b + 8 * (i >> 2) + 4 * h + (i & 3);
                    if (key >= lim) s[b][i] = NEG;
                }
        }
        if constexpr (MASKED) {
            const int kend = min(kv0 + kBN, sk);
            const bool lane_all = kend <= a_hi || kv0 >= c_lo || (kv0 >= w_lo && kend <= w_hi);
            if (__builtin_amdgcn_ballot_w64(!lane_all) != 0) {
#pragma unroll
                for (int b = 0; b < 2; b++)
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const int key = kv0 + 32 * b + 8 * (i >> 2) + 4 * h + (i & 3);
                        const bool vis = key < a_hi || key >= c_lo || (key >= w_lo && key < w_hi);
                        if (!vis) s[b][i] = NEG;
                    }
            }
        }
    };

    // The first phase of a walk has no previous pair to multiply: it is unrolled apart (part 0) and runs
    // the K groups only.
#pragma unroll
    for (int part = 0; part < 2; part++) {
    const bool first = part == 0;
    const int m_begin = part == 0 ? 0 : 1;
    const int m_end = part == 0 ? 1 : np;
#pragma unroll 1
    for (int m = m_begin; m < m_end; m++) {
        // ---- matrix phase: group 0 in slot 2m, group 1 in slot 2m+1 ----
        __builtin_amdgcn_s_setprio(1);
        constexpr int kAhead = MASKED ? 2 : 3;
        const int g0 = first ? D / 16 : 0;   // the first phase starts at the K groups
        // DMA issue slots: all of the phase's loads go out during the FIRST tile of the pair, one
        // instruction after each of its first groups, in the order the next phase reads the tiles
        // (V of its first tile, K of its first tile, then the second tile's). A load takes well over
        // a thousand cycles to land when every CU streams K/V; issued from the second tile's groups
        // they were still in flight at the end of the phase (330 cycles of every matrix phase
        // spent in the wait below, measured with shader-clock stamps).
        auto hook_dma = [&](int g) {
            g -= g0;
            if constexpr (kIt == 2) {
                if (g == 0) Dma::issue_prepared(dv0, 0);
                if (g == 1) Dma::issue_prepared(dv0, 1);
                if (g == 2) Dma::issue_prepared(dk0, 0);
                if (g == 3) Dma::issue_prepared(dk0, 1);
                if (g == 4) Dma::issue_prepared(dv1, 0);
                if (g == 5) Dma::issue_prepared(dv1, 1);
                if (g == 6) Dma::issue_prepared(dk1, 0);
                if (g == 7) Dma::issue_prepared(dk1, 1);
            } else {
                if (g == 0) Dma::issue_prepared(dv0, 0);
                if (g == 1) Dma::issue_prepared(dk0, 0);
                if (g == 2) Dma::issue_prepared(dv1, 0);
                if (g == 3) Dma::issue_prepared(dk1, 0);
            }
        };
        auto hook_none = [](int) {};
        // (dense launches address the fragments through the flipped pointers; on masked launches, whose phases
        // read ahead less, that measured 0.6 % slower than an add per fragment, so they keep the adds)
        if constexpr (MASKED) {
            if (first) {
                mfma_phase<false, kAhead, decltype(hook_dma)&, D>(vbuf(2 * m - 2), kbuf(2 * m), rb, pb0, o, qf, s0, s_init, hook_dma);
                mfma_phase<false, kAhead, decltype(hook_none)&, D>(vbuf(2 * m - 1), kbuf(2 * m + 1), rb, pb1, o, qf, s1, s_init, hook_none);
            } else {
                mfma_phase<true, kAhead, decltype(hook_dma)&, D>(vbuf(2 * m - 2), kbuf(2 * m), rb, pb0, o, qf, s0, s_init, hook_dma);
                mfma_phase<true, kAhead, decltype(hook_none)&, D>(vbuf(2 * m - 1), kbuf(2 * m + 1), rb, pb1, o, qf, s1, s_init, hook_none);
            }
        } else if (first) {
            mfma_phase<false, kAhead, decltype(hook_dma)&, D>(va, ka, 0, pb0, o, qf, s0, s_init, hook_dma);
            mfma_phase<false, kAhead, decltype(hook_none)&, D>(va, ka, kTileBytes, pb1, o, qf, s1, s_init, hook_none);
        } else {
            mfma_phase<true, kAhead, decltype(hook_dma)&, D>(va, ka, 0, pb0, o, qf, s0, s_init, hook_dma);
            mfma_phase<true, kAhead, decltype(hook_none)&, D>(va, ka, kTileBytes, pb1, o, qf, s1, s_init, hook_none);
        }
        __builtin_amdgcn_s_setprio(0);
        wait_vmcnt<0>();             // this wave's loads of this phase have landed
        __builtin_amdgcn_sched_barrier(0);
        block_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // ---- VALU phase: group 0 in slot 2m+1, group 1 in slot 2m+2 ----
        mask_tile(s0, 2 * m);
        mask_tile(s1, 2 * m + 1);
        if (FIXED && !first) softmax_tile_pair_fixed<!LOG2DOM>(s0, s1, st, sl2, pb0, pb1);
        else softmax_tile_pair_off<!LOG2DOM, kNO>(s0, s1, st, o, s_init, sl2, pb0, pb1);
        // P and the row sum must be complete before the barrier: without this the
        // compiler sinks the exponentials past it, into the matrix phase
        asm volatile("" ::"v"(pb0[0]), "v"(pb0[1]), "v"(pb0[2]), "v"(pb0[3]), "v"(pb1[0]), "v"(pb1[1]),
                     "v"(pb1[2]), "v"(pb1[3]), "v"(st.l_acc));
        if constexpr (!MASKED) {
#pragma unroll
            for (int dk = 0; dk < D / 16; dk++) ka[dk] = flip(ka[dk], 2 * kTileBytes);   // the other pair of K buffers
#pragma unroll
            for (int db = 0; db < D / 32; db++) va[db] = flip(va[db], 2 * kTileBytes);   // ... and of V buffers
        }
        dk0 = target_k(2 * m + 4);   // for matrix phase m+1
        dk1 = target_k(2 * m + 5);
        dv0 = target_v(2 * m + 2);
        dv1 = target_v(2 * m + 3);
        if (grp == 0 || m + 1 < np) {
            __builtin_amdgcn_sched_barrier(0);
            block_barrier();
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    }
    // O += P V of the last pair (their V landed before the last barrier both groups passed)
    pv_tile<D>(vbuf(2 * np - 2), rb.v, pb0, o);
    pv_tile<D>(vbuf(2 * np - 1), rb.v, pb1, o);

    if constexpr (FIXED) {
        // Did the fixed offset hold? Every row sum below 2^100 (its reciprocal a normal number with room to spare) and every accumulator finite
        // (x * 0 is NaN for an infinite or NaN x). One vote per wave through 8 words of LDS behind the rings.
        float chk = 0.f;
#pragma unroll
        for (int db = 0; db < kNO; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) chk = __builtin_fmaf(o[db][i], 0.f, chk);
        const bool lane_ok = (pair_sum(st.l_acc) < 0x1p+100f) && (chk == 0.f);
        auto* votes = (__attribute__((address_space(3))) unsigned*)(smem + 2 * kRing2 * kTileBytes);
        if (lane == 0) votes[wave] = __builtin_amdgcn_ballot_w64(!lane_ok) != 0 ? 1u : 0u;
        __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0): the vote is written before the barrier
        block_barrier();   // ... behind which every wave is past its last read of both rings
        const u32x4 v0 = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(votes);
        const u32x4 v1 = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(votes + 4);
        const unsigned any = v0[0] | v0[1] | v0[2] | v0[3] | v1[0] | v1[1] | v1[2] | v1[3];
        if (__builtin_amdgcn_readfirstlane(any) != 0) {
            if (tid == 0) atomicAdd(&g_exact_pass_reruns, 1ull);
            return false;
        }
    }

    const float l_tot = pair_sum(st.l_acc);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    const int row = wave * 32 + c32;
    if constexpr (!MASKED) {
        if (p.kv_split > 1) {
            // partial result of this split: O / l in f32 and log2 of the sum of 2^(s * sl2) it covers
            if (row < qlen) {
                const size_t prow = ((size_t)sp * (p.total / (p.nqt * p.kv_split)) + bh) * sq + q0 + row;
                float* po = p.part_o + prow * kD;
#pragma unroll
                for (int db = 0; db < kNO; db++)
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        f32x4 r;
#pragma unroll
                        for (int x = 0; x < 4; x++) r[x] = o[db][4 * g + x] * inv;
                        global_store<f32x4>(po + 32 * db + 8 * g + 4 * h, r);
                    }
                if (h == 0)
                    p.part_lse[prow] = l_tot > 0.f ? st.template log2_offset<!LOG2DOM>(sl2) + __builtin_log2f(l_tot) : NEG;
            }
            return true;
        }
    }
    if (out_is_bf16) {
        // bf16 rows through this wave's own 32 x 2D-byte slice of the K ring (every K read is behind the last
        // barrier and no load is in flight): scattered 8-byte pieces in, whole rows out, 16 bytes per
        // lane and 1 KB (D = 128) of consecutive output per store instruction
        constexpr int kRowB = 2 * kD, kCh = kRowB / 16;
        lds_u8* my = smem + wave * (32 * kRowB);
#pragma unroll
        for (int db = 0; db < kNO; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                f32x4 r;
#pragma unroll
                for (int x = 0; x < 4; x++) r[x] = o[db][4 * g + x] * inv;
                const bf16x4 rb4 = __builtin_convertvector(r, bf16x4);
                const int ch = (4 * db + g) ^ (c32 & (kCh - 1));
                *reinterpret_cast<__attribute__((address_space(3))) bf16x4*>(my + c32 * kRowB + (ch << 4) + 8 * h) = rb4;
            }
        // (same-wave LDS writes and reads complete in order; the compiler waits on the reads' data)
        constexpr int kRowsPer = 64 / kCh;           // rows one store instruction covers
        const int lr = lane / kCh, lc = lane % kCh;
        uint16_t* ob = out_bf16 + ((size_t)bh * sq + q0 + wave * 32) * kD;
#pragma unroll
        for (int i = 0; i < 32 / kRowsPer; i++) {
            const int rr = i * kRowsPer + lr;
            const u32x4 val = *reinterpret_cast<const __attribute__((address_space(3))) u32x4*>(
                my + rr * kRowB + ((lc ^ (rr & (kCh - 1))) << 4));
            if (wave * 32 + rr < qlen) global_store<u32x4>(ob + (size_t)rr * kD + lc * 8, val);
        }
    } else if (row < qlen) {
        const size_t base = ((size_t)bh * sq + q0 + row) * kD;
#pragma unroll
        for (int db = 0; db < kNO; db++)
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int d0 = 32 * db + 8 * g + 4 * h;
                f32x4 r;
#pragma unroll
                for (int x = 0; x < 4; x++) r[x] = o[db][4 * g + x] * inv;
                if (out_is_bf16) {
                    const bf16x4 rb4 = __builtin_convertvector(r, bf16x4);
                    global_store<bf16x4>(out_bf16 + base + d0, rb4);
                } else {
                    global_store<f32x4>(out_f32 + base + d0, r);
                }
            }
    }
    return true;
}

// The softmax offset rides in the C operand of the K Q^T MFMAs (softmax_tile_pair_off): a score costs one multiply,
// one exponential and one add. LOG2DOM: the call's scale * log2(e) is exactly 1 (scores are base-2 logarithms as
// they leave the MFMAs) and the multiply is gone too. FIXED (launches that write bf16 and whose queries all see key 0): the first pass keeps
// the offset of the first 128 keys (flash_item); the others keep the running max throughout.
template <bool MASKED, int D, bool LOG2DOM, bool FIXED>
__global__ __launch_bounds__(512, 2) void flash_fwd_pp2(const FlashParams p) {
    const int tid = threadIdx.x;
    int wave = __builtin_amdgcn_readfirstlane(tid >> 6), block = blockIdx.x;
    if constexpr (!FIXED) {
        flash_item<MASKED, D, LOG2DOM, false>(p, wave, tid & 63, block);
    } else {
        if (flash_item<MASKED, D, LOG2DOM, true>(p, wave, tid & 63, block)) return;
        // The second pass shares nothing with the first but two scalars: its inputs are made opaque (the lane
        // index counted anew from the execution mask, the kernel arguments read again from their segment, of which
        // FlashParams is the whole), so that the compiler keeps no value of the first pass alive for it. It runs
        // once in a blue moon; the first pass is the kernel.
        using ConstParams = const __attribute__((address_space(4))) FlashParams;
        ConstParams* again = (ConstParams*)__builtin_amdgcn_kernarg_segment_ptr();
        int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        asm volatile("" : "+v"(lane), "+s"(wave), "+s"(block), "+s"(again));
        flash_item<MASKED, D, LOG2DOM, false>(*again, wave, lane, block);
    }
}

// Merge of the split-KV partials: out[row] = sum_s w_s O_s / sum_s w_s with w_s = 2^(lse_s - max lse).
// One thread per (row, 4 d).
template <bool OUT16>
__global__ __launch_bounds__(256) void splitkv_merge_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_lse, void* __restrict__ out,
                                                            size_t rows, int d, int splits) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int d4 = d >> 2;
    if (i >= rows * d4) return;
    const size_t row = i / d4;
    const int c = (int)(i - row * d4) * 4;
    float m = neg_inf();
    for (int s = 0; s < splits; s++) m = __builtin_fmaxf(m, part_lse[(size_t)s * rows + row]);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float wsum = 0.f;
    if (m != neg_inf()) {
        for (int s = 0; s < splits; s++) {
            const float w = fast_exp2(part_lse[(size_t)s * rows + row] - m);
            const f32x4 o = *reinterpret_cast<const f32x4*>(part_o + ((size_t)s * rows + row) * d + c);
            wsum += w;
#pragma unroll
            for (int x = 0; x < 4; x++) acc[x] += w * o[x];
        }
    }
    const float inv = wsum > 0.f ? 1.f / wsum : 0.f;
#pragma unroll
    for (int x = 0; x < 4; x++) acc[x] *= inv;
    if constexpr (OUT16) {
        *reinterpret_cast<bf16x4*>((uint16_t*)out + row * d + c) = __builtin_convertvector(acc, bf16x4);
    } else {
        *reinterpret_cast<f32x4*>((float*)out + row * d + c) = acc;
    }
}

}  // namespace fv

extern "C" hipError_t fv_internal_launch_splitkv_merge(const float* part_o, const float* part_lse, void* out,
                                                       int out_is_bf16, size_t rows, int d, int splits,
                                                       hipStream_t st) {
    const size_t n = rows * (size_t)(d / 4), blocks = (n + 255) / 256;
    if (blocks == 0) return hipSuccess;
    if (out_is_bf16)
        hipLaunchKernelGGL(fv::splitkv_merge_kernel<true>, dim3((unsigned)blocks), dim3(256), 0, st, part_o, part_lse,
                           out, rows, d, splits);
    else
        hipLaunchKernelGGL(fv::splitkv_merge_kernel<false>, dim3((unsigned)blocks), dim3(256), 0, st, part_o, part_lse,
                           out, rows, d, splits);
    return hipGetLastError();
}

// ---- host launchers -------------------------------------------------------------

extern "C" int fv_internal_flash_block_m(void) { return fv::kPpBM; }

namespace {
// The kernel's dynamic LDS limit (128 KB at D = 128), once per device.
template <bool MASKED, int D, bool LOG2DOM, bool FIXED>
hipError_t flash_attr() {
    static std::atomic<unsigned long long> attr_done;
    constexpr int lds = 2 * fv::kRing2 * fv::TileGeo<D>::kTile + fv::kVoteBytes;
    return fv_set_max_lds_once((const void*)fv::flash_fwd_pp2<MASKED, D, LOG2DOM, FIXED>, lds, attr_done);
}
template <bool MASKED, int D, bool LOG2DOM, bool FIXED>
hipError_t launch_flash_as(const fv::FlashParams* p, hipStream_t stream) {
    constexpr int lds = 2 * fv::kRing2 * fv::TileGeo<D>::kTile + fv::kVoteBytes;
    hipError_t e = flash_attr<MASKED, D, LOG2DOM, FIXED>();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((fv::flash_fwd_pp2<MASKED, D, LOG2DOM, FIXED>), dim3(p->per_xcd * 8), dim3(512), lds, stream, *p);
    return hipGetLastError();
}
// FASTVIDEO_SDPA_RUNNING_MAX=1: every launch keeps the running max (no fixed-offset first pass).
bool running_max_forced() {
    static const bool v = [] {
        const char* e = getenv("FASTVIDEO_SDPA_RUNNING_MAX");
        return e && *e && strcmp(e, "0") != 0;
    }();
    return v;
}
// A call whose scale * log2(e) is exactly 1 (scale = ln 2: the caller folded the softmax scale into Q) runs
// the form without the per-score multiply.
std::atomic<unsigned long long> g_log2_domain_launches{0};
template <bool MASKED, int D, bool FIXED>
hipError_t launch_flash_fixed(const fv::FlashParams* p, hipStream_t stream) {
    if (p->sl2 != 1.0f) return launch_flash_as<MASKED, D, false, FIXED>(p, stream);
    g_log2_domain_launches.fetch_add(1, std::memory_order_relaxed);
    return launch_flash_as<MASKED, D, true, FIXED>(p, stream);
}
// Launches whose result is rounded to bf16 make their first pass with the fixed offset: on a row that one late
// key dominates, that key's P is then a rounded bf16 number instead of exactly 1 (up to 2^-8 relative on the row),
// which a bf16 result absorbs; f32 results keep the running max. Masked launches take it where every query sees
// key 0, the first key of every tile's walk, so that its offset is a score of its own: block-causal without a
// window or with sink blocks, and the VDN mask (rows before the video and frame 0 are visible to every query).
// Under a window without a sink a query's first visible key may lie anywhere in the walk: running max.
template <bool MASKED, int D>
hipError_t launch_flash(const fv::FlashParams* p, hipStream_t stream) {
    const bool offset_is_a_score = !MASKED || p->mask_mode == 2 || (p->mask_mode == 1 && (p->win == 0 || p->sink > 0));
    if (p->out_is_bf16 && offset_is_a_score && !running_max_forced()) return launch_flash_fixed<MASKED, D, true>(p, stream);
    return launch_flash_fixed<MASKED, D, false>(p, stream);
}
}  // namespace

extern "C" uint64_t fv_sdpa_log2_domain_launches(void) { return g_log2_domain_launches.load(std::memory_order_relaxed); }

extern "C" hipError_t fv_internal_exact_pass_reruns(unsigned long long* out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(fv::g_exact_pass_reruns), sizeof *out, 0, hipMemcpyDeviceToHost);
}

extern "C" hipError_t fv_internal_init_flash(void) {
    hipError_t e = flash_attr<false, 128, false, false>();
    if (e == hipSuccess) e = flash_attr<true, 128, false, false>();
    if (e == hipSuccess) e = flash_attr<false, 64, false, false>();
    if (e == hipSuccess) e = flash_attr<true, 64, false, false>();
    if (e == hipSuccess) e = flash_attr<false, 128, true, false>();
    if (e == hipSuccess) e = flash_attr<true, 128, true, false>();
    if (e == hipSuccess) e = flash_attr<false, 64, true, false>();
    if (e == hipSuccess) e = flash_attr<true, 64, true, false>();
    if (e == hipSuccess) e = flash_attr<false, 128, false, true>();
    if (e == hipSuccess) e = flash_attr<false, 64, false, true>();
    if (e == hipSuccess) e = flash_attr<false, 128, true, true>();
    if (e == hipSuccess) e = flash_attr<false, 64, true, true>();
    if (e == hipSuccess) e = flash_attr<true, 128, false, true>();
    if (e == hipSuccess) e = flash_attr<true, 64, false, true>();
    if (e == hipSuccess) e = flash_attr<true, 128, true, true>();
    if (e == hipSuccess) e = flash_attr<true, 64, true, true>();
    return e;
}

extern "C" hipError_t fv_internal_launch_flash(const fv::FlashParams* p, int masked, int d,
                                               hipStream_t stream) {
    if (d == 128) return masked ? launch_flash<true, 128>(p, stream) : launch_flash<false, 128>(p, stream);
    if (d == 64) return masked ? launch_flash<true, 64>(p, stream) : launch_flash<false, 64>(p, stream);
    return hipErrorInvalidValue;
}
