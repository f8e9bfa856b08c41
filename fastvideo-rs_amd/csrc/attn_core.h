// Building blocks shared by the gfx950 attention kernels that stage K/V tiles
// with direct global->LDS loads (global_load_lds_dwordx4) into XOR-swizzled,
// unpadded [64 keys][128 d] bf16 tiles.
//
// LDS tile layout (16 KB): row r is 256 B = 16 chunks of 16 B; logical chunk c
// of row r lives at chunk position c ^ swz(r), with
//   K tiles: swz(r) = r & 15        (32 consecutive keys reading one chunk
//                                    column hit 16 distinct positions)
//   V tiles: swz(r) = (r & 3) << 2  (the 4 rows of a transposed 4x16 read land
//                                    in 4 disjoint 64 B bank groups)
// The LDS-DMA write puts lane i's 16 B at base + 16 i, so the swizzle is applied
// on the global side: lane i fetches the chunk that belongs at its position.
#pragma once
#include "fv_common.h"
#include <type_traits>

namespace fv {

constexpr int kTileRows = 64;
constexpr int kRowBytes = 256;
constexpr int kTileBytes = kTileRows * kRowBytes;   // 16 KB (head dim 128)

// Tile geometry by head dim D (128 or 64): rows of 2 D bytes, 16-byte chunks, and the XOR
// swizzles that make the operand reads bank-conflict free.
//   D = 128 (256 B rows, 16 chunks): K chunk ^ (row & 15); V chunk ^ ((row & 3) << 2).
//   D = 64  (128 B rows,  8 chunks): two rows share a 256 B bank line, so the K swizzle
//     advances every second row, chunk ^ ((row >> 1) & 7), and the V swizzle separates
//     rows j and j+2 of a transposed 4-row read, chunk ^ (((row >> 1) & 1) << 2).
template <int D>
struct TileGeo {
    static_assert(D == 128 || D == 64, "head dim 128 or 64");
    static constexpr int kRow = 2 * D;                   // bytes per row
    static constexpr int kTile = kTileRows * kRow;       // bytes per tile
    static constexpr int kChunks = kRow / 16;            // 16-byte chunks per row
    static constexpr int kRowsPerDma = 1024 / kRow;      // rows one wave-wide DMA instruction covers
    static constexpr int kDmaPerTile = kTile / 1024;
    static constexpr int kVGroups = D / 16;              // PV groups per tile (2 MFMAs each)
    static constexpr int kKGroups = D / 16;              // QK groups per tile
    static constexpr int kGroups = kVGroups + kKGroups;
    static FV_DEV int kswz(int r) { return D == 128 ? (r & 15) : ((r >> 1) & 7); }
    static FV_DEV int vswz(int r) { return D == 128 ? ((r & 3) << 2) : (((r >> 1) & 1) << 2); }
};

typedef __attribute__((address_space(1))) void glb_void;
typedef __attribute__((address_space(3))) void lds_void;

// LDS-DMA: one wave-wide `global_load_lds_dwordx4` copies, per lane i, 16 B from the lane's global
// address to LDS byte address lds_base + 16 i (lds_base wave-uniform, in m0). It is issued as inline
// asm so that the compiler's wait-count insertion does not serialise later LDS reads of OTHER buffers
// behind it; the kernels order these loads with wait_vmcnt<N>() + block_barrier() themselves.

// Workgroup barrier without the memory fences of __syncthreads() (a fence
// would wait for every outstanding LDS-DMA load, defeating the prefetch). LDS
// reads issued before it have been consumed by then (their MFMA waited on them).
FV_DEV void block_barrier() { asm volatile("s_barrier" ::: "memory"); }

// s_waitcnt vmcnt(N) alone (expcnt / lgkmcnt untouched), gfx9 encoding.
template <int N>
FV_DEV void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt is 6 bits");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// LDS-DMA with a wave-uniform 64-bit base (SGPR pair) + per-lane byte offset.
FV_DEV void lds_dma16_s(unsigned lds_base, const void* sbase_in, unsigned voff) {
    // pin the base to an SGPR pair even where the compiler's divergence analysis
    // (branches on the wave index) would otherwise place it in VGPRs
    const unsigned long long a = (unsigned long long)sbase_in;
    // (readfirstlane returns int: widen through unsigned, or a low half with bit 31 set
    // would sign-extend over the high half)
    const unsigned lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)a);
    const unsigned hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(a >> 32));
    const unsigned long long sbase = ((unsigned long long)hi << 32) | (unsigned long long)lo;
    asm volatile(
        "s_mov_b32 m0, %0\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %1, %2"
        :
        : "s"(lds_base), "v"(voff), "s"(sbase)
        : "memory");   // m0 is a reserved scratch register: the compiler sets it right before each of
                       // its own uses and keeps nothing live in it across statements
}

// Per-lane source offsets of the tile loads, computed once per kernel: a wave-wide
// DMA instruction moves 1 KB = 4 rows of 256 B (D = 128) or 8 rows of 128 B (D = 64);
// with NW waves sharing a 64-row tile a wave issues ITER = (tile KB) / NW of them;
// lane i fetches the 16 B chunk that belongs at its position of its row.
template <int NW, int D = 128>
struct TileDma {
    using G = TileGeo<D>;
    static constexpr int ITER = G::kDmaPerTile / NW;
    static_assert(ITER >= 1, "more waves than DMA instructions per tile");
    unsigned koff[ITER];   // byte offset from the tile's first row, K swizzle
    unsigned voff[ITER];   // same, V swizzle
    FV_DEV void init(int wave, int lane) {
        const int p = lane % G::kChunks;
#pragma unroll
        for (int it = 0; it < ITER; it++) {
            const int r = (wave * ITER + it) * G::kRowsPerDma + lane / G::kChunks;
            koff[it] = r * G::kRow + ((p ^ G::kswz(r)) << 4);
            voff[it] = r * G::kRow + ((p ^ G::vswz(r)) << 4);
        }
    }
    // A tile load prepared ahead of its issue: everything the DMA instructions need,
    // so that issuing them from inside a matrix phase costs 3 instructions each.
    struct Prepared {
        unsigned long long base;   // wave-uniform global address of the tile's first row
        unsigned lds;              // wave-uniform LDS byte address of this wave's first row
        unsigned off[ITER];        // per-lane byte offsets (tail rows clamped)
    };
    template <bool IS_V>
    FV_DEV Prepared prepare(lds_u8* buf, const uint16_t* tile_base, int rows_valid, int wave) const {
        Prepared d;
        d.base = (unsigned long long)tile_base;
        d.lds = __builtin_amdgcn_readfirstlane((unsigned)(size_t)buf + wave * ITER * 1024);
#pragma unroll
        for (int it = 0; it < ITER; it++) d.off[it] = IS_V ? voff[it] : koff[it];
        if (rows_valid < kTileRows) {
#pragma unroll
            for (int it = 0; it < ITER; it++) {
                const int over = max(0, (int)(d.off[it] / G::kRow) - (rows_valid - 1));
                d.off[it] -= over * G::kRow;
            }
        }
        return d;
    }
    static FV_DEV void issue_prepared(const Prepared& d, int it) {
        lds_dma16_s(d.lds + it * 1024, (const void*)d.base, d.off[it]);
    }
    // tile_base (wave-uniform) points at the tile's first row. Rows >= rows_valid
    // re-read the last valid row: the caller masks their scores to -inf, so their
    // content only has to be finite data the tensor already holds.
    // one of the ITER instructions of a full tile's load
    template <bool IS_V>
    FV_DEV void issue_one(lds_u8* buf, const uint16_t* tile_base, int wave, int it) const {
        const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)buf + wave * ITER * 1024);
        lds_dma16_s(base + it * 1024, tile_base, IS_V ? voff[it] : koff[it]);
    }
    template <bool IS_V>
    FV_DEV void issue(lds_u8* buf, const uint16_t* tile_base, int rows_valid, int wave) const {
        const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(size_t)buf + wave * ITER * 1024);
        if (rows_valid >= kTileRows) {
#pragma unroll
            for (int it = 0; it < ITER; it++)
                lds_dma16_s(base + it * 1024, tile_base, IS_V ? voff[it] : koff[it]);
        } else {
#pragma unroll
            for (int it = 0; it < ITER; it++) {
                const unsigned off = IS_V ? voff[it] : koff[it];
                const int over = max(0, (int)(off / G::kRow) - (rows_valid - 1));
                lds_dma16_s(base + it * 1024, tile_base, off - over * G::kRow);
            }
        }
    }
};

// Per-lane read bases into a swizzled tile.
struct TileReadBases {
    int k;   // K A-operand: ^ (dk << 5), + kb * 32 rows
    int v;   // V^T A-operand (transposed read): ^ (db << 6), + (16 t + 8 g) rows
};
template <int D = 128>
FV_DEV TileReadBases tile_read_bases(int lane) {
    using G = TileGeo<D>;
    const int h = lane >> 5, c32 = lane & 31;
    const int b16 = lane >> 4, i16 = lane & 15;
    TileReadBases b;
    // K: lane reads logical chunk 2 dk + h of row c32 (+32): physical (2 dk + h) ^ kswz(row)
    b.k = c32 * G::kRow + ((G::kswz(c32) ^ h) << 4);
    // V^T: lane reads 8 bytes at d = 32 db + 16 (b16 & 1) + 4 (i16 & 3) of row 4 h + i16/4 (+16 t, +8)
    const int r = 4 * h + (i16 >> 2);
    const int c_lane = 2 * (b16 & 1) + ((i16 & 3) >> 1);
    b.v = r * G::kRow + ((G::vswz(r) ^ c_lane) << 4) + 8 * (i16 & 1);
    return b;
}

// S^T (64 keys x 32 queries) = K Q^T for one wave: s[b][i] is key
// 32 b + 8 (i/4) + 4 (lane/32) + i%4 of the tile, query lane%32.
FV_DEV void qk_tile(const lds_u8* kb, int k_base, const bf16x8 (&qf)[8], f32x16 (&s)[2]) {
#pragma unroll
    for (int b = 0; b < 2; b++) {
#pragma unroll
        for (int i = 0; i < 16; i++) s[b][i] = 0.f;
#pragma unroll
        for (int dk = 0; dk < 8; dk++) {
            const bf16x8 a = lds_read_b128(kb + (k_base ^ (dk << 5)) + b * 32 * kRowBytes);
            s[b] = mfma32(a, qf[dk], s[b]);
        }
    }
}

// qk_tile with `side(g)` after MFMA g (0..15): side work that rides under the matrix pipe. Every S block
// starts from `s_init` (the C operand of its first MFMA): zeros, or minus the softmax offset of the lane's query.
template <class Side>
FV_DEV void qk_tile_side(const lds_u8* kb, int k_base, const bf16x8 (&qf)[8], f32x16 (&s)[2], const f32x16& s_init,
                         Side&& side) {
#pragma unroll
    for (int b = 0; b < 2; b++) {
#pragma unroll
        for (int dk = 0; dk < 8; dk++) {
            const bf16x8 a = lds_read_b128(kb + (k_base ^ (dk << 5)) + b * 32 * kRowBytes);
            s[b] = mfma32(a, qf[dk], dk == 0 ? s_init : s[b]);
            __builtin_amdgcn_sched_barrier(0);
            side(b * 8 + dk);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

constexpr float kRescaleLog2 = 6.0f;

// Online softmax in base 2 with the offset riding in the matrix pipe. The K Q^T MFMAs of every S block start from
// `negoff` (16 copies of minus the lane's offset, in raw score units) as their C operand, so the scores arrive as
// x = s - off and P = 2^(sl2 * x): one two-operand multiply and one v_exp_f32 per score, no three-operand
// multiply-add (measured on MI355X against P = exp2(fma(s, sl2, -m * sl2)): same cycles, 1.7 % less time on the
// long dense launches and 2.3 % on block-causal ones, which run at the chip's power limit). SCALED == false is
// the form for calls whose sl2 = scale * log2(e) is exactly 1 (the caller folded the softmax scale into Q, e.g.
// into the q RMSNorm output): the multiply is gone as well.
// State per lane (= per query; lanes l and l^32 hold the same query): `off` the offset, `r` the running max
// relative to it (-inf until the query has seen a finite score), `l_acc` the lane's share of the row sum.
// When sl2 * r exceeds kRescaleLog2 in some lane (or a query sees its first finite score) every lane moves its
// offset to its running max: l and O are scaled by 2^(-sl2 r), this phase's scores lose r, negoff is rewritten
// (wave-uniform branch, rare). The final O / l is exact for any such policy: P and l always share an offset.
struct SoftmaxOffState {
    float r, off, l_acc;
    FV_DEV void init() {
        r = neg_inf();
        off = 0.f;
        l_acc = 0.f;
    }
    // base-2 logarithm of the row sum's scale: sum_k 2^(sl2 s_k) = l * 2^(sl2 off)
    template <bool SCALED>
    FV_DEV float log2_offset(float sl2) const { return SCALED ? off * sl2 : off; }
};

// The rescale decision and its (rare) execution for NS score blocks of 16: returns nothing, updates st, o, the
// scores and negoff. mx: the lane pair's max over this phase's scores (relative to the offset).
template <bool SCALED, int NO, int NS>
FV_DEV void softmax_off_rescale(float mx, SoftmaxOffState& st, f32x16 (&o)[NO], f32x16& negoff, float sl2,
                                f32x16* const (&sc)[NS]) {
    const float NEG = neg_inf();
    const float r_new = __builtin_fmaxf(st.r, mx);
    const bool need = ((SCALED ? r_new * sl2 : r_new) > kRescaleLog2) || (st.r == NEG && r_new != NEG);
    if (__builtin_amdgcn_ballot_w64(need) != 0) {
        const float delta = (r_new == NEG) ? 0.f : r_new;
        const float alpha = (st.r == NEG) ? 0.f : fast_exp2(SCALED ? -delta * sl2 : -delta);
        st.l_acc *= alpha;
#pragma unroll
        for (int db = 0; db < NO; db++)
#pragma unroll
            for (int i = 0; i < 16; i++) o[db][i] *= alpha;
#pragma unroll
        for (int b = 0; b < NS; b++)
#pragma unroll
            for (int i = 0; i < 16; i++) (*sc[b])[i] -= delta;   // -inf stays -inf
        st.off += delta;
#pragma unroll
        for (int i = 0; i < 16; i++) negoff[i] = -st.off;
        st.r = (r_new == NEG) ? NEG : 0.f;
    } else {
        st.r = r_new;
    }
}

// 32 keys x 32 queries of scores (relative to the offset) to P: exponentials, row-sum share, bf16 pack (RNE).
// pb[t] is the B operand (16 key slots x 32 queries) of key group t.
template <bool SCALED>
FV_DEV void softmax_off_block(const f32x16& sb, SoftmaxOffState& st, float sl2, bf16x8& p_lo, bf16x8& p_hi) {
    f32x16 e;
#pragma unroll
    for (int i = 0; i < 16; i++) {
        e[i] = fast_exp2(SCALED ? sb[i] * sl2 : sb[i]);
        st.l_acc += e[i];
    }
    f32x8 f0, f1;
#pragma unroll
    for (int x = 0; x < 8; x++) {
        f0[x] = e[x];
        f1[x] = e[8 + x];
    }
    p_lo = __builtin_convertvector(f0, bf16x8);
    p_hi = __builtin_convertvector(f1, bf16x8);
}

// A pair of tiles (128 keys) with one shared max / rescale decision.
template <bool SCALED, int NO = 4>
FV_DEV void softmax_tile_pair_off(f32x16 (&s0)[2], f32x16 (&s1)[2], SoftmaxOffState& st, f32x16 (&o)[NO],
                                  f32x16& negoff, float sl2, bf16x8 (&pb0)[4], bf16x8 (&pb1)[4]) {
    float mx = s0[0][0];
#pragma unroll
    for (int i = 1; i < 16; i++) mx = __builtin_fmaxf(mx, s0[0][i]);
#pragma unroll
    for (int i = 0; i < 16; i++) mx = __builtin_fmaxf(mx, s0[1][i]);
#pragma unroll
    for (int b = 0; b < 2; b++)
#pragma unroll
        for (int i = 0; i < 16; i++) mx = __builtin_fmaxf(mx, s1[b][i]);
    mx = pair_max(mx);
    f32x16* const sc[4] = {&s0[0], &s0[1], &s1[0], &s1[1]};
    softmax_off_rescale<SCALED, NO, 4>(mx, st, o, negoff, sl2, sc);
#pragma unroll
    for (int b = 0; b < 2; b++) softmax_off_block<SCALED>(s0[b], st, sl2, pb0[2 * b], pb0[2 * b + 1]);
#pragma unroll
    for (int b = 0; b < 2; b++) softmax_off_block<SCALED>(s1[b], st, sl2, pb1[2 * b], pb1[2 * b + 1]);
}

// A pair of tiles with the offset left where it is: no row max, no rescale decision. For walks whose caller
// checks afterwards that no row sum outgrew the f32 range comfortably (and redoes the walk with
// softmax_tile_pair_off if one did).
template <bool SCALED>
FV_DEV void softmax_tile_pair_fixed(const f32x16 (&s0)[2], const f32x16 (&s1)[2], SoftmaxOffState& st, float sl2,
                                    bf16x8 (&pb0)[4], bf16x8 (&pb1)[4]) {
#pragma unroll
    for (int b = 0; b < 2; b++) softmax_off_block<SCALED>(s0[b], st, sl2, pb0[2 * b], pb0[2 * b + 1]);
#pragma unroll
    for (int b = 0; b < 2; b++) softmax_off_block<SCALED>(s1[b], st, sl2, pb1[2 * b], pb1[2 * b + 1]);
}

// One tile. `side(part)` runs after the rescale (part 0) and after each 32-key half of the exponentials
// (parts 1, 2): slots for side work, such as tile DMA issue, spread through the VALU stream.
template <bool SCALED, class Side>
FV_DEV void softmax_tile_side_off(f32x16 (&s)[2], SoftmaxOffState& st, f32x16 (&o)[4], f32x16& negoff, float sl2,
                                  bf16x8 (&pb)[4], Side&& side) {
    float mx = s[0][0];
#pragma unroll
    for (int i = 1; i < 16; i++) mx = __builtin_fmaxf(mx, s[0][i]);
#pragma unroll
    for (int i = 0; i < 16; i++) mx = __builtin_fmaxf(mx, s[1][i]);
    mx = pair_max(mx);
    f32x16* const sc[2] = {&s[0], &s[1]};
    softmax_off_rescale<SCALED, 4, 2>(mx, st, o, negoff, sl2, sc);
    side(0);
#pragma unroll
    for (int b = 0; b < 2; b++) {
        softmax_off_block<SCALED>(s[b], st, sl2, pb[2 * b], pb[2 * b + 1]);
        side(1 + b);
    }
}

// O^T (128 d x 32 queries) += V^T P^T.
template <int D = 128>
FV_DEV void pv_tile(const lds_u8* vb, int v_base, const bf16x8 (&pb)[4], f32x16 (&o)[D / 32]) {
    constexpr int kRow = TileGeo<D>::kRow;
#pragma unroll
    for (int t = 0; t < 4; t++) {
#pragma unroll
        for (int db = 0; db < D / 32; db++) {
            const int a0 = (v_base ^ (db << 6)) + (16 * t) * kRow;
            const s16x4 lo = lds_read_tr16_b64(vb + a0);
            const s16x4 hi = lds_read_tr16_b64(vb + a0 + 8 * kRow);
            s16x8 a;
            a.lo = lo;
            a.hi = hi;
            o[db] = mfma32(__builtin_bit_cast(bf16x8, a), pb[t], o[db]);
        }
    }
}

// One MFMA phase with a deep, explicit LDS prefetch: O^T += V^T P^T of the
// previous tile (groups 0-7, if DO_PV) followed by S^T = K Q^T of the current
// one (groups 8-15). A group is 2 operand fragments (8 VGPRs) feeding 2 MFMAs on
// different accumulators; the first K MFMA of a key block takes `s_init` as its C operand (zeros, or minus the
// softmax offset of the lane's query). kAhead (2-3, bounded by the 256-VGPR budget) groups are always in flight ahead of the group
// being multiplied, so an MFMA waits on a read issued kAhead x 64 cycles of
// matrix-pipe time earlier instead of on LDS latency plus the 64 B/clk per-SIMD
// LDS return path. sched_barrier keeps the compiler from re-serialising reads
// behind MFMAs.
// The operand fragments are addressed through per-lane LDS pointers that already hold the buffer's place
// (`va[db]`: V^T fragments of d block db, `ka[dk]`: K fragments of d chunk dk, both for the FIRST tile of a pair;
// `tile_off` = 0 or one tile adds the second one as an immediate), so a read costs no address arithmetic.
template <bool DO_PV, int kAhead, class Hook, int D = 128>
FV_DEV void mfma_phase(const lds_u8* const (&va)[D / 32], const lds_u8* const (&ka)[D / 16], const int tile_off,
                       const bf16x8 (&pb)[4], f32x16 (&o)[D / 32], const bf16x8 (&qf)[D / 16],
                       f32x16 (&s)[2], const f32x16& s_init, Hook&& hook) {
    using G = TileGeo<D>;
    constexpr int NV = G::kVGroups, NG = G::kGroups;
    constexpr int G0 = DO_PV ? 0 : NV;
    constexpr int kPerT = D / 64;   // V groups per 16-key group t (each covers two 32-wide d blocks)
    bf16x8 f[NG][2];
    auto issue = [&](int g) {
        if (g < NV) {         // V^T fragments: key group t, d blocks 2*(g % kPerT) + {0, 1}
#pragma unroll
            for (int x = 0; x < 2; x++) {
                const int t = g / kPerT, db = 2 * (g % kPerT) + x;
                const lds_u8* a0 = va[db] + ((16 * t) * G::kRow + tile_off);
                s16x8 a;
                a.lo = lds_read_tr16_b64(a0);
                a.hi = lds_read_tr16_b64(a0 + 8 * G::kRow);
                f[g][x] = __builtin_bit_cast(bf16x8, a);
            }
        } else {              // K fragments: d chunk dk = g - NV, key blocks 0 and 1
#pragma unroll
            for (int x = 0; x < 2; x++)
                f[g][x] = lds_read_b128(ka[g - NV] + (x * 32 * G::kRow + tile_off));
        }
    };
    auto run = [&](int g) {
        if (g < NV) {
#pragma unroll
            for (int x = 0; x < 2; x++) {
                const int t = g / kPerT, db = 2 * (g % kPerT) + x;
                o[db] = mfma32(f[g][x], pb[t], o[db]);
            }
        } else {
#pragma unroll
            for (int x = 0; x < 2; x++)   // S is born at dk == 0, not before the PV part, from the C operand s_init
                s[x] = mfma32(f[g][x], qf[g - NV], g == NV ? s_init : s[x]);
        }
    };
#pragma unroll
    for (int g = G0; g < G0 + kAhead && g < NG; g++) issue(g);
#pragma unroll
    for (int g = G0; g < NG; g++) {
        if (g + kAhead < NG) issue(g + kAhead);
        __builtin_amdgcn_sched_barrier(0);
        run(g);
        __builtin_amdgcn_sched_barrier(0);
        hook(g);   // side work (tile DMA issue) that rides under the matrix pipe
    }
}

// mfma_phase for one tile given by its V and K buffers (wave-uniform) and the lane's read bases: the fragment
// addresses are formed here, an add per fragment.
template <bool DO_PV, int kAhead, class Hook, int D = 128>
FV_DEV void mfma_phase(const lds_u8* vb, const lds_u8* kb, const TileReadBases& rb,
                       const bf16x8 (&pb)[4], f32x16 (&o)[D / 32], const bf16x8 (&qf)[D / 16],
                       f32x16 (&s)[2], const f32x16& s_init, Hook&& hook) {
    const lds_u8* va[D / 32];
    const lds_u8* ka[D / 16];
#pragma unroll
    for (int db = 0; db < D / 32; db++) va[db] = vb + (rb.v ^ (db << 6));
#pragma unroll
    for (int dk = 0; dk < D / 16; dk++) ka[dk] = kb + (rb.k ^ (dk << 5));
    mfma_phase<DO_PV, kAhead, Hook, D>(va, ka, 0, pb, o, qf, s, s_init, static_cast<Hook&&>(hook));
}

// Q^T fragments for the wave's 32 queries: rows row0 + lane%32 of a row-major
// [rows][128] bf16 tensor; rows >= nrows read as zero.
template <int D = 128>
FV_DEV void load_q_frags(const uint16_t* q, int row, bool ok, int lane, bf16x8 (&qf)[D / 16]) {
    const uint16_t* src = q + (size_t)row * D + 8 * (lane >> 5);
#pragma unroll
    for (int dk = 0; dk < D / 16; dk++) {
        u32x4 t = {0u, 0u, 0u, 0u};
        if (ok) t = *reinterpret_cast<const u32x4*>(src + 16 * dk);
        qf[dk] = __builtin_bit_cast(bf16x8, t);
    }
    // Drain these (compiler-tracked) loads here: a wait the compiler would
    // otherwise place inside the main loop also counts the untracked LDS-DMA
    // loads in flight there and would stall on them.
    __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
}

}  // namespace fv
