// Launch parameter blocks and internal launcher prototypes shared by the kernel
// translation units and the C ABI (fv_api.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace fv {

struct FlashParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    float* out_f32;
    uint16_t* out_bf16;
    int out_is_bf16;
    int sq, sk;
    float sl2;          // scale * log2(e)
    int nqt;            // query tiles per (batch, head)
    int total;          // bh * nqt
    int per_xcd;        // ceil(total / 8)
    int mask_mode;      // 0 none, 1 block-causal, 2 VDN window
    int ft, win, sink;  // block-causal: block tokens, window blocks, sink blocks; VDN window: ft = frame tokens
    int vs, ve, frames, chunk, radius;   // VDN window: video rows [vs, ve), frame count, chunk, radius
    // elements between consecutive (batch, head) planes of q, k and v: s * d when contiguous, larger
    // when the operand is a row window of a longer plane (a KV cache read in place)
    long q_plane, k_plane, v_plane;
    // Split-KV (dense launches only): kv_split > 1 gives every (head, query tile) kv_split workgroups,
    // each walking split_tiles key tiles and writing its own normalised partial output (f32
    // [split][bh][sq][d]) and base-2 log-sum-exp ([split][bh][sq]) for the merge kernel.
    int kv_split, split_tiles;
    float* part_o;
    float* part_lse;
};

struct VsaFineParams {
    const uint16_t* qt;           // tile-ordered bf16 [bh, nb*64, 128]
    const uint16_t* kt;
    const uint16_t* vt;
    const unsigned* selected;     // [bh, nb, topk]
    const int* block_sizes;       // [nb]
    float* out;                   // [bh, q_tiles*64, 128] f32, tile-slot order
    int num_tiles, topk;
    float sl2;
    int q_base, q_tiles;          // query tiles [q_base, q_base + q_tiles)
    int total, per_xcd;           // bh * q_tiles, ceil(total / 8)
    // Fused combine (whole-op entry): when `final_out` is set the kernel writes
    // final_out[token] = coarse[tile] * gate[token] + sparse instead of `out`, in token order.
    float* final_out;             // [bh, seq, 128] f32 or null
    const float* coarse;          // [bh, num_tiles, 128]
    const void* gate;             // [bh, seq, 128] f32 / bf16 or null (gate of one)
    int gate_is_bf16;
    const int* slot_src;          // [num_tiles * 64]
    long seq;
};

// The key-tile walk of one query tile of a masked launch: up to three ascending, non-overlapping
// ranges of 64-key tiles, [0, n0), [a1, a1 + n1) and [a2, a2 + n2), ne = n0 + n1 + n2 tiles in all
// (ne == 0: no query of the tile sees any key). Every key visible to any query of the tile lies in
// a walked tile; which scores inside a walked tile count is decided per lane.
//   block-causal (rt/attn.rs:449-453): the sink tiles, then the band of the tile's blocks;
//   VDN window (rt/attn.rs:483-510): rows before the video + frame 0, the window frames of the
//   tile, the last frame + rows after the video; a tile holding an anchor / global row walks all.
struct TileWalk {
    int a1, a2, n0, n1, ne;
};
// (Params: FlashParams, or the same struct read through another address space)
template <class Params>
__host__ __device__ inline TileWalk mask_tile_walk(const Params& p, int q0, int qlen, int nkt) {
    constexpr int kKeys = 64;
    const int sk = p.sk;
    auto imin = [](int a, int b) { return a < b ? a : b; };
    auto imax = [](int a, int b) { return a > b ? a : b; };
    int a1 = 0, a2 = 0, b0, b1, b2 = 0;
    if (p.mask_mode == 1) {
        const int ft = p.ft, win = p.win;
        const int fq_lo = q0 / ft, fq_hi = (q0 + qlen - 1) / ft;
        const long hi_l = (long)(fq_hi + 1) * ft;
        const int hi_tok = (int)(hi_l < (long)sk ? hi_l : (long)sk);
        const int lo_tok = imin(hi_tok, win > 0 ? imax(0, fq_lo - win + 1) * ft : 0);
        const long sink_l = (long)p.sink * ft;
        const int sink_tok = (int)(sink_l < (long)sk ? sink_l : (long)sk);
        b0 = (sink_tok + kKeys - 1) / kKeys;
        a1 = lo_tok / kKeys;
        b1 = (hi_tok + kKeys - 1) / kKeys;
    } else {
        const int vs = p.vs, ve = p.ve, t = p.ft, last = p.frames - 1, c = p.chunk, r = p.radius;
        auto lo_frame = [&](int f) { return imax(0, c > 0 ? (f / c - r) * c : f - r); };
        auto hi_frame = [&](int f) { return imin(last, c > 0 ? (f / c + r + 1) * c - 1 : f + r); };
        const bool inner_tile = q0 >= vs + t && q0 + qlen <= ve - t;   // frames 1 .. last-1 only
        if (inner_tile) {
            const int fmin = (q0 - vs) / t, fmax = (q0 + qlen - 1 - vs) / t;
            b0 = (vs + t + kKeys - 1) / kKeys;
            a1 = (vs + lo_frame(fmin) * t) / kKeys;
            b1 = (vs + (hi_frame(fmax) + 1) * t + kKeys - 1) / kKeys;
            a2 = (ve - t) / kKeys;
            b2 = nkt;
        } else {
            b0 = nkt;
            b1 = 0;
        }
    }
    // ranges may touch or overlap: each starts no earlier than the previous one ends
    b0 = imin(b0, nkt);
    a1 = imax(a1, b0);
    b1 = imin(imax(b1, a1), nkt);
    a2 = imax(a2, b1);
    b2 = imax(b2, a2);
    TileWalk w;
    w.a1 = a1;
    w.a2 = a2;
    w.n0 = b0;
    w.n1 = b1 - a1;
    w.ne = w.n0 + w.n1 + (imin(b2, nkt) - imin(a2, nkt));
    return w;
}

}  // namespace fv

extern "C" int fv_internal_flash_block_m(void);   // queries per workgroup of the flash kernel in use
extern "C" hipError_t fv_internal_launch_flash(const fv::FlashParams* p, int masked, int d,
                                               hipStream_t stream);
extern "C" hipError_t fv_internal_exact_pass_reruns(unsigned long long* out);
extern "C" hipError_t fv_internal_launch_tile_mean(const void* x, int x_is_bf16, const int* slot_src,
                                                   const int* block_sizes, float* out, size_t bh,
                                                   size_t seq, int dim, int num_tiles, int round16,
                                                   hipStream_t st);
extern "C" hipError_t fv_internal_launch_coarse(const float* qc, const float* kc, const float* vc,
                                                float* scores, float* coarse, size_t bh, int nb,
                                                int dim, float scale, hipStream_t st);
extern "C" hipError_t fv_internal_launch_topk(const float* scores, unsigned* out, int rows, int n, int k,
                                              hipStream_t st);
extern "C" hipError_t fv_internal_launch_tile_scan3(const void* const x[3], int x_is_bf16, const int* slot_src,
                                                    const int* block_sizes, uint16_t* const tiles[3],
                                                    float* const means[3], const float* copy_mul, size_t bh, size_t seq,
                                                    size_t padded, int num_tiles, hipStream_t st);
extern "C" hipError_t fv_internal_launch_tile_qkv(const void* x, int x_is_bf16, const int* slot_src,
                                                  uint16_t* xt, size_t bh, size_t seq, size_t padded,
                                                  int dim, hipStream_t st);
// 1 = launched, 0 = not this kernel's head dim / alignment, < 0 = -(hipError_t)
extern "C" int fv_internal_launch_composed_mfma(const float* q, const float* k, const float* v, const float* mask,
                                                long mask_bh_stride, float* out, size_t bh, int sq, int sk, int d,
                                                float scale, hipStream_t st);
extern "C" hipError_t fv_internal_launch_splitkv_merge(const float* part_o, const float* part_lse, void* out,
                                                       int out_is_bf16, size_t rows, int d, int splits,
                                                       hipStream_t st);
extern "C" hipError_t fv_internal_init_flash(void);
extern "C" hipError_t fv_internal_init_vsa(void);
extern "C" hipError_t fv_internal_launch_fine(const fv::VsaFineParams* p, hipStream_t st);
extern "C" hipError_t fv_internal_launch_combine(const float* sparse, const float* coarse,
                                                 const void* gate, int gate_is_bf16,
                                                 const int* slot_src, float* out, size_t bh,
                                                 size_t seq, int num_tiles, int q_base, int q_tiles,
                                                 int round16, hipStream_t st);

// Error plumbing of the C ABI (defined in fv_api.hip): the message is kept per thread.
int fv_fail_hip(hipError_t e, const char* what);   // returns -(int)e
int fv_decline(const char* why);                    // returns FV_DECLINED
int fv_invalid(const char* why);                    // returns -(int)hipErrorInvalidValue

// Raise a kernel's dynamic LDS limit once per device (the attribute belongs to the function
// on the current device). `done` holds one bit per device ordinal; concurrent first calls may
// both set the attribute, which is harmless.
inline hipError_t fv_set_max_lds_once(const void* fn, int bytes, std::atomic<unsigned long long>& done) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const unsigned long long bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}
