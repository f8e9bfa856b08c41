// C ABI of the VSA stages and the whole VSA op, plus the host-side geometry
// (tile plan, top-k rule, block-causal predicate, shard ranges). Declarations
// and reference citations live in include/fv_sdpa_hip.h.
#include "../../include/fv_sdpa_hip.h"

#include <limits.h>
#include <math.h>
#include <stdlib.h>

#include "fv_internal.h"

namespace {

constexpr size_t kTile = 64;
constexpr size_t kTopkMaxN = 4096;

bool fits_int(size_t x) { return x <= (size_t)INT_MAX; }
size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct VsaWorkspace {
    size_t qc, kc, vc, scores, coarse, selected, qt, kt, vt, total;
};

VsaWorkspace vsa_layout(size_t bh, size_t nb, size_t topk, size_t dim) {
    VsaWorkspace w;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        const size_t at = off;
        off += align256(bytes);
        return at;
    };
    const size_t padded = nb * kTile;
    w.qc = take(bh * nb * dim * 4);
    w.kc = take(bh * nb * dim * 4);
    w.vc = take(bh * nb * dim * 4);
    w.scores = take(bh * nb * nb * 4);
    w.coarse = take(bh * nb * dim * 4);
    w.selected = take(bh * nb * topk * 4);
    w.qt = take(bh * padded * dim * 2);
    w.kt = take(bh * padded * dim * 2);
    w.vt = take(bh * padded * dim * 2);
    w.total = off;
    return w;
}

}  // namespace

extern "C" {

// ---- host geometry ------------------------------------------------------------------

// rt/envflag.rs:32-34 -> settings/parse.rs:43-45: the trimmed value through Rust's `str::parse::<f64>`, 0.8 when
// unset or unparsable. strtod takes two forms Rust's grammar does not (hex floats, "nan(...)"): refused here, so
// both sides fall back to the default on the same strings.
double fv_vsa_default_sparsity(void) {
    const char* v = getenv("FASTVIDEO_VSA_SPARSITY");
    if (!v) return 0.8;
    while (*v == ' ' || *v == '\t' || *v == '\n' || *v == '\r' || *v == '\v' || *v == '\f') v++;
    for (const char* c = v; *c; c++)
        if (*c == 'x' || *c == 'X' || *c == 'p' || *c == 'P' || *c == '(') return 0.8;
    char* end = nullptr;
    const double x = strtod(v, &end);
    if (end == v) return 0.8;
    while (*end == ' ' || *end == '\t' || *end == '\n' || *end == '\r' || *end == '\v' || *end == '\f') end++;
    return *end == '\0' ? x : 0.8;
}

size_t fv_vsa_topk_for(double sparsity, size_t num_tiles) {
    double keep = ceil((1.0 - sparsity) * (double)num_tiles);
    if (!(keep >= 1.0)) keep = 1.0;
    const size_t hi = num_tiles > 1 ? num_tiles : 1;
    return keep >= (double)hi ? hi : (size_t)keep;
}

int fv_vsa_tile_plan(size_t t, size_t h, size_t w, size_t dims_out[5], int32_t* slot_src,
                     uint32_t* token_slot, int32_t* block_sizes) {
    if (t == 0 || h == 0 || w == 0) return fv_invalid("vsa: empty grid");
    const size_t nt = (t + 3) / 4, nh = (h + 3) / 4, nw = (w + 3) / 4;
    const size_t nb = nt * nh * nw, seq = t * h * w, padded = nb * kTile;
    if (!fits_int(padded)) return fv_invalid("vsa: grid too large");
    if (dims_out) {
        dims_out[0] = nt;
        dims_out[1] = nh;
        dims_out[2] = nw;
        dims_out[3] = seq;
        dims_out[4] = padded;
    }
    if (!slot_src || !token_slot || !block_sizes) return FV_OK;
    for (size_t i = 0; i < padded; i++) slot_src[i] = -1;
    size_t tile = 0;
    for (size_t a = 0; a < nt; a++)
        for (size_t b = 0; b < nh; b++)
            for (size_t c = 0; c < nw; c++, tile++) {
                size_t slot = tile * kTile;
                for (size_t z = 4 * a; z < t && z < 4 * a + 4; z++)
                    for (size_t y = 4 * b; y < h && y < 4 * b + 4; y++)
                        for (size_t x = 4 * c; x < w && x < 4 * c + 4; x++, slot++) {
                            const size_t token = (z * h + y) * w + x;
                            slot_src[slot] = (int32_t)token;
                            token_slot[token] = (uint32_t)slot;
                        }
                block_sizes[tile] = (int32_t)(slot - tile * kTile);
            }
    return FV_OK;
}

int fv_block_causal_allows(size_t block_tokens, size_t window, size_t sink, size_t q, size_t k) {
    const size_t bt = block_tokens ? block_tokens : 1;
    const size_t tq = q / bt, tk = k / bt;
    if (tk < sink) return 1;
    return tk <= tq && (window == 0 || tq - tk < window);
}

void fv_block_causal_dense_mask(size_t block_tokens, size_t window, size_t sink, size_t sq,
                                size_t sk, float* mask) {
    for (size_t q = 0; q < sq; q++)
        for (size_t k = 0; k < sk; k++)
            mask[q * sk + k] = fv_block_causal_allows(block_tokens, window, sink, q, k) ? 0.0f : -1e9f;
}

int fv_vdn_window_allows(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                         size_t radius, size_t q, size_t k) {
    const size_t vs = video_start, ve = video_start + frames * frame_tokens, t = frame_tokens ? frame_tokens : 1;
    if (q < vs || q >= ve || k < vs || k >= ve) return 1;
    const size_t last = frames - 1;
    const size_t qf = (q - vs) / t, kf = (k - vs) / t;
    if (qf == 0 || kf == 0 || qf == last || kf == last) return 1;
    // a radius or chunk past the clip reaches every frame: clamped so that the products stay in range
    const long long f = (long long)qf, c = (long long)(chunk > frames ? frames : chunk),
                    r = (long long)(radius > frames ? frames : radius), kk = (long long)kf;
    const long long lo = c > 0 ? (f / c - r) * c : f - r;
    const long long hi = c > 0 ? (f / c + r + 1) * c - 1 : f + r;
    return kk >= lo && kk <= hi;
}

void fv_vdn_window_dense_mask(size_t video_start, size_t frame_tokens, size_t frames, size_t chunk,
                              size_t radius, size_t sq, size_t sk, float* mask) {
    for (size_t q = 0; q < sq; q++)
        for (size_t k = 0; k < sk; k++)
            mask[q * sk + k] =
                fv_vdn_window_allows(video_start, frame_tokens, frames, chunk, radius, q, k) ? 0.0f : -1e9f;
}

int fv_block_causal_tile_walk(size_t block_tokens, size_t window, size_t sink, size_t sq, size_t sk, size_t q0,
                              int out4[4]) {
    const size_t lim = (size_t)INT_MAX;
    const size_t bm = (size_t)fv_internal_flash_block_m();
    if (!out4) return fv_invalid("block_causal_tile_walk: null output");
    if (block_tokens == 0 || window > lim || sink > lim || sq == 0 || sk == 0 || q0 >= sq || q0 % bm != 0 ||
        (sq > sk ? sq : sk) + block_tokens > lim)
        return fv_decline("block_causal_tile_walk: parameters outside the kernel's range");
    fv::FlashParams p{};
    p.mask_mode = 1;
    p.sq = (int)sq;
    p.sk = (int)sk;
    p.ft = (int)block_tokens;
    p.win = (int)window;
    p.sink = (int)sink;
    const int qlen = (int)(sq - q0 < bm ? sq - q0 : bm);
    const fv::TileWalk w = fv::mask_tile_walk(p, (int)q0, qlen, (int)((sk + 63) / 64));
    out4[0] = w.n0;
    out4[1] = w.a1;
    out4[2] = w.n1;
    out4[3] = w.ne;
    return FV_OK;
}

int fv_block_causal_for(size_t num_frames_per_block, long long local_attn_size, size_t frame_tokens,
                        size_t out3[3]) {
    const size_t fpb = num_frames_per_block ? num_frames_per_block : 1;
    size_t window = 0;
    if (local_attn_size >= 0) {
        const size_t l = (size_t)local_attn_size;
        if (l == 0 || l % fpb != 0) return 0;
        window = l / fpb;
    }
    out3[0] = fpb * frame_tokens;
    out3[1] = window;
    out3[2] = 0;
    return 1;
}

void fv_sp_shard_ranges(size_t seq, size_t world, size_t* out) {
    if (world == 0) world = 1;
    size_t start = 0;
    for (size_t r = 0; r < world; r++) {
        const size_t len = seq / world + (r < seq % world ? 1 : 0);
        out[2 * r] = start;
        out[2 * r + 1] = len;
        start += len;
    }
}

// ---- device stages --------------------------------------------------------------------

int fv_vsa_tile_mean(const void* x, int x_is_bf16, const int32_t* slot_src, const int32_t* block_sizes,
                     float* out, size_t bh, size_t seq, size_t dim, size_t num_tiles, int round16,
                     void* stream) {
    if (!x || !block_sizes || !out) return fv_invalid("vsa_tile_mean: null operand");
    if (bh == 0 || num_tiles == 0) return FV_OK;
    if (dim == 0 || dim % 4 != 0 || !fits_int(dim) || !fits_int(num_tiles) || bh > 65535)
        return fv_decline("vsa_tile_mean: needs dim % 4 == 0 and bh <= 65535");
    hipError_t e = fv_internal_launch_tile_mean(x, x_is_bf16, slot_src, block_sizes, out, bh, seq, (int)dim,
                                                (int)num_tiles, round16, (hipStream_t)stream);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "vsa_tile_mean");
}

int fv_vsa_coarse(const float* qc, const float* kc, const float* vc, float* scores, float* coarse,
                  size_t bh, size_t num_tiles, size_t dim, float scale, void* stream) {
    if (!qc || !kc || !scores || (coarse && !vc)) return fv_invalid("vsa_coarse: null operand");
    if (bh == 0 || num_tiles == 0) return FV_OK;
    if (bh > 65535 || num_tiles > kTopkMaxN || !fits_int(dim) || (coarse && dim != 128))
        return fv_decline("vsa_coarse: needs bh <= 65535, num_tiles <= 4096, dim == 128");
    hipError_t e = fv_internal_launch_coarse(qc, kc, vc, scores, coarse, bh, (int)num_tiles, (int)dim, scale,
                                             (hipStream_t)stream);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "vsa_coarse");
}

int fv_vsa_topk(const float* scores, uint32_t* out, size_t rows, size_t n, size_t k, void* stream) {
    if (!scores || !out) return fv_invalid("vsa_topk: null operand");
    if (rows == 0 || k == 0) return FV_OK;
    if (n == 0 || n > kTopkMaxN || !fits_int(rows) || !fits_int(k))
        return fv_decline("vsa_topk: needs 1 <= n <= 4096");
    hipError_t e = fv_internal_launch_topk(scores, out, (int)rows, (int)n, (int)k, (hipStream_t)stream);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "vsa_topk");
}

int fv_vsa_tile_qkv(const void* x, int x_is_bf16, const int32_t* slot_src, uint16_t* xt, size_t bh,
                    size_t seq, size_t padded, size_t dim, void* stream) {
    if (!x || !slot_src || !xt) return fv_invalid("vsa_tile_qkv: null operand");
    if (bh == 0 || padded == 0) return FV_OK;
    if (dim == 0 || dim % 8 != 0 || !fits_int(dim) || bh > 65535 || !fits_int(padded * (dim / 8) / 256 + 1))
        return fv_decline("vsa_tile_qkv: needs dim % 8 == 0 and bh <= 65535");
    hipError_t e = fv_internal_launch_tile_qkv(x, x_is_bf16, slot_src, xt, bh, seq, padded, (int)dim,
                                               (hipStream_t)stream);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "vsa_tile_qkv");
}

int fv_vsa_fine(const uint16_t* qt, const uint16_t* kt, const uint16_t* vt, const uint32_t* selected,
                const int32_t* block_sizes, float* out, size_t bh, size_t num_tiles, size_t topk,
                size_t dim, float scale, size_t q_base, size_t q_tiles, void* stream) {
    if (!qt || !kt || !vt || !selected || !block_sizes || !out) return fv_invalid("vsa_fine: null operand");
    if (bh == 0 || q_tiles == 0) return FV_OK;
    if (dim != 128 || topk == 0 || topk > num_tiles || !fits_int(num_tiles * kTile) ||
        q_base + q_tiles > num_tiles || !(scale > 0.0f) || !(scale < 3.0e38f) ||
        bh * q_tiles > (size_t)INT_MAX / 2)
        return fv_decline("vsa_fine: needs dim == 128, 1 <= topk <= num_tiles, scale > 0");
    fv::VsaFineParams p;
    p.qt = qt;
    p.kt = kt;
    p.vt = vt;
    p.selected = selected;
    p.block_sizes = block_sizes;
    p.out = out;
    p.num_tiles = (int)num_tiles;
    p.topk = (int)topk;
    p.sl2 = scale * 1.4426950408889634f;
    p.q_base = (int)q_base;
    p.q_tiles = (int)q_tiles;
    p.total = (int)(bh * q_tiles);
    p.per_xcd = (p.total + 7) / 8;
    p.final_out = nullptr;
    p.coarse = nullptr;
    p.gate = nullptr;
    p.gate_is_bf16 = 0;
    p.slot_src = nullptr;
    p.seq = 0;
    hipError_t e = fv_internal_launch_fine(&p, (hipStream_t)stream);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "vsa_fine");
}

static int combine_common(const float* sparse, const float* coarse, const void* gate, int gate_is_bf16,
                          const int32_t* slot_src, float* out, size_t bh, size_t seq, size_t dim,
                          size_t num_tiles, size_t q_base, size_t q_tiles, int round16, void* stream) {
    if (!sparse || !coarse || !slot_src || !out) return fv_invalid("vsa_combine: null operand");
    if (bh == 0 || q_tiles == 0) return FV_OK;
    if (dim != 128 || bh > 65535 || !fits_int(num_tiles * kTile) || q_base + q_tiles > num_tiles)
        return fv_decline("vsa_combine: needs dim == 128 and bh <= 65535");
    hipError_t e = fv_internal_launch_combine(sparse, coarse, gate, gate_is_bf16, slot_src, out, bh, seq,
                                              (int)num_tiles, (int)q_base, (int)q_tiles, round16,
                                              (hipStream_t)stream);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "vsa_combine");
}

int fv_vsa_combine(const float* sparse, const float* coarse, const void* gate, int gate_is_bf16,
                   const int32_t* slot_src, float* out, size_t bh, size_t seq, size_t dim,
                   size_t num_tiles, size_t q_base, size_t q_tiles, void* stream) {
    return combine_common(sparse, coarse, gate, gate_is_bf16, slot_src, out, bh, seq, dim, num_tiles, q_base,
                          q_tiles, 0, stream);
}

int fv_vsa_combine_round16(const float* sparse, const float* coarse, const void* gate, int gate_is_bf16,
                           const int32_t* slot_src, float* out, size_t bh, size_t seq, size_t dim,
                           size_t num_tiles, size_t q_base, size_t q_tiles, void* stream) {
    return combine_common(sparse, coarse, gate, gate_is_bf16, slot_src, out, bh, seq, dim, num_tiles, q_base,
                          q_tiles, 1, stream);
}

size_t fv_vsa_workspace_bytes(size_t bh, size_t num_tiles, size_t topk, size_t dim) {
    return vsa_layout(bh, num_tiles, topk, dim).total;
}

// The whole op. tiled != 0: q/k/v are bf16 [bh, num_tiles*64, 128] already in tile-slot order (zero
// padding slots), so the tile means read them in place and the tile pass is skipped.
static int vsa_attention_common(const void* q, const void* k, const void* v, int qkv_is_bf16, int tiled,
                                const void* gate, int gate_is_bf16, const int32_t* slot_src,
                                const int32_t* block_sizes, float* out, void* workspace,
                                size_t workspace_bytes, uint32_t* selected_out, size_t bh, size_t seq,
                                size_t num_tiles, size_t topk, size_t dim, float scale, void* stream) {
    if (!q || !k || !v || !slot_src || !block_sizes || !out || !workspace)
        return fv_invalid("vsa_attention: null operand");
    if (topk < 1) topk = 1;                 // rt/vsa.rs:373 `topk.clamp(1, nb)`
    if (topk > num_tiles) topk = num_tiles;
    if (dim != 128 || num_tiles == 0 || num_tiles > kTopkMaxN || bh == 0 || bh > 65535)
        return fv_decline("vsa_attention: needs dim == 128, 1 <= num_tiles <= 4096, 1 <= bh <= 65535");
    const size_t padded = num_tiles * kTile;
    if (!(scale > 0.0f) || !(scale < 3.0e38f) || !fits_int(padded) || bh * num_tiles > (size_t)INT_MAX / 2)
        return fv_decline("vsa_attention: needs a finite scale > 0 and a tile count that fits one launch");
    const VsaWorkspace w = vsa_layout(bh, num_tiles, topk, dim);
    const size_t need = tiled ? w.qt : w.total;   // the tile-ordered copies are the tail of the layout
    if (workspace_bytes < need) return fv_invalid("vsa_attention: workspace too small (fv_vsa_workspace_bytes)");
    if (((uintptr_t)workspace & 255) != 0) return fv_invalid("vsa_attention: workspace must be 256-byte aligned");
    char* ws = (char*)workspace;
    float* qc = (float*)(ws + w.qc);
    float* kc = (float*)(ws + w.kc);
    float* vc = (float*)(ws + w.vc);
    float* scores = (float*)(ws + w.scores);
    float* coarse = (float*)(ws + w.coarse);
    uint32_t* sel = selected_out ? selected_out : (uint32_t*)(ws + w.selected);
    const uint16_t *qt = (const uint16_t*)q, *kt = (const uint16_t*)k, *vt = (const uint16_t*)v;
    hipStream_t st = (hipStream_t)stream;
    hipError_t e;
    int rc;
    bool fold = false;
    // 1 + 4. tile means (rt/vsa.rs:378-384) and the tile-ordered bf16 copies for the fine stage (rt/vsa.rs:406-414)
    //    of q, k and v in ONE scan: every token row is read once, written to its slot as bf16 and added, unrounded
    //    and in slot order, to its tile's mean. Operands that arrive tile-ordered are only pooled.
    {
        float* const means[3] = {qc, kc, vc};
        const void* const src[3] = {q, k, v};
        if (!tiled) {
            uint16_t* const tiles[3] = {(uint16_t*)(ws + w.qt), (uint16_t*)(ws + w.kt), (uint16_t*)(ws + w.vt)};
            // f32 queries get their one rounding here: with the fold switch on (fv_rt_fold_scale), of
            // q * (scale * log2 e), and the fine kernel then runs its form without the per-score multiply
            const float c = scale * 1.4426950408889634f;
            const float copy_mul[3] = {c, 1.0f, 1.0f};
            fold = !qkv_is_bf16 && fv_rt_fold_scale() && c != 1.0f && c < 3.0e38f;
            e = fv_internal_launch_tile_scan3(src, qkv_is_bf16, slot_src, block_sizes, tiles, means,
                                              fold ? copy_mul : nullptr, bh, seq, padded, (int)num_tiles, st);
            qt = tiles[0], kt = tiles[1], vt = tiles[2];
        } else {
            e = fv_internal_launch_tile_scan3(src, 1, nullptr, block_sizes, nullptr, means, nullptr, bh, padded, padded,
                                              (int)num_tiles, st);
        }
        if (e != hipSuccess) return fv_fail_hip(e, "vsa_tile_scan");
    }
    // 2. coarse attention over tiles; raw scores kept for the selection (rt/vsa.rs:385-394)
    if ((rc = fv_vsa_coarse(qc, kc, vc, scores, coarse, bh, num_tiles, dim, scale, stream))) return rc;
    // 3. top-k tiles per query tile (rt/vsa.rs:398-400)
    if ((rc = fv_vsa_topk(scores, sel, bh * num_tiles, num_tiles, topk, stream))) return rc;
    // 5. out = coarse * gate + sparse, back in token order: fused into the fine kernel's epilogue
    //    (no f32 sparse buffer: 2 x 200 MB of traffic and 200 MB of workspace less at Wan 480p)
    fv::VsaFineParams p;
    p.qt = qt;
    p.kt = kt;
    p.vt = vt;
    p.selected = sel;
    p.block_sizes = block_sizes;
    p.out = nullptr;
    p.num_tiles = (int)num_tiles;
    p.topk = (int)topk;
    p.sl2 = fold ? 1.0f : scale * 1.4426950408889634f;
    p.q_base = 0;
    p.q_tiles = (int)num_tiles;
    p.total = (int)(bh * num_tiles);
    p.per_xcd = (p.total + 7) / 8;
    p.final_out = out;
    p.coarse = coarse;
    p.gate = gate;
    p.gate_is_bf16 = gate_is_bf16;
    p.slot_src = slot_src;
    p.seq = (long)seq;
    e = fv_internal_launch_fine(&p, st);
    return e == hipSuccess ? FV_OK : fv_fail_hip(e, "vsa_fine (fused combine)");
}

int fv_vsa_attention(const void* q, const void* k, const void* v, int qkv_is_bf16, const void* gate,
                     int gate_is_bf16, const int32_t* slot_src, const int32_t* block_sizes, float* out,
                     void* workspace, size_t workspace_bytes, uint32_t* selected_out, size_t bh,
                     size_t seq, size_t num_tiles, size_t topk, size_t dim, float scale, void* stream) {
    return vsa_attention_common(q, k, v, qkv_is_bf16, 0, gate, gate_is_bf16, slot_src, block_sizes, out, workspace,
                                workspace_bytes, selected_out, bh, seq, num_tiles, topk, dim, scale, stream);
}

int fv_vsa_attention_tiled(const uint16_t* qt, const uint16_t* kt, const uint16_t* vt, const void* gate,
                           int gate_is_bf16, const int32_t* slot_src, const int32_t* block_sizes, float* out,
                           void* workspace, size_t workspace_bytes, uint32_t* selected_out, size_t bh,
                           size_t seq, size_t num_tiles, size_t topk, size_t dim, float scale, void* stream) {
    return vsa_attention_common(qt, kt, vt, 1, 1, gate, gate_is_bf16, slot_src, block_sizes, out, workspace,
                                workspace_bytes, selected_out, bh, seq, num_tiles, topk, dim, scale, stream);
}

}  // extern "C"
