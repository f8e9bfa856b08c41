"""numpy-facing ctypes bindings over the C oracle (oracle/fv_oracle.c).

Test infrastructure only. Each wrapper keeps the C function's name without
the ``fvo_`` prefix; see fv_oracle.h for the reference citations.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfv_oracle.so")


def build(force=False):
    """Compile libfv_oracle.so with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libfv_oracle.so"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_f32p = C.POINTER(C.c_float)
_u16p = C.POINTER(C.c_uint16)
_u32p = C.POINTER(C.c_uint32)
_i32p = C.POINTER(C.c_int32)
_i64p = C.POINTER(C.c_int64)
_szp = C.POINTER(C.c_size_t)
_sz = C.c_size_t


def _declare(l):
    l.fvo_bf16_rne_bits.argtypes = [C.c_float]
    l.fvo_bf16_rne_bits.restype = C.c_uint16
    l.fvo_bf16_round.argtypes = [C.c_float]
    l.fvo_bf16_round.restype = C.c_float
    l.fvo_quantize_bf16.argtypes = [_f32p, _f32p, _sz]
    l.fvo_to_bf16_bits.argtypes = [_f32p, _u16p, _sz]
    l.fvo_from_bf16_bits.argtypes = [_u16p, _f32p, _sz]
    l.fvo_matmul.argtypes = [_f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, C.c_int]
    l.fvo_softmax_last.argtypes = [_f32p, _f32p, _sz, _sz]
    l.fvo_sdpa_composed.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz,
                                    C.c_float, C.c_int]
    l.fvo_sdpa_composed_rows.argtypes = [_f32p, _f32p, _f32p, _i64p, _i64p, _sz, _f32p, _sz,
                                         _sz, _sz, _sz, C.c_float, C.c_int]
    l.fvo_sdpa_f64.argtypes = [_f32p, _f32p, _f32p, _i64p, _f32p, _sz, _sz, _sz, _sz,
                               C.c_double, C.c_int]
    l.fvo_sdpa_f64_rows.argtypes = [_f32p, _f32p, _f32p, _i64p, _i64p, _sz, _f32p, _sz, _sz,
                                    _sz, _sz, C.c_double, C.c_int]
    l.fvo_block_causal_allows.argtypes = [_sz, _sz, _sz, _sz, _sz]
    l.fvo_block_causal_allows.restype = C.c_int
    l.fvo_block_causal_dense_mask.argtypes = [_sz, _sz, _sz, _sz, _sz, _f32p]
    l.fvo_block_causal_for.argtypes = [_sz, C.c_int64, _sz, _szp]
    l.fvo_block_causal_for.restype = C.c_int
    l.fvo_causal_temporal_mask.argtypes = [_szp, _sz, C.c_int64, _sz, _sz, _sz, _f32p]
    l.fvo_topk_for.argtypes = [C.c_double, _sz]
    l.fvo_topk_for.restype = _sz
    l.fvo_tile_plan.argtypes = [_sz, _sz, _sz, _szp, _i32p, _u32p, _u32p]
    l.fvo_tile_plan.restype = C.c_int
    l.fvo_vsa_attention_host.argtypes = [_f32p, _f32p, _f32p, _f32p, _i32p, _u32p, _sz, _sz,
                                         _sz, _sz, _sz, _sz, C.c_float, _f32p, _u32p]
    l.fvo_vsa_attention_host.restype = C.c_int
    l.fvo_sortable.argtypes = [C.c_float]
    l.fvo_sortable.restype = C.c_uint32
    l.fvo_topk_device_order.argtypes = [_f32p, _u32p, _sz, _sz, _sz]
    l.fvo_topk_host_order.argtypes = [_f32p, _u32p, _sz, _sz, _sz]
    l.fvo_vsa_tile_mean.argtypes = [_f32p, _i32p, _u32p, _f32p, _sz, _sz, _sz, _sz, C.c_int]
    l.fvo_vsa_combine.argtypes = [_f32p, _f32p, _f32p, _i32p, _f32p, _sz, _sz, _sz, _sz, _sz, _sz, C.c_int]
    l.fvo_vsa_coarse_scores.argtypes = [_f32p, _f32p, _f32p, _sz, _sz, _sz, C.c_float]
    l.fvo_shard_ranges.argtypes = [_sz, _sz, _szp]
    l.fvo_vdn_window_allows.argtypes = [_sz, _sz, _sz, _sz, _sz, _sz, _sz]
    l.fvo_vdn_window_allows.restype = C.c_int
    l.fvo_vdn_window_dense_mask.argtypes = [_sz, _sz, _sz, _sz, _sz, _sz, _sz, _f32p]
    for fn in (l.fvo_qk_norm_rope_bhsd, l.fvo_wan_qk_norm_rope16):
        fn.argtypes = [_f32p, _f32p, _f32p, _f32p, _f32p, _sz, _sz, _sz, _sz, _sz, _sz, C.c_float]
    l.fvo_split_heads_bhsd.argtypes = [_f32p, _f32p, _sz, _sz, _sz, _sz, _sz, _sz]
    l.fvo_merge_heads.argtypes = [_f32p, _f32p, _sz, _sz, _sz, _sz]


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t):
    return a.ctypes.data_as(t) if a is not None else None


def default_threads(bh):
    """The reference parallelises host matmul over batch*heads only (rayon)."""
    return max(1, min(int(bh), os.cpu_count() or 1))


# ---- bf16 -------------------------------------------------------------------

def bf16_rne_bits(x):
    return int(lib().fvo_bf16_rne_bits(C.c_float(x)))


def quantize_bf16(x):
    x = _f32(x)
    y = np.empty_like(x)
    lib().fvo_quantize_bf16(_p(x, _f32p), _p(y, _f32p), x.size)
    return y


def to_bf16_bits(x):
    x = _f32(x)
    y = np.empty(x.shape, dtype=np.uint16)
    lib().fvo_to_bf16_bits(_p(x, _f32p), _p(y, _u16p), x.size)
    return y


def from_bf16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.uint16)
    y = np.empty(x.shape, dtype=np.float32)
    lib().fvo_from_bf16_bits(_p(x, _u16p), _p(y, _f32p), x.size)
    return y


# ---- host tensor ops ----------------------------------------------------------

def matmul(a, b, threads=1):
    a, b = _f32(a), _f32(b)
    batch, m, k = a.shape
    _, k2, n = b.shape
    assert k == k2 and b.shape[0] == batch
    out = np.empty((batch, m, n), dtype=np.float32)
    lib().fvo_matmul(_p(a, _f32p), _p(b, _f32p), _p(out, _f32p), batch, m, k, n, threads)
    return out


def softmax_last(x):
    x = _f32(x)
    out = np.empty_like(x)
    width = x.shape[-1]
    lib().fvo_softmax_last(_p(x, _f32p), _p(out, _f32p), x.size // width, width)
    return out


def _bc(mask_bc):
    if mask_bc is None:
        return None
    return np.ascontiguousarray(mask_bc, dtype=np.int64)


def sdpa_composed(q, k, v, scale=None, mask=None, threads=None):
    """q [bh,sq,d], k/v [bh,sk,d]; mask None or additive [sq,sk]."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    bh, sq, d = q.shape
    sk = k.shape[1]
    scale = np.float32(1.0) / np.sqrt(np.float32(d)) if scale is None else np.float32(scale)
    m = _f32(mask) if mask is not None else None
    out = np.empty((bh, sq, d), dtype=np.float32)
    lib().fvo_sdpa_composed(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(m, _f32p),
                            _p(out, _f32p), bh, sq, sk, d, C.c_float(scale),
                            threads or default_threads(bh))
    return out


def sdpa_composed_rows(q, k, v, rows, scale=None, mask_bc=None, threads=None):
    q, k, v = _f32(q), _f32(k), _f32(v)
    bh, sq, d = q.shape
    sk = k.shape[1]
    scale = np.float32(1.0) / np.sqrt(np.float32(d)) if scale is None else np.float32(scale)
    rows = np.ascontiguousarray(rows, dtype=np.int64)
    bc = _bc(mask_bc)
    out = np.empty((bh, rows.size, d), dtype=np.float32)
    lib().fvo_sdpa_composed_rows(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(bc, _i64p),
                                 _p(rows, _i64p), rows.size, _p(out, _f32p), bh, sq, sk, d,
                                 C.c_float(scale), threads or default_threads(bh))
    return out


def sdpa_f64(q, k, v, scale=None, mask_bc=None, rows=None, threads=None):
    q, k, v = _f32(q), _f32(k), _f32(v)
    bh, sq, d = q.shape
    sk = k.shape[1]
    scale = 1.0 / np.sqrt(float(d)) if scale is None else float(scale)
    bc = _bc(mask_bc)
    threads = threads or (os.cpu_count() or 1)
    if rows is None:
        out = np.empty((bh, sq, d), dtype=np.float32)
        lib().fvo_sdpa_f64(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(bc, _i64p),
                           _p(out, _f32p), bh, sq, sk, d, scale, threads)
        return out
    rows = np.ascontiguousarray(rows, dtype=np.int64)
    out = np.empty((bh, rows.size, d), dtype=np.float32)
    lib().fvo_sdpa_f64_rows(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(bc, _i64p),
                            _p(rows, _i64p), rows.size, _p(out, _f32p), bh, sq, sk, d, scale,
                            threads)
    return out


# ---- block-causal ---------------------------------------------------------------

def block_causal_allows(block_tokens, window, sink, q, k):
    return bool(lib().fvo_block_causal_allows(block_tokens, window, sink, q, k))


def block_causal_dense_mask(block_tokens, window, sink, sq, sk):
    m = np.empty((sq, sk), dtype=np.float32)
    lib().fvo_block_causal_dense_mask(block_tokens, window, sink, sq, sk, _p(m, _f32p))
    return m


def block_causal_for(num_frames_per_block, local_attn_size, frame_tokens):
    out = (C.c_size_t * 3)()
    ok = lib().fvo_block_causal_for(num_frames_per_block, local_attn_size, frame_tokens, out)
    return tuple(int(x) for x in out) if ok else None


def causal_temporal_mask(patch, num_frames_per_block, local_attn_size, frames, height, width):
    p = (C.c_size_t * 3)(*patch)
    tf, hf, wf = frames // max(patch[0], 1), height // max(patch[1], 1), width // max(patch[2], 1)
    seq = tf * hf * wf
    m = np.empty((seq, seq), dtype=np.float32)
    lib().fvo_causal_temporal_mask(p, num_frames_per_block, local_attn_size, frames, height,
                                   width, _p(m, _f32p))
    return m


# ---- VSA ---------------------------------------------------------------------------

def topk_for(sparsity, num_tiles):
    return int(lib().fvo_topk_for(float(sparsity), num_tiles))


class TilePlan:
    """C/rt/vsa.rs:42-109."""

    def __init__(self, grid):
        t, h, w = grid
        dims = (C.c_size_t * 5)()
        if lib().fvo_tile_plan(t, h, w, dims, None, None, None) != 0:
            raise ValueError(f"vsa: empty grid {grid}")
        self.grid = tuple(grid)
        self.tiles = (int(dims[0]), int(dims[1]), int(dims[2]))
        self.seq, self.padded = int(dims[3]), int(dims[4])
        nb = self.tiles[0] * self.tiles[1] * self.tiles[2]
        self.slot_src = np.empty(self.padded, dtype=np.int32)
        self.token_slot = np.empty(self.seq, dtype=np.uint32)
        self.block_sizes = np.empty(nb, dtype=np.uint32)
        lib().fvo_tile_plan(t, h, w, dims, _p(self.slot_src, _i32p), _p(self.token_slot, _u32p),
                            _p(self.block_sizes, _u32p))

    @property
    def num_tiles(self):
        return self.block_sizes.size


def vsa_attention_host(q, k, v, gate, plan, topk, b, heads, dim, scale, return_selected=False):
    q, k, v = _f32(q).reshape(-1), _f32(k).reshape(-1), _f32(v).reshape(-1)
    want = b * heads * plan.seq * dim
    for name, buf in (("q", q), ("k", k), ("v", v)):
        if buf.size != want:
            raise ValueError(f"vsa: {name} has {buf.size} elements, want {want}")
    g = None
    if gate is not None:
        g = _f32(gate).reshape(-1)
        if g.size != want:
            raise ValueError("vsa: gate shape must match q")
    nb = plan.num_tiles
    topk = min(max(int(topk), 1), nb)
    out = np.empty(want, dtype=np.float32)
    sel = np.empty((b * heads, nb, topk), dtype=np.uint32) if return_selected else None
    lib().fvo_vsa_attention_host(_p(q, _f32p), _p(k, _f32p), _p(v, _f32p), _p(g, _f32p),
                                 _p(plan.slot_src, _i32p), _p(plan.block_sizes, _u32p), plan.seq,
                                 nb, topk, b, heads, dim, C.c_float(scale), _p(out, _f32p),
                                 _p(sel, _u32p))
    out = out.reshape(b * heads, plan.seq, dim)
    return (out, sel) if return_selected else out


def sortable(x):
    return int(lib().fvo_sortable(C.c_float(x)))


def _topk(fn, scores, k):
    scores = _f32(scores)
    rows, n = scores.reshape(-1, scores.shape[-1]).shape
    out = np.empty((rows, k), dtype=np.uint32)
    fn(_p(scores, _f32p), _p(out, _u32p), rows, n, k)
    return out


def topk_device_order(scores, k):
    return _topk(lib().fvo_topk_device_order, scores, k)


def topk_host_order(scores, k):
    return _topk(lib().fvo_topk_host_order, scores, k)


def vsa_tile_mean(x, plan, round16=False):
    x = _f32(x)
    bh, seq, dim = x.shape
    out = np.empty((bh, plan.num_tiles, dim), dtype=np.float32)
    lib().fvo_vsa_tile_mean(_p(x, _f32p), _p(plan.slot_src, _i32p), _p(plan.block_sizes, _u32p),
                            _p(out, _f32p), bh, seq, dim, plan.num_tiles, int(round16))
    return out


def vsa_combine(sparse, coarse, gate, plan, seq, round16=False, q_base=0, q_tiles=None, out=None):
    """C/rt/kernels/core.cu:803-835. sparse [bh, q_tiles*64, dim] tile-slot order, coarse [bh, nb, dim],
    gate [bh, seq, dim] or None; rows of `out` no tile covers keep their value (zeros if fresh)."""
    sparse, coarse = _f32(sparse), _f32(coarse)
    bh, nb, dim = coarse.shape
    q_tiles = nb - q_base if q_tiles is None else q_tiles
    gate = _f32(gate) if gate is not None else None
    out = np.zeros((bh, seq, dim), dtype=np.float32) if out is None else out
    lib().fvo_vsa_combine(_p(sparse, _f32p), _p(coarse, _f32p), _p(gate, _f32p) if gate is not None else None,
                          _p(plan.slot_src, _i32p), _p(out, _f32p), bh, seq, dim, nb, q_base, q_tiles, int(round16))
    return out


def vsa_coarse_scores(qc, kc, scale):
    qc, kc = _f32(qc), _f32(kc)
    bh, nb, dim = qc.shape
    out = np.empty((bh, nb, nb), dtype=np.float32)
    lib().fvo_vsa_coarse_scores(_p(qc, _f32p), _p(kc, _f32p), _p(out, _f32p), bh, nb, dim,
                                C.c_float(scale))
    return out


def shard_ranges(seq, world):
    w = max(world, 1)
    out = (C.c_size_t * (2 * w))()
    lib().fvo_shard_ranges(seq, world, out)
    return [(int(out[2 * r]), int(out[2 * r + 1])) for r in range(w)]


# ---- producer / consumer either side of the SDPA call ---------------------------------

def _qk(fn, proj, col_off, heads, w, rope, eps):
    proj, w = _f32(proj), _f32(w)
    batch, seq, src_width = proj.shape
    d = w.size // heads
    cos = sin = None
    if rope is not None:
        cos, sin = _f32(rope[0]), _f32(rope[1])
        assert cos.shape == (seq, d) and sin.shape == (seq, d)
    out = np.empty((batch, heads, seq, d), dtype=np.float32)
    fn(_p(proj, _f32p), _p(w, _f32p), _p(cos, _f32p), _p(sin, _f32p), _p(out, _f32p), batch, seq, heads, d,
       src_width, col_off, eps)
    return out


def qk_norm_rope_bhsd(proj, col_off, heads, w, rope=None, eps=1e-6):
    """rt/ops.rs:2304-2350 (f32 op). proj [batch, seq, src_width], w [heads*d], rope (cos, sin) [seq, d]."""
    return _qk(lib().fvo_qk_norm_rope_bhsd, proj, col_off, heads, w, rope, eps)


def wan_qk_norm_rope16(proj, col_off, heads, w, rope=None, eps=1e-6):
    """wan/fuse.rs:290-343 host twin (bf16 rounding points of WAN_QK_NORM_ROPE)."""
    return _qk(lib().fvo_wan_qk_norm_rope16, proj, col_off, heads, w, rope, eps)


def split_heads_bhsd(proj, col_off, heads, d):
    proj = _f32(proj)
    batch, seq, src_width = proj.shape
    out = np.empty((batch, heads, seq, d), dtype=np.float32)
    lib().fvo_split_heads_bhsd(_p(proj, _f32p), _p(out, _f32p), batch, seq, heads, d, src_width, col_off)
    return out


def merge_heads(x):
    x = _f32(x)
    batch, heads, seq, d = x.shape
    out = np.empty((batch, seq, heads * d), dtype=np.float32)
    lib().fvo_merge_heads(_p(x, _f32p), _p(out, _f32p), batch, heads, seq, d)
    return out


# ---- VDN-H3 window mask ------------------------------------------------------------------

def vdn_window_allows(video_start, frame_tokens, frames, chunk, radius, q, k):
    return bool(lib().fvo_vdn_window_allows(video_start, frame_tokens, frames, chunk, radius, q, k))


def vdn_window_dense_mask(video_start, frame_tokens, frames, chunk, radius, sq, sk):
    m = np.empty((sq, sk), dtype=np.float32)
    lib().fvo_vdn_window_dense_mask(video_start, frame_tokens, frames, chunk, radius, sq, sk, _p(m, _f32p))
    return m
