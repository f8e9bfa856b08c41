"""VSA geometry and stage wrappers over the C ABI (mirrors rt/vsa.rs: TILE,
topk_for, TilePlan, VsaCtx, vsa_attention_device). Geometry runs in the
library's host code; stages run on the GPU. torch carries device memory only.
"""
import ctypes as C

import numpy as np
import torch

from . import _lib

TILE = (4, 4, 4)
TILE_ELEMS = 64

__all__ = ["TILE", "TILE_ELEMS", "topk_for", "TilePlan", "VsaCtx", "vsa_tile_mean", "vsa_coarse", "vsa_topk",
           "vsa_tile_qkv", "vsa_fine", "vsa_combine", "vsa_attention_device", "vsa_attention_tiled", "block_causal_allows",
           "block_causal_dense_mask", "block_causal_for", "shard_ranges"]


def _stream():
    return torch.cuda.current_stream().cuda_stream


def topk_for(sparsity, num_tiles):
    return int(_lib.lib().fv_vsa_topk_for(float(sparsity), num_tiles))


class TilePlan:
    """rt/vsa.rs:42-109: host arrays slot_src, token_slot, block_sizes."""

    def __init__(self, grid):
        t, h, w = grid
        dims = (C.c_size_t * 5)()
        rc = _lib.lib().fv_vsa_tile_plan(t, h, w, dims, None, None, None)
        if rc != 0:
            raise ValueError(f"vsa: empty grid {tuple(grid)}")
        self.grid = tuple(grid)
        self.tiles = (int(dims[0]), int(dims[1]), int(dims[2]))
        self.seq, self.padded = int(dims[3]), int(dims[4])
        nb = self.tiles[0] * self.tiles[1] * self.tiles[2]
        self.slot_src = np.empty(self.padded, dtype=np.int32)
        self.token_slot = np.empty(self.seq, dtype=np.uint32)
        self.block_sizes = np.empty(nb, dtype=np.int32)
        _lib.check(_lib.lib().fv_vsa_tile_plan(t, h, w, dims, self.slot_src.ctypes.data, self.token_slot.ctypes.data,
                                               self.block_sizes.ctypes.data))

    @property
    def num_tiles(self):
        return self.block_sizes.size


class VsaCtx:
    """rt/vsa.rs:326-347: the uploaded tiling and top-k of one latent grid."""

    def __init__(self, grid, sparsity=None, device="cuda"):
        if sparsity is None:     # wan/transformer.rs:2194: FASTVIDEO_VSA_SPARSITY, else 0.8
            sparsity = float(_lib.lib().fv_vsa_default_sparsity())
        self.sparsity = sparsity
        self.plan = TilePlan(grid)
        self.topk = topk_for(sparsity, self.plan.num_tiles)
        self.seq = self.plan.seq
        self.slot_src = torch.from_numpy(self.plan.slot_src).to(device)
        self.token_slot = torch.from_numpy(self.plan.token_slot.astype(np.int32)).to(device)   # u32 bits
        self.padded = self.plan.padded
        self.block_sizes = torch.from_numpy(self.plan.block_sizes).to(device)

    @property
    def num_tiles(self):
        return self.plan.num_tiles


def _is16(t):
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise ValueError("want f32 or bf16")


def _chk(t, name, dtypes=(torch.float32, torch.bfloat16)):
    if not (t.is_cuda and t.is_contiguous() and t.dtype in dtypes):
        raise ValueError(f"{name}: want a contiguous CUDA tensor of {dtypes}")


def vsa_tile_mean(x, ctx, round16=False, tiled=False):
    """`tiled`: x is already in tile-slot order, [bh, padded, dim]."""
    _chk(x, "x")
    bh, seq, dim = x.shape
    assert seq == (ctx.padded if tiled else ctx.seq)
    out = torch.empty((bh, ctx.num_tiles, dim), device=x.device, dtype=torch.float32)
    _lib.check(_lib.lib().fv_vsa_tile_mean(x.data_ptr(), _is16(x), None if tiled else ctx.slot_src.data_ptr(),
                                           ctx.block_sizes.data_ptr(),
                                           out.data_ptr(), bh, seq, dim, ctx.num_tiles, int(round16), _stream()))
    return out


def vsa_coarse(qc, kc, vc, scale, want_coarse=True):
    for n, t in (("qc", qc), ("kc", kc)):
        _chk(t, n, (torch.float32,))
    bh, nb, dim = qc.shape
    scores = torch.empty((bh, nb, nb), device=qc.device, dtype=torch.float32)
    coarse = torch.empty((bh, nb, dim), device=qc.device, dtype=torch.float32) if want_coarse else None
    _lib.check(_lib.lib().fv_vsa_coarse(qc.data_ptr(), kc.data_ptr(), vc.data_ptr() if vc is not None else None,
                                        scores.data_ptr(), coarse.data_ptr() if coarse is not None else None, bh, nb,
                                        dim, scale, _stream()))
    return scores, coarse


def vsa_topk(scores, k):
    _chk(scores, "scores", (torch.float32,))
    n = scores.shape[-1]
    rows = scores.numel() // n
    out = torch.empty(scores.shape[:-1] + (k,), device=scores.device, dtype=torch.int32)
    _lib.check(_lib.lib().fv_vsa_topk(scores.data_ptr(), out.data_ptr(), rows, n, k, _stream()))
    return out


def vsa_tile_qkv(x, ctx):
    _chk(x, "x")
    bh, seq, dim = x.shape
    padded = ctx.plan.padded
    out = torch.empty((bh, padded, dim), device=x.device, dtype=torch.bfloat16)
    _lib.check(_lib.lib().fv_vsa_tile_qkv(x.data_ptr(), _is16(x), ctx.slot_src.data_ptr(), out.data_ptr(), bh, seq,
                                          padded, dim, _stream()))
    return out


def vsa_fine(qt, kt, vt, selected, ctx, scale, q_base=0, q_tiles=None):
    for n, t in (("qt", qt), ("kt", kt), ("vt", vt)):
        _chk(t, n, (torch.bfloat16,))
    _chk(selected, "selected", (torch.int32,))
    bh, padded, dim = qt.shape
    nb = ctx.num_tiles
    assert padded == nb * TILE_ELEMS and kt.shape == qt.shape and vt.shape == qt.shape
    topk = selected.shape[-1]
    assert selected.shape == (bh, nb, topk)
    q_tiles = nb - q_base if q_tiles is None else q_tiles
    out = torch.empty((bh, q_tiles * TILE_ELEMS, dim), device=qt.device, dtype=torch.float32)
    _lib.check(_lib.lib().fv_vsa_fine(qt.data_ptr(), kt.data_ptr(), vt.data_ptr(), selected.data_ptr(),
                                      ctx.block_sizes.data_ptr(), out.data_ptr(), bh, nb, topk, dim, scale, q_base,
                                      q_tiles, _stream()))
    return out


def vsa_combine(sparse, coarse, gate, ctx, out=None, q_base=0, q_tiles=None, round16=False):
    """rt/ops.rs:1574-1601 `vsa_combine_device` / `vsa_combine_round_device` (`round16`: the H3
    family's bf16 combine, every step rounded to bf16)."""
    _chk(sparse, "sparse", (torch.float32,))
    _chk(coarse, "coarse", (torch.float32,))
    bh, nb, dim = coarse.shape
    q_tiles = nb - q_base if q_tiles is None else q_tiles
    if out is None:
        out = torch.zeros((bh, ctx.seq, dim), device=sparse.device, dtype=torch.float32)
    g16 = 0
    if gate is not None:
        _chk(gate, "gate")
        g16 = _is16(gate)
    entry = _lib.lib().fv_vsa_combine_round16 if round16 else _lib.lib().fv_vsa_combine
    _lib.check(entry(sparse.data_ptr(), coarse.data_ptr(), gate.data_ptr() if gate is not None else None,
                     g16, ctx.slot_src.data_ptr(), out.data_ptr(), bh, ctx.seq, dim, nb, q_base,
                     q_tiles, _stream()))
    return out


def vsa_attention_device(q, k, v, gate, ctx, scale, topk=None, return_selected=False):
    """rt/vsa.rs:358-424. q/k/v [bh, seq, 128] f32 or bf16 (same dtype); out f32."""
    for n, t in (("q", q), ("k", k), ("v", v)):
        _chk(t, n)
    if not (q.dtype == k.dtype == v.dtype and q.shape == k.shape == v.shape):
        raise ValueError("vsa: q, k, v must share dtype and shape")
    bh, seq, dim = q.shape
    if seq != ctx.seq:
        raise ValueError(f"vsa: q has {seq} tokens, the plan {ctx.seq}")
    if gate is not None:
        _chk(gate, "gate")
        if gate.shape != q.shape:
            raise ValueError("vsa: gate shape must match q")
    nb = ctx.num_tiles
    topk = min(max(int(ctx.topk if topk is None else topk), 1), nb)
    out = torch.empty((bh, seq, dim), device=q.device, dtype=torch.float32)
    nbytes = int(_lib.lib().fv_vsa_workspace_bytes(bh, nb, topk, dim))
    ws = torch.empty(nbytes, device=q.device, dtype=torch.uint8)
    sel = torch.empty((bh, nb, topk), device=q.device, dtype=torch.int32) if return_selected else None
    _lib.check(_lib.lib().fv_vsa_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), _is16(q),
                                           gate.data_ptr() if gate is not None else None,
                                           _is16(gate) if gate is not None else 0, ctx.slot_src.data_ptr(),
                                           ctx.block_sizes.data_ptr(), out.data_ptr(), ws.data_ptr(), nbytes,
                                           sel.data_ptr() if sel is not None else None, bh, seq, nb, topk, dim, scale,
                                           _stream()))
    return (out, sel) if return_selected else out


def vsa_attention_tiled(qt, kt, vt, gate, ctx, scale, topk=None, return_selected=False):
    """`vsa_attention_device` on q/k/v that a producer already wrote tile-ordered:
    qt/kt/vt bf16 [bh, padded, 128] with zero padding slots (`qk_norm_rope_tiles`, `split_heads_tiles`);
    gate and out stay in token order. Same result, bit for bit, as `vsa_attention_device` on the
    token-ordered bf16 tensors; the tile pass and its three buffers are not needed."""
    for n, t in (("qt", qt), ("kt", kt), ("vt", vt)):
        _chk(t, n, (torch.bfloat16,))
    bh, padded, dim = qt.shape
    if not (qt.shape == kt.shape == vt.shape) or padded != ctx.padded:
        raise ValueError(f"vsa: tile-ordered q, k, v must be [bh, {ctx.padded}, dim]")
    if gate is not None:
        _chk(gate, "gate")
        if tuple(gate.shape) != (bh, ctx.seq, dim):
            raise ValueError("vsa: gate must be [bh, seq, dim] in token order")
    nb = ctx.num_tiles
    topk = min(max(int(ctx.topk if topk is None else topk), 1), nb)
    out = torch.empty((bh, ctx.seq, dim), device=qt.device, dtype=torch.float32)
    nbytes = int(_lib.lib().fv_vsa_workspace_bytes(bh, nb, topk, dim))
    ws = torch.empty(nbytes, device=qt.device, dtype=torch.uint8)
    sel = torch.empty((bh, nb, topk), device=qt.device, dtype=torch.int32) if return_selected else None
    _lib.check(_lib.lib().fv_vsa_attention_tiled(qt.data_ptr(), kt.data_ptr(), vt.data_ptr(),
                                                 gate.data_ptr() if gate is not None else None,
                                                 _is16(gate) if gate is not None else 0, ctx.slot_src.data_ptr(),
                                                 ctx.block_sizes.data_ptr(), out.data_ptr(), ws.data_ptr(), nbytes,
                                                 sel.data_ptr() if sel is not None else None, bh, ctx.seq, nb, topk,
                                                 dim, scale, _stream()))
    return (out, sel) if return_selected else out


# ---- host helpers ------------------------------------------------------------------------

def block_causal_allows(block_tokens, window, sink, q, k):
    return bool(_lib.lib().fv_block_causal_allows(block_tokens, window, sink, q, k))


def block_causal_dense_mask(block_tokens, window, sink, sq, sk):
    m = np.empty((sq, sk), dtype=np.float32)
    _lib.lib().fv_block_causal_dense_mask(block_tokens, window, sink, sq, sk, m.ctypes.data)
    return m


def block_causal_for(num_frames_per_block, local_attn_size, frame_tokens):
    out = (C.c_size_t * 3)()
    ok = _lib.lib().fv_block_causal_for(num_frames_per_block, local_attn_size, frame_tokens, out)
    return tuple(int(x) for x in out) if ok else None


def shard_ranges(seq, world):
    w = max(world, 1)
    out = (C.c_size_t * (2 * w))()
    _lib.lib().fv_sp_shard_ranges(seq, world, out)
    return [(int(out[2 * r]), int(out[2 * r + 1])) for r in range(w)]
