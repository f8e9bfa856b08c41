"""Producer / consumer either side of the SDPA call over the C ABI (mirrors
CudaTensor::qk_norm_rope_bhsd / split_heads_bhsd / merge_heads, rt/ops.rs:528-620, and
wan::fuse::qk_norm_rope, wan/fuse.rs:290-343). torch carries device memory only.
"""
import torch

from . import _lib

__all__ = ["qk_norm_rope_bhsd", "split_heads_bhsd", "merge_heads", "qk_norm_rope_tiles", "split_heads_tiles"]


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _is16(t, name):
    if not (t.is_cuda and t.is_contiguous()):
        raise ValueError(f"{name}: want a contiguous CUDA tensor")
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise ValueError(f"{name}: want f32 or bf16")


def qk_norm_rope_bhsd(proj, col_off, heads, weight, rope=None, eps=1e-6, out_bf16=None, tiles=None, out=None,
                      out_mul=1.0):
    """proj [batch, seq, width] -> [batch, heads, seq, d]. out_bf16 (default: proj is bf16)
    selects the bf16 kernel with its rounding points; otherwise the f32 op. `tiles` (a VsaCtx): the
    head planes are written in the plan's tile-slot order, [batch, heads, padded, d], padding zero
    (`out`: a buffer from an earlier call, whose padding rows are zero already). `out_mul`: a factor on
    every output value, applied in f32 before the write (scale * log2(e) for an SDPA call at ln 2)."""
    batch, seq, width = proj.shape
    if tiles is not None and seq != tiles.seq:
        raise ValueError(f"qk norm: proj has {seq} tokens, the tile plan {tiles.seq}")
    if heads == 0 or weight.numel() % heads or col_off + weight.numel() > width:
        raise ValueError("qk norm: weight / columns")
    d = weight.numel() // heads
    cos = sin = None
    if rope is not None:
        cos, sin = rope
        for t in (cos, sin):
            if tuple(t.shape) != (seq, d) or t.dtype != torch.float32 or not t.is_cuda or not t.is_contiguous():
                raise ValueError(f"qk norm: rope tables must be contiguous f32 [{seq}, {d}]")
        if d % 2:
            raise ValueError("qk norm: rope needs an even head dim")
    x16, w16 = _is16(proj, "proj"), _is16(weight, "weight")
    out_bf16 = bool(x16) if out_bf16 is None else bool(out_bf16)
    odt = torch.bfloat16 if out_bf16 else torch.float32
    if tiles is not None:
        if out is None:
            out = torch.zeros((batch, heads, tiles.padded, d), device=proj.device, dtype=odt)
        elif tuple(out.shape) != (batch, heads, tiles.padded, d) or out.dtype != odt or not out.is_contiguous():
            raise ValueError("qk norm: out must be a contiguous [batch, heads, padded, d] tensor of the output type")
        _lib.check(_lib.lib().fv_qk_norm_rope_tiles(proj.data_ptr(), x16, weight.data_ptr(), w16,
                                                    cos.data_ptr() if cos is not None else None,
                                                    sin.data_ptr() if sin is not None else None, out.data_ptr(),
                                                    int(out_bf16), batch, seq, heads, d, width, col_off, eps,
                                                    float(out_mul), tiles.token_slot.data_ptr(), tiles.padded,
                                                    _stream()))
        return out
    out = torch.empty((batch, heads, seq, d), device=proj.device, dtype=odt)
    _lib.check(_lib.lib().fv_qk_norm_rope_bhsd(proj.data_ptr(), x16, weight.data_ptr(), w16,
                                               cos.data_ptr() if cos is not None else None,
                                               sin.data_ptr() if sin is not None else None, out.data_ptr(),
                                               int(out_bf16), batch, seq, heads, d, width, col_off, eps,
                                               float(out_mul), _stream()))
    return out


def qk_norm_rope_tiles(proj, col_off, heads, weight, ctx, rope=None, eps=1e-6, out_bf16=None, out=None, out_mul=1.0):
    """`qk_norm_rope_bhsd` writing VSA's tile-slot order directly (ctx: a VsaCtx)."""
    return qk_norm_rope_bhsd(proj, col_off, heads, weight, rope, eps, out_bf16, tiles=ctx, out=out, out_mul=out_mul)


def split_heads_tiles(proj, col_off, heads, d, ctx, out=None):
    """`split_heads_bhsd` writing VSA's tile-slot order: [batch, heads, padded, d], padding zero."""
    batch, seq, width = proj.shape
    if seq != ctx.seq:
        raise ValueError(f"split heads: proj has {seq} tokens, the tile plan {ctx.seq}")
    is16 = _is16(proj, "proj")
    if out is None:
        out = torch.zeros((batch, heads, ctx.padded, d), device=proj.device, dtype=proj.dtype)
    elif tuple(out.shape) != (batch, heads, ctx.padded, d) or out.dtype != proj.dtype or not out.is_contiguous():
        raise ValueError("split heads: out must be a contiguous [batch, heads, padded, d] tensor of proj's type")
    _lib.check(_lib.lib().fv_split_heads_tiles(proj.data_ptr(), out.data_ptr(), is16, batch, seq, heads, d, width,
                                               col_off, ctx.token_slot.data_ptr(), ctx.padded, _stream()))
    return out


def split_heads_bhsd(proj, col_off, heads, d):
    batch, seq, width = proj.shape
    is16 = _is16(proj, "proj")
    out = torch.empty((batch, heads, seq, d), device=proj.device, dtype=proj.dtype)
    _lib.check(_lib.lib().fv_split_heads_bhsd(proj.data_ptr(), out.data_ptr(), is16, batch, seq, heads, d, width,
                                              col_off, _stream()))
    return out


def merge_heads(x):
    batch, heads, seq, d = x.shape
    is16 = _is16(x, "x")
    out = torch.empty((batch, seq, heads * d), device=x.device, dtype=x.dtype)
    _lib.check(_lib.lib().fv_merge_heads(x.data_ptr(), out.data_ptr(), is16, batch, heads, seq, d, _stream()))
    return out
