"""Producer / consumer either side of the SDPA call over the C ABI (mirrors
CudaTensor::qk_norm_rope_bhsd / split_heads_bhsd / merge_heads, rt/ops.rs:528-620, and
wan::fuse::qk_norm_rope, wan/fuse.rs:290-343). torch carries device memory only.
"""
import torch

from . import _lib

__all__ = ["qk_norm_rope_bhsd", "split_heads_bhsd", "merge_heads"]


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


def qk_norm_rope_bhsd(proj, col_off, heads, weight, rope=None, eps=1e-6, out_bf16=None):
    """proj [batch, seq, width] -> [batch, heads, seq, d]. out_bf16 (default: proj is bf16)
    selects the bf16 kernel with its rounding points; otherwise the f32 op."""
    batch, seq, width = proj.shape
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
    out = torch.empty((batch, heads, seq, d), device=proj.device, dtype=torch.bfloat16 if out_bf16 else torch.float32)
    _lib.check(_lib.lib().fv_qk_norm_rope_bhsd(proj.data_ptr(), x16, weight.data_ptr(), w16,
                                               cos.data_ptr() if cos is not None else None,
                                               sin.data_ptr() if sin is not None else None, out.data_ptr(),
                                               int(out_bf16), batch, seq, heads, d, width, col_off, eps, _stream()))
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
