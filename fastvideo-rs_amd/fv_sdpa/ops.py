"""torch-tensor wrappers over the kernel-level C ABI (include/fv_sdpa_hip.h).

Every wrapper validates on the host what the kernel assumes (device, dtype,
contiguity, shapes) before the launch.
"""
import math

import torch

from . import _lib

__all__ = ["sdpa_dense_bf16", "sdpa_dense_bf16_windows", "sdpa_dense_bf16_splitkv", "splitkv_choose", "sdpa_block_causal_bf16", "sdpa_vdn_window_bf16", "cast_f32_bf16", "cast_bf16_f32", "softmax_last", "sdpa_supported"]


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need(t, dtype, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous()):
        raise ValueError(f"{name}: want a contiguous CUDA tensor of {dtype}")


def _bhsd(q, k, v):
    for n, t in (("q", q), ("k", k), ("v", v)):
        _need(t, torch.bfloat16, n)
    if q.dim() != 3 or k.dim() != 3 or v.dim() != 3:
        raise ValueError("want [bh, s, d] operands")
    bh, sq, d = q.shape
    if k.shape != v.shape or k.shape[0] != bh or k.shape[2] != d:
        raise ValueError(f"k/v {tuple(k.shape)}/{tuple(v.shape)} do not match q {tuple(q.shape)}")
    return bh, sq, k.shape[1], d


def sdpa_supported(b, h, sq, sk, d):
    return bool(_lib.lib().fv_sdpa_supported(b, h, sq, sk, d))


def sdpa_dense_bf16(q, k, v, scale=None, out_bf16=False):
    bh, sq, sk, d = _bhsd(q, k, v)
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.empty((bh, sq, d), device=q.device, dtype=torch.bfloat16 if out_bf16 else torch.float32)
    _lib.check(_lib.lib().fv_sdpa_dense_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                             int(out_bf16), bh, sq, sk, d, scale, _stream()))
    return out


def _plane_rows(t, name):
    """Rows per plane of a [bh, s, d] bf16 tensor that is contiguous or a row window
    (`base[:, a:b]`) of a contiguous [bh, rows, d] tensor."""
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.bfloat16 and t.dim() == 3):
        raise ValueError(f"{name}: want a [bh, s, d] CUDA bf16 tensor")
    bh, s, d = t.shape
    sb, ss, sd = t.stride()
    if sd != 1 or ss != d or (bh > 1 and (sb % d or sb < s * d)):
        raise ValueError(f"{name}: want contiguous rows and one plane stride (a row window of a [bh, rows, d] tensor)")
    return sb // d if bh > 1 else s


def sdpa_dense_bf16_windows(q, k, v, scale=None, out_bf16=False):
    """`sdpa_dense_bf16` on row windows of longer planes (`cache[:, start:end]`), read in place."""
    rows = [_plane_rows(t, n) for t, n in ((q, "q"), (k, "k"), (v, "v"))]
    bh, sq, d = q.shape
    if k.shape != v.shape or k.shape[0] != bh or k.shape[2] != d:
        raise ValueError(f"k/v {tuple(k.shape)}/{tuple(v.shape)} do not match q {tuple(q.shape)}")
    sk = k.shape[1]
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.empty((bh, sq, d), device=q.device, dtype=torch.bfloat16 if out_bf16 else torch.float32)
    _lib.check(_lib.lib().fv_sdpa_dense_bf16_strided(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                                     int(out_bf16), bh, sq, sk, d, scale, rows[0], rows[1], rows[2],
                                                     _stream()))
    return out


def splitkv_choose(bh, sq, sk):
    """Key splits the library would use for this shape on the current device (1 = none)."""
    return int(_lib.lib().fv_sdpa_splitkv_choose(bh, sq, sk))


def sdpa_dense_bf16_splitkv(q, k, v, splits=None, scale=None, out_bf16=False):
    """`sdpa_dense_bf16_windows` with the keys of every query tile split over `splits` workgroups
    (default: the library's choice) and merged: for calls with few query tiles and many keys."""
    rows = [_plane_rows(t, n) for t, n in ((q, "q"), (k, "k"), (v, "v"))]
    bh, sq, d = q.shape
    if k.shape != v.shape or k.shape[0] != bh or k.shape[2] != d:
        raise ValueError(f"k/v {tuple(k.shape)}/{tuple(v.shape)} do not match q {tuple(q.shape)}")
    sk = k.shape[1]
    lib = _lib.lib()
    splits = splitkv_choose(bh, sq, sk) if splits is None else int(splits)
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.empty((bh, sq, d), device=q.device, dtype=torch.bfloat16 if out_bf16 else torch.float32)
    nbytes = int(lib.fv_sdpa_splitkv_workspace_bytes(bh, sq, d, max(splits, 1)))
    ws = torch.empty(max(nbytes, 256), device=q.device, dtype=torch.uint8)
    _lib.check(lib.fv_sdpa_dense_bf16_splitkv(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), int(out_bf16), bh,
                                              sq, sk, d, scale, rows[0], rows[1], rows[2], splits, ws.data_ptr(), nbytes,
                                              _stream()))
    return out


def sdpa_block_causal_bf16(q, k, v, block_tokens, window=0, sink=0, scale=None, out_bf16=False, out=None):
    bh, sq, sk, d = _bhsd(q, k, v)
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    want = torch.bfloat16 if out_bf16 else torch.float32
    if out is None:
        out = torch.empty((bh, sq, d), device=q.device, dtype=want)
    elif out.dtype != want or tuple(out.shape) != (bh, sq, d) or not out.is_contiguous() or out.device != q.device:
        raise ValueError(f"out must be a contiguous {want} tensor of shape {(bh, sq, d)} on {q.device}")
    _lib.check(_lib.lib().fv_sdpa_block_causal_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                                    int(out_bf16), bh, sq, sk, d, scale, block_tokens, window,
                                                    sink, _stream()))
    return out


def sdpa_vdn_window_bf16(q, k, v, video_start, frame_tokens, frames, chunk=0, radius=0, scale=None, out_bf16=False):
    bh, sq, sk, d = _bhsd(q, k, v)
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = torch.empty((bh, sq, d), device=q.device, dtype=torch.bfloat16 if out_bf16 else torch.float32)
    _lib.check(_lib.lib().fv_sdpa_vdn_window_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                                                  int(out_bf16), bh, sq, sk, d, scale, video_start, frame_tokens,
                                                  frames, chunk, radius, _stream()))
    return out


def cast_f32_bf16(x, mul=None):
    """bf16(x) (RNE), or bf16(x * mul) with the product in f32."""
    _need(x, torch.float32, "x")
    y = torch.empty(x.shape, device=x.device, dtype=torch.bfloat16)
    if mul is None:
        _lib.check(_lib.lib().fv_cast_f32_bf16(x.data_ptr(), y.data_ptr(), x.numel(), _stream()))
    else:
        _lib.check(_lib.lib().fv_cast_f32_bf16_scaled(x.data_ptr(), y.data_ptr(), x.numel(), float(mul), _stream()))
    return y


def cast_bf16_f32(x):
    _need(x, torch.bfloat16, "x")
    y = torch.empty(x.shape, device=x.device, dtype=torch.float32)
    _lib.check(_lib.lib().fv_cast_bf16_f32(x.data_ptr(), y.data_ptr(), x.numel(), _stream()))
    return y


def softmax_last(x, out_bf16=False, out=None):
    """Softmax over the trailing axis of an f32 tensor (rt/ops.rs:377-401 `softmax_last_device` /
    `softmax_last_bf16_device`); `out=x` runs the f32 form in place."""
    _need(x, torch.float32, "x")
    width = x.shape[-1] if x.dim() else 1
    rows = x.numel() // width if width else 0
    if out is None:
        out = torch.empty(x.shape, device=x.device, dtype=torch.bfloat16 if out_bf16 else torch.float32)
    else:
        _need(out, torch.bfloat16 if out_bf16 else torch.float32, "out")
        if out.shape != x.shape:
            raise ValueError("out: shape differs from x")
    _lib.check(_lib.lib().fv_softmax_last(x.data_ptr(), out.data_ptr(), int(out_bf16), rows, width, _stream()))
    return out
