"""Python mirror of the causal-Wan KV cache (crates/fastvideo-cudarc/src/wan/causal.rs:38-57 `KvSpec`,
276-336 `KvMove` / `KvSpec::plan`, 341-723 `CausalKvCache::new_static`) over the library's C++ host
layer. The windows `update` returns are torch views of the layer's persistent buffers (no copy);
`sdpa(q, kw, vw, Plan.kv_window())` reads them in place.
"""
import collections
import ctypes as C

import torch

from . import _lib
from .sdpa import TensorError, _desc, _FvTensor

__all__ = ["KvSpec", "KvMove", "KvBlockKey", "KvRope", "CausalKvCache", "kv_copy_tokens", "kv_shift_tokens_down", "rope_bhsd"]


class KvMove:
    """wan/causal.rs:276-287."""

    def __init__(self, evicted, local_start, local_end, window_start):
        self.evicted, self.local_start, self.local_end, self.window_start = evicted, local_start, local_end, window_start

    def __repr__(self):
        return f"KvMove(evicted={self.evicted}, local=[{self.local_start}, {self.local_end}), window_start={self.window_start})"


class KvBlockKey(collections.namedtuple("KvBlockKey", "local_end appends evicted rebase take_raw")):
    """wan/causal.rs:365-378: what a block forward does to the cache; equal keys, equal device work."""


class KvRope:
    """wan/causal.rs:59-76."""
    ABSOLUTE, RELATIVISTIC, REBASED_SINK = 0, 1, 2


class KvSpec:
    """wan/causal.rs:38-57."""

    def __init__(self, frame_tokens, capacity, sink, max_attention, rolling, rope=KvRope.ABSOLUTE):
        self.frame_tokens, self.capacity, self.sink = int(frame_tokens), int(capacity), int(sink)
        self.max_attention, self.rolling = int(max_attention), bool(rolling)
        self.relativistic = rope == KvRope.RELATIVISTIC
        self.rebase_sink = rope == KvRope.REBASED_SINK and self.sink > 0

    @property
    def rope(self):
        return KvRope.RELATIVISTIC if self.relativistic else (KvRope.REBASED_SINK if self.rebase_sink else KvRope.ABSOLUTE)

    @staticmethod
    def rolling_window(frame_tokens, local_attn_frames, sink_frames, rope=KvRope.ABSOLUTE):
        """wan/causal.rs:110-131 `KvSpec::rolling`."""
        if local_attn_frames == 0 or sink_frames >= local_attn_frames:
            raise TensorError(f"causal kv: sink {sink_frames} frames must be below the window ({local_attn_frames} frames)")
        n = local_attn_frames * frame_tokens
        return KvSpec(frame_tokens, n, sink_frames * frame_tokens, n, True, rope)

    def sink_target(self, end_frame):
        """wan/causal.rs:136-138."""
        return max(end_frame - self.window_frames(), 0)

    @staticmethod
    def global_window(frame_tokens, frames, sink_frames=0):
        """wan/causal.rs:97-106: `local_attn_size == -1`, a `frames`-frame window that refuses longer clips."""
        n = frames * frame_tokens
        return KvSpec(frame_tokens, n, sink_frames * frame_tokens, n, False)

    def plan(self, global_end, local_end_prev, current_start, n):
        """wan/causal.rs:289-336."""
        out = (C.c_size_t * 4)()
        lib = _lib.lib()
        rc = lib.fv_kv_plan(self.capacity, self.sink, self.max_attention, self.frame_tokens, int(self.rolling),
                            global_end, local_end_prev, current_start, n, out)
        if rc != 0:
            raise TensorError(lib.fv_sdpa_last_error().decode())
        return KvMove(*(int(x) for x in out))

    def window_frames(self):
        return self.max_attention // max(self.frame_tokens, 1)


class _DevView:
    """Exposes a device row window to torch through the CUDA array interface."""

    def __init__(self, ptr, shape, plane_rows, bf16, keep):
        b, h, s, d = shape
        esz = 2 if bf16 else 4
        self._keep = keep
        self.__cuda_array_interface__ = {
            "shape": tuple(shape), "typestr": "<i2" if bf16 else "<f4", "data": (int(ptr), False), "version": 2,
            "strides": (h * plane_rows * d * esz, plane_rows * d * esz, d * esz, esz)}


class CausalKvCache:
    """wan/causal.rs:341-723. static (`new_static`, the default here): persistent [b, h, capacity, d]
    buffers per layer, written in place; static=False (`new`): every write builds the layer's K / V anew."""

    def __init__(self, spec, num_layers, static=True):
        self.spec = spec
        self._layers = num_layers
        make = _lib.lib().fv_kv_cache_new if static else _lib.lib().fv_kv_cache_new_dynamic
        self._h = make(spec.capacity, spec.sink, spec.max_attention, spec.frame_tokens,
                                             int(spec.rolling), spec.rope, num_layers)
        if not self._h:
            raise TensorError("causal kv: could not create the cache")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            try:
                torch.cuda.synchronize()
                _lib.lib().fv_kv_cache_free(h)
            except Exception:
                pass

    def update(self, layer, k, v, current_start):
        """Writes the block's k / v [b, h, n, d]; returns the (K, V) windows its queries read."""
        lib = _lib.lib()
        dk, dv = _desc(k, "k"), _desc(v, "v")
        kw, vw = _FvTensor(), _FvTensor()
        rc = lib.fv_kv_cache_update(self._h, layer, C.byref(dk), C.byref(dv), current_start, C.byref(kw), C.byref(vw),
                                    torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise TensorError(lib.fv_sdpa_last_error().decode())

        def view(t):
            shape = tuple(int(t.shape[i]) for i in range(t.rank))
            rows = int(t.plane_rows) or shape[2]
            x = torch.as_tensor(_DevView(t.data, shape, rows, bool(t.dtype), self), device=k.device)
            return x.view(torch.bfloat16) if t.dtype else x

        return view(kw), view(vw)

    def reset(self):
        _lib.lib().fv_kv_cache_reset(self._h)

    def is_static(self):
        return bool(_lib.lib().fv_kv_cache_is_static(self._h))

    def set_sink_guard(self, on):
        _lib.lib().fv_kv_cache_set_sink_guard(self._h, int(bool(on)))

    def pointers(self, layer=0):
        """(global_end, local_end) of a layer."""
        return self.pointers4(layer)[:2]

    def pointers4(self, layer=0):
        """(global_end, local_end, sink_at, raw_valid) of a layer (wan/causal.rs:353-360)."""
        out = (C.c_size_t * 4)()
        _lib.check(_lib.lib().fv_kv_cache_pointers(self._h, layer, out))
        return int(out[0]), int(out[1]), int(out[2]), bool(out[3])

    def set_pointers(self, per_layer):
        """wan/causal.rs:457-476: one (global_end, local_end, sink_at, raw_valid) per layer."""
        flat = (C.c_size_t * (4 * len(per_layer)))(*[int(x) for p in per_layer for x in p])
        lib = _lib.lib()
        if lib.fv_kv_cache_set_pointers(self._h, flat, len(per_layer)) != 0:
            raise TensorError(lib.fv_sdpa_last_error().decode())

    def advance(self, current_start, n, sink_target=0):
        """wan/causal.rs:503-536: the bookkeeping of one block forward without its device work."""
        lib = _lib.lib()
        if lib.fv_kv_cache_advance(self._h, current_start, n, sink_target) != 0:
            raise TensorError(lib.fv_sdpa_last_error().decode())

    def block_key(self, current_start, n, sink_target=0):
        """wan/causal.rs:477-502: (local_end, appends, evicted, rebase, take_raw) of a forward of n tokens at
        current_start; forwards with equal keys launch the same device work."""
        out = (C.c_size_t * 5)()
        lib = _lib.lib()
        if lib.fv_kv_cache_block_key(self._h, current_start, n, sink_target, out) != 0:
            raise TensorError(lib.fv_sdpa_last_error().decode())
        return KvBlockKey(int(out[0]), bool(out[1]), int(out[2]), bool(out[3]), bool(out[4]))

    def rebase_sink(self, target, orig, new):
        """wan/causal.rs:733-776: re-rope every layer's sink keys to start at frame `target`;
        orig / new = (cos, sin) f32 [sink_tokens, d] tables of the sink's own frames / of the target's."""
        for t in (*orig, *new):
            if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.float32 and t.dim() == 2
                    and t.shape[0] == self.spec.sink):
                raise ValueError("rebase_sink: tables must be contiguous f32 [sink_tokens, d] CUDA tensors")
        lib = _lib.lib()
        rc = lib.fv_kv_cache_rebase_sink(self._h, target, orig[0].data_ptr(), orig[1].data_ptr(), new[0].data_ptr(),
                                         new[1].data_ptr(), torch.cuda.current_stream().cuda_stream)
        if rc != 0:
            raise TensorError(lib.fv_sdpa_last_error().decode())

    def bytes(self):
        return int(_lib.lib().fv_kv_cache_bytes(self._h))


def _flat(t, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.is_contiguous() and t.dim() == 3
            and t.dtype in (torch.float32, torch.bfloat16)):
        raise ValueError(f"{name}: want a contiguous [bh, rows, d] CUDA tensor of f32 or bf16")
    return t


def kv_copy_tokens(dst, dst_off, src, src_off, length):
    """wan/causal.rs:199-232 on [bh, rows, d] tensors."""
    _flat(dst, "dst"), _flat(src, "src")
    if dst.dtype != src.dtype or dst.shape[0] != src.shape[0] or dst.shape[2] != src.shape[2]:
        raise ValueError("kv copy: dst and src differ in dtype, planes or head dim")
    _lib.check(_lib.lib().fv_kv_copy_tokens(dst.data_ptr(), dst.shape[1], dst_off, src.data_ptr(), src.shape[1], src_off,
                                            length, dst.shape[0], dst.shape[2], int(dst.dtype == torch.bfloat16),
                                            torch.cuda.current_stream().cuda_stream))


def kv_shift_tokens_down(t, frm, to, length):
    """wan/causal.rs:234-248 on a [bh, rows, d] tensor."""
    _flat(t, "t")
    _lib.check(_lib.lib().fv_kv_shift_tokens_down(t.data_ptr(), t.shape[1], frm, to, length, t.shape[0], t.shape[2],
                                                  int(t.dtype == torch.bfloat16),
                                                  torch.cuda.current_stream().cuda_stream))


def rope_bhsd(x, cos, sin, negate_sin=False, out_bf16=None):
    """wan/causal.rs:250-274 `rope_bhsd_f32` (out_bf16=False) / `rope_bhsd` (x's dtype): interleaved RoPE
    of x [b, h, s, d] (f32 or bf16, contiguous) with even-slot tables [s, d]."""
    if not (x.is_cuda and x.is_contiguous() and x.dim() == 4 and x.dtype in (torch.float32, torch.bfloat16)):
        raise ValueError("rope_bhsd: want a contiguous [b, h, s, d] CUDA tensor of f32 or bf16")
    b, h, s, d = x.shape
    for t in (cos, sin):
        if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.float32 and tuple(t.shape) == (s, d)):
            raise ValueError(f"rope_bhsd: tables must be contiguous f32 [{s}, {d}]")
    o16 = (x.dtype == torch.bfloat16) if out_bf16 is None else bool(out_bf16)
    out = torch.empty((b, h, s, d), device=x.device, dtype=torch.bfloat16 if o16 else torch.float32)
    _lib.check(_lib.lib().fv_rope_bhsd(x.data_ptr(), int(x.dtype == torch.bfloat16), s, cos.data_ptr(), sin.data_ptr(),
                                       int(bool(negate_sin)), out.data_ptr(), int(o16), s, b * h, s, d,
                                       torch.cuda.current_stream().cuda_stream))
    return out
