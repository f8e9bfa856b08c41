"""Python mirror of the causal-Wan KV cache (crates/fastvideo-cudarc/src/wan/causal.rs:38-57 `KvSpec`,
276-336 `KvMove` / `KvSpec::plan`, 341-723 `CausalKvCache::new_static`) over the library's C++ host
layer. The windows `update` returns are torch views of the layer's persistent buffers (no copy);
`sdpa(q, kw, vw, Plan.kv_window())` reads them in place.
"""
import ctypes as C

import torch

from . import _lib
from .sdpa import TensorError, _desc, _FvTensor

__all__ = ["KvSpec", "KvMove", "CausalKvCache", "kv_copy_tokens", "kv_shift_tokens_down"]


class KvMove:
    """wan/causal.rs:276-287."""

    def __init__(self, evicted, local_start, local_end, window_start):
        self.evicted, self.local_start, self.local_end, self.window_start = evicted, local_start, local_end, window_start

    def __repr__(self):
        return f"KvMove(evicted={self.evicted}, local=[{self.local_start}, {self.local_end}), window_start={self.window_start})"


class KvSpec:
    """wan/causal.rs:38-57 (absolute RoPE policy only)."""

    def __init__(self, frame_tokens, capacity, sink, max_attention, rolling):
        self.frame_tokens, self.capacity, self.sink = int(frame_tokens), int(capacity), int(sink)
        self.max_attention, self.rolling = int(max_attention), bool(rolling)

    @staticmethod
    def rolling_window(frame_tokens, local_attn_frames, sink_frames):
        """wan/causal.rs:110-131 `KvSpec::rolling` with KvRope::Absolute."""
        if local_attn_frames == 0 or sink_frames >= local_attn_frames:
            raise TensorError(f"causal kv: sink {sink_frames} frames must be below the window ({local_attn_frames} frames)")
        n = local_attn_frames * frame_tokens
        return KvSpec(frame_tokens, n, sink_frames * frame_tokens, n, True)

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
    """wan/causal.rs:341-723, static mode: persistent [b, h, capacity, d] buffers per layer."""

    def __init__(self, spec, num_layers):
        self.spec = spec
        self._h = _lib.lib().fv_kv_cache_new(spec.capacity, spec.sink, spec.max_attention, spec.frame_tokens,
                                             int(spec.rolling), num_layers)
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

    def set_sink_guard(self, on):
        _lib.lib().fv_kv_cache_set_sink_guard(self._h, int(bool(on)))

    def pointers(self, layer=0):
        out = (C.c_size_t * 2)()
        _lib.check(_lib.lib().fv_kv_cache_pointers(self._h, layer, out))
        return int(out[0]), int(out[1])

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
