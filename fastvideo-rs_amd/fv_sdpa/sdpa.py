"""Python mirror of `rt::sdpa::sdpa(q, k, v, &Plan)` (crates/fastvideo-cudarc/src/rt/sdpa.rs:29-164)
over the library's C++ host layer (`fv_rt_sdpa`). Same constructors, same error
messages; tensors are torch CUDA tensors (device memory only).
"""
import ctypes as C
from contextlib import contextmanager

import torch

from . import _lib

__all__ = ["Plan", "BlockCausal", "VdnWindow", "sdpa", "with_bf16_act", "bf16_activations", "with_fold_scale", "fold_scale", "rt_stats", "TensorError",
           "BACKENDS", "STEPS", "parse_backend", "backend", "with_backend", "shape_of", "dense_route"]


class TensorError(RuntimeError):
    """rt/tensor.rs:92-98 `TensorError::Message`. `rc` is the C ABI's return: -hipErrorInvalidValue (-1) for a
    refused argument, the negated hipError_t of a failed allocation (-2 out of memory) or launch otherwise."""

    def __init__(self, message, rc=None):
        super().__init__(message)
        self.rc = rc


class _FvTensor(C.Structure):
    _fields_ = [("data", C.c_void_p), ("dtype", C.c_int), ("rank", C.c_int), ("shape", C.c_size_t * 8),
                ("plane_rows", C.c_size_t)]


class _FvPlan(C.Structure):
    _fields_ = [("kind", C.c_int), ("has_scale", C.c_int), ("scale", C.c_float), ("mask", C.POINTER(_FvTensor)),
                ("fp8_first", C.c_int), ("block_tokens", C.c_size_t), ("window", C.c_size_t), ("sink", C.c_size_t),
                ("video_start", C.c_size_t), ("frame_tokens", C.c_size_t), ("frames", C.c_size_t),
                ("chunk", C.c_size_t), ("radius", C.c_size_t), ("kv_flash", C.c_int)]


class BlockCausal:
    """rt/attn.rs:441-467."""

    def __init__(self, block_tokens, window=0, sink=0):
        self.block_tokens, self.window, self.sink = block_tokens, window, sink

    def allows(self, q, k):
        return bool(_lib.lib().fv_block_causal_allows(self.block_tokens, self.window, self.sink, q, k))

    def dense_mask(self, sq, sk):
        from .vsa import block_causal_dense_mask

        return block_causal_dense_mask(self.block_tokens, self.window, self.sink, sq, sk)


class VdnWindow:
    """rt/attn.rs:469-524."""

    def __init__(self, video_start, frame_tokens, frames, chunk=0, radius=0):
        self.video_start, self.frame_tokens, self.frames, self.chunk, self.radius = (video_start, frame_tokens,
                                                                                     frames, chunk, radius)

    def _args(self):
        return self.video_start, self.frame_tokens, self.frames, self.chunk, self.radius

    def video_end(self):
        return self.video_start + self.frames * self.frame_tokens

    def allows(self, q, k):
        return bool(_lib.lib().fv_vdn_window_allows(*self._args(), q, k))

    def dense_mask(self, sq, sk):
        import numpy as np

        m = np.empty((sq, sk), dtype=np.float32)
        _lib.lib().fv_vdn_window_dense_mask(*self._args(), sq, sk, m.ctypes.data)
        return m


class Plan:
    """rt/sdpa.rs:29-137."""

    DENSE, COMPOSED, BLOCK_CAUSAL, VDN_WINDOW, KV_WINDOW = range(5)

    def __init__(self, kind, scale=None, mask=None, fp8=False, causal=None, kv_flash=None, window=None):
        self.kind, self.scale, self.mask, self.fp8, self.causal, self.kv_flash = kind, scale, mask, fp8, causal, kv_flash
        self.window = window

    @staticmethod
    def dense(scale=None):
        return Plan.masked(scale, None)

    @staticmethod
    def masked(scale=None, mask=None):
        return Plan(Plan.DENSE, scale, mask)

    def fp8_first(self):
        if self.kind == Plan.DENSE and self.mask is None:
            return Plan(Plan.DENSE, self.scale, None, fp8=True)
        return self

    @staticmethod
    def composed(scale=None, mask=None):
        return Plan(Plan.COMPOSED, scale, mask)

    @staticmethod
    def block_causal(scale, mask):
        return Plan(Plan.BLOCK_CAUSAL, scale, causal=mask)

    @staticmethod
    def vdn_window(scale, mask):
        return Plan(Plan.VDN_WINDOW, scale, window=mask)

    @staticmethod
    def kv_window():
        return Plan(Plan.KV_WINDOW)

    @staticmethod
    def kv_window_with(flash):
        return Plan(Plan.KV_WINDOW, kv_flash=bool(flash))


def _window_rows(t):
    """plane_rows of a BHSD tensor that is a row window (`base[:, :, a:b]`) of a contiguous
    [b, h, rows, d] tensor, else None."""
    if t.dim() != 4:
        return None
    b, h, s, d = t.shape
    sb, sh, ss, sd = t.stride()
    if sd != 1 or ss != d or sh % d or sh < s * d or (b > 1 and sb != h * sh):
        return None
    return sh // d


def _desc(t, name):
    rows = 0
    if isinstance(t, torch.Tensor) and t.is_cuda and not t.is_contiguous():
        rows = _window_rows(t) or 0
        if not rows:
            raise ValueError(f"{name}: want a contiguous CUDA tensor or a row window of a BHSD one")
    elif not (isinstance(t, torch.Tensor) and t.is_cuda):
        raise ValueError(f"{name}: want a contiguous CUDA tensor")
    if t.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError(f"{name}: want f32 or bf16")
    if t.dim() > 8:
        raise ValueError(f"{name}: rank > 8")
    d = _FvTensor()
    d.data, d.dtype, d.rank = t.data_ptr(), int(t.dtype == torch.bfloat16), t.dim()
    d.plane_rows = rows
    for i, s in enumerate(t.shape):
        d.shape[i] = s
    return d


class _Owned:
    """Frees the library-allocated result when the wrapping tensor dies."""

    def __init__(self, ptr, stream):
        self.ptr, self.stream = ptr, stream

    def __del__(self):
        try:
            _lib.lib().fv_rt_free(self.ptr, self.stream)
        except Exception:
            pass


def sdpa(q, k, v, plan):
    """rt/sdpa.rs:141-164. Returns a new [b, h, sq, d] tensor (bf16 under bf16 activations, else f32)."""
    lib = _lib.lib()
    dq, dk, dv = _desc(q, "q"), _desc(k, "k"), _desc(v, "v")
    p = _FvPlan()
    p.kind = plan.kind
    p.has_scale, p.scale = (1, float(plan.scale)) if plan.scale is not None else (0, 0.0)
    dm = None
    if plan.mask is not None:
        dm = _desc(plan.mask, "mask")
        p.mask = C.pointer(dm)
    p.fp8_first = int(plan.fp8)
    if plan.causal is not None:
        p.block_tokens, p.window, p.sink = plan.causal.block_tokens, plan.causal.window, plan.causal.sink
    if plan.window is not None:
        p.video_start, p.frame_tokens, p.frames, p.chunk, p.radius = plan.window._args()
    p.kv_flash = -1 if plan.kv_flash is None else int(plan.kv_flash)
    out = _FvTensor()
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.fv_rt_sdpa(C.byref(dq), C.byref(dk), C.byref(dv), C.byref(p), C.byref(out), stream)
    if rc != 0:
        raise TensorError(lib.fv_sdpa_last_error().decode(), rc)
    shape = tuple(out.shape[i] for i in range(out.rank))
    dtype = torch.bfloat16 if out.dtype else torch.float32
    n = 1
    for s in shape:
        n *= s
    # copy into torch-owned memory, then hand the library's buffer back (stream-ordered)
    owner = _Owned(out.data, stream)
    nbytes = n * (2 if out.dtype else 4)
    res = torch.empty(shape, device=q.device, dtype=dtype)
    if nbytes:
        from torch.cuda import current_stream  # noqa: F401

        _hip_copy(res.data_ptr(), out.data, nbytes, stream)
    del owner
    return res


_hiprt = None


def _hip_copy(dst, src, nbytes, stream):
    global _hiprt
    if _hiprt is None:
        _hiprt = C.CDLL("libamdhip64.so")
        _hiprt.hipMemcpyAsync.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        _hiprt.hipMemcpyAsync.restype = C.c_int
    rc = _hiprt.hipMemcpyAsync(dst, src, nbytes, 3, stream)   # hipMemcpyDeviceToDevice
    if rc != 0:
        raise TensorError(f"hipMemcpyAsync failed: {rc}")


def bf16_activations():
    return bool(_lib.lib().fv_rt_bf16_activations())


@contextmanager
def with_bf16_act(on):
    """rt/tensor.rs `with_bf16_act(on, f)`."""
    lib = _lib.lib()
    lib.fv_rt_set_bf16_activations(int(bool(on)))
    try:
        yield
    finally:
        lib.fv_rt_set_bf16_activations(-1)


def fold_scale():
    return bool(_lib.lib().fv_rt_fold_scale())


@contextmanager
def with_fold_scale(on):
    """Per-thread override of FASTVIDEO_SDPA_FOLD_SCALE: whether `sdpa` folds scale * log2(e) into the one
    rounding of an f32 q (and runs the kernel at scale = ln 2)."""
    lib = _lib.lib()
    lib.fv_rt_set_fold_scale(int(bool(on)))
    try:
        yield
    finally:
        lib.fv_rt_set_fold_scale(-1)


def rt_stats():
    out = (C.c_uint64 * 5)()
    _lib.lib().fv_rt_stats(out)
    return dict(zip(("fused", "causal", "composed", "casts", "masks"), (int(x) for x in out)))


# rt/sdpa_rule.rs:178-207 `Backend` and the collapsed `Step` (the NVIDIA alternates are gone)
BACKENDS = ("dense", "cublas", "flash", "host", "sparse")
STEPS = ("retired", "fused", "composed")


def parse_backend(v):
    """rt/sdpa_rule.rs:199-207: a FASTVIDEO_SDPA value -> backend name (unknown = "dense")."""
    return BACKENDS[_lib.lib().fv_rt_parse_backend(str(v).encode())]


def backend():
    return BACKENDS[_lib.lib().fv_rt_backend()]


@contextmanager
def with_backend(name):
    """Per-thread override of FASTVIDEO_SDPA for the calls inside the block."""
    lib = _lib.lib()
    lib.fv_rt_set_backend(BACKENDS.index(name))
    try:
        yield
    finally:
        lib.fv_rt_set_backend(-1)


def _shape4(x):
    x = tuple(int(i) for i in x)
    if len(x) != 4:
        raise TensorError("sdpa expects BHSD")
    return (C.c_size_t * 4)(*x)


def dense_route(q_shape, k_shape, v_shape, masked=False, backend_name="dense"):
    """rt/sdpa_rule.rs:409-437: the kernels a dense call tries, in order."""
    steps = (C.c_int * 4)()
    n = _lib.lib().fv_rt_dense_route(_shape4(q_shape), _shape4(k_shape), _shape4(v_shape), int(bool(masked)),
                                     BACKENDS.index(backend_name), steps, None)
    if n < 0:
        raise TensorError("dense_route: bad arguments")
    return [STEPS[steps[i]] for i in range(n)]


def shape_of(q_shape, k_shape, v_shape):
    """rt/sdpa_rule.rs:373-390 `Shape::of`: (sq, sk, dims) with dims = (b, h, sq, sk, d) or None."""
    steps, dims = (C.c_int * 4)(), (C.c_size_t * 5)()
    _lib.lib().fv_rt_dense_route(_shape4(q_shape), _shape4(k_shape), _shape4(v_shape), 0, 0, steps, dims)
    d = tuple(int(x) for x in dims)
    return int(q_shape[2]), int(k_shape[2]), (d if any(d) else None)
