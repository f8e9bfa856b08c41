"""Loader for libfv_sdpa_hip.so (the C ABI in include/fv_sdpa_hip.h).

There is no fallback: a missing library or symbol raises, and no function here
ever computes on the host.
"""
import ctypes as C
import os

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# FV_SDPA_HIP_LIB names another build of the same library (the host-sanitizer build of `make ubsan`)
LIB_PATH = os.environ.get("FV_SDPA_HIP_LIB") or os.path.join(_PKG, "libfv_sdpa_hip.so")
CSRC = os.path.join(_PKG, "csrc")

FV_OK = 0
FV_DECLINED = 1

_sz = C.c_size_t
_vp = C.c_void_p

# name -> (restype, argtypes); must list every symbol include/fv_sdpa_hip.h declares
SIGNATURES = {
    "fv_sdpa_last_error": (C.c_char_p, []),
    "fv_sdpa_arch": (C.c_char_p, []),
    "fv_sdpa_supported": (C.c_int, [_sz, _sz, _sz, _sz, _sz]),
    "fv_sdpa_is_log2_domain_scale": (C.c_int, [C.c_float]),
    "fv_sdpa_log2_domain_launches": (C.c_uint64, []),
    "fv_sdpa_exact_pass_reruns": (C.c_uint64, []),
    "fv_sdpa_dense_bf16": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, C.c_float, _vp]),
    "fv_sdpa_dense_bf16_strided": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, C.c_float, _sz, _sz, _sz,
                                             _vp]),
    "fv_sdpa_splitkv_choose": (_sz, [_sz, _sz, _sz]),
    "fv_sdpa_splitkv_workspace_bytes": (_sz, [_sz, _sz, _sz, _sz]),
    "fv_sdpa_dense_bf16_splitkv": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, C.c_float, _sz, _sz, _sz,
                                             _sz, _vp, _sz, _vp]),
    "fv_sdpa_splitkv_static_bytes": (_sz, []),
    "fv_sdpa_splitkv_static_splits": (_sz, [_sz, _sz, _sz, _sz, _sz]),
    "fv_sdpa_dense_bf16_splitkv_static": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, C.c_float, _sz, _sz,
                                                    _sz, _sz, _vp]),
    "fv_kv_plan": (C.c_int, [_sz, _sz, _sz, _sz, C.c_int, _sz, _sz, _sz, _sz, _vp]),
    "fv_kv_copy_tokens": (C.c_int, [_vp, _sz, _sz, _vp, _sz, _sz, _sz, _sz, _sz, C.c_int, _vp]),
    "fv_kv_shift_tokens_down": (C.c_int, [_vp, _sz, _sz, _sz, _sz, _sz, _sz, C.c_int, _vp]),
    "fv_kv_cache_new": (_vp, [_sz, _sz, _sz, _sz, C.c_int, C.c_int, _sz]),
    "fv_kv_cache_new_dynamic": (_vp, [_sz, _sz, _sz, _sz, C.c_int, C.c_int, _sz]),
    "fv_kv_cache_is_static": (C.c_int, [_vp]),
    "fv_kv_cache_rebase_sink": (C.c_int, [_vp, _sz, _vp, _vp, _vp, _vp, _vp]),
    "fv_kv_cache_set_pointers": (C.c_int, [_vp, _vp, _sz]),
    "fv_kv_cache_advance": (C.c_int, [_vp, _sz, _sz, _sz]),
    "fv_kv_cache_block_key": (C.c_int, [_vp, _sz, _sz, _sz, _vp]),
    "fv_rope_bhsd": (C.c_int, [_vp, C.c_int, _sz, _vp, _vp, C.c_int, _vp, C.c_int, _sz, _sz, _sz, _sz, _vp]),
    "fv_kv_cache_free": (None, [_vp]),
    "fv_kv_cache_reset": (None, [_vp]),
    "fv_kv_cache_set_sink_guard": (None, [_vp, C.c_int]),
    "fv_kv_cache_pointers": (C.c_int, [_vp, _sz, _vp]),
    "fv_kv_cache_bytes": (_sz, [_vp]),
    "fv_kv_cache_update": (C.c_int, [_vp, _sz, _vp, _vp, _sz, _vp, _vp, _vp]),
    "fv_sdpa_block_causal_bf16": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, C.c_float,
                                            _sz, _sz, _sz, _vp]),
    "fv_cast_f32_bf16": (C.c_int, [_vp, _vp, _sz, _vp]),
    "fv_cast_f32_bf16_scaled": (C.c_int, [_vp, _vp, _sz, C.c_float, _vp]),
    "fv_softmax_last": (C.c_int, [_vp, _vp, C.c_int, _sz, _sz, _vp]),
    "fv_cast_bf16_f32": (C.c_int, [_vp, _vp, _sz, _vp]),
    "fv_sdpa_composed_f32": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _vp, _sz, _sz, _sz, _sz, C.c_float, _vp]),
    "fv_sdpa_init": (C.c_int, []),
    "fv_rt_sdpa": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp]),
    "fv_rt_free": (C.c_int, [_vp, _vp]),
    "fv_rt_set_bf16_activations": (None, [C.c_int]),
    "fv_rt_bf16_activations": (C.c_int, []),
    "fv_rt_set_fold_scale": (None, [C.c_int]),
    "fv_rt_fold_scale": (C.c_int, []),
    "fv_rt_stats": (None, [_vp]),
    "fv_rt_log_level": (C.c_int, []),
    "fv_rt_parse_log_level": (C.c_int, [C.c_char_p]),
    "fv_vsa_default_sparsity": (C.c_double, []),
    "fv_rt_parse_backend": (C.c_int, [C.c_char_p]),
    "fv_rt_backend": (C.c_int, []),
    "fv_rt_set_backend": (None, [C.c_int]),
    "fv_rt_dense_route": (C.c_int, [_vp, _vp, _vp, C.c_int, C.c_int, _vp, _vp]),
    "fv_vsa_topk_for": (_sz, [C.c_double, _sz]),
    "fv_vsa_tile_plan": (C.c_int, [_sz, _sz, _sz, _vp, _vp, _vp, _vp]),
    "fv_vsa_tile_mean": (C.c_int, [_vp, C.c_int, _vp, _vp, _vp, _sz, _sz, _sz, _sz, C.c_int, _vp]),
    "fv_vsa_coarse": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, C.c_float, _vp]),
    "fv_vsa_topk": (C.c_int, [_vp, _vp, _sz, _sz, _sz, _vp]),
    "fv_vsa_tile_qkv": (C.c_int, [_vp, C.c_int, _vp, _vp, _sz, _sz, _sz, _sz, _vp]),
    "fv_vsa_fine": (C.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, C.c_float, _sz, _sz, _vp]),
    "fv_vsa_combine": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _vp]),
    "fv_vsa_combine_round16": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp, _vp, _sz, _sz, _sz, _sz, _sz, _sz, _vp]),
    "fv_vsa_workspace_bytes": (_sz, [_sz, _sz, _sz, _sz]),
    "fv_vsa_attention": (C.c_int, [_vp, _vp, _vp, C.c_int, _vp, C.c_int, _vp, _vp, _vp, _vp, _sz, _vp,
                                   _sz, _sz, _sz, _sz, _sz, C.c_float, _vp]),
    "fv_vsa_attention_tiled": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _vp, _vp, _vp, _vp, _sz, _vp,
                                         _sz, _sz, _sz, _sz, _sz, C.c_float, _vp]),
    "fv_block_causal_allows": (C.c_int, [_sz, _sz, _sz, _sz, _sz]),
    "fv_block_causal_dense_mask": (None, [_sz, _sz, _sz, _sz, _sz, _vp]),
    "fv_block_causal_for": (C.c_int, [_sz, C.c_longlong, _sz, _vp]),
    "fv_block_causal_tile_walk": (C.c_int, [_sz, _sz, _sz, _sz, _sz, _sz, _vp]),
    "fv_sp_shard_ranges": (None, [_sz, _sz, _vp]),
    "fv_sdpa_vdn_window_bf16": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, C.c_float,
                                          _sz, _sz, _sz, _sz, _sz, _vp]),
    "fv_vdn_window_allows": (C.c_int, [_sz, _sz, _sz, _sz, _sz, _sz, _sz]),
    "fv_vdn_window_dense_mask": (None, [_sz, _sz, _sz, _sz, _sz, _sz, _sz, _vp]),
    "fv_qk_norm_rope_bhsd": (C.c_int, [_vp, C.c_int, _vp, C.c_int, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, _sz,
                                       _sz, C.c_float, C.c_float, _vp]),
    "fv_split_heads_bhsd": (C.c_int, [_vp, _vp, C.c_int, _sz, _sz, _sz, _sz, _sz, _sz, _vp]),
    "fv_merge_heads": (C.c_int, [_vp, _vp, C.c_int, _sz, _sz, _sz, _sz, _vp]),
    "fv_qk_norm_rope_tiles": (C.c_int, [_vp, C.c_int, _vp, C.c_int, _vp, _vp, _vp, C.c_int, _sz, _sz, _sz, _sz, _sz,
                                        _sz, C.c_float, C.c_float, _vp, _sz, _vp]),
    "fv_split_heads_tiles": (C.c_int, [_vp, _vp, C.c_int, _sz, _sz, _sz, _sz, _sz, _sz, _vp, _sz, _vp]),
}

_lib = None


class FvError(RuntimeError):
    """A negative return of the C ABI (a HIP error)."""


class FvDeclined(RuntimeError):
    """FV_DECLINED: the kernel does not take this call; nothing ran."""


def build(force=True):
    """Compile the library in-tree with the committed Makefile (hipcc, gfx950)."""
    import subprocess

    cmd = ["make", "-C", CSRC, "-j8"] + (["-B"] if force else [])
    subprocess.check_call(cmd)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no CPU fallback)")
        l = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(l, name)  # AttributeError if the symbol is missing
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def last_error():
    return lib().fv_sdpa_last_error().decode()


def check(rc):
    if rc == FV_OK:
        return
    if rc == FV_DECLINED:
        raise FvDeclined(last_error())
    raise FvError(f"rc={rc}: {last_error()}")
