"""CPU-side checks of the shipped library: it loads, exports every symbol the
header declares, and its host-side geometry (tile plan, top-k rule, block-causal
predicate, shard ranges) equals the oracle's restatement of the reference and
the reference's own known answers. No GPU calls.
"""
import ctypes
import os
import re

import numpy as np
import pytest

from util import ROOT

import fv_sdpa
from fv_sdpa import _lib


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fv_sdpa_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(fv_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 20
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert fv_sdpa.lib().fv_sdpa_arch() == b"gfx950"
    assert isinstance(fv_sdpa.lib().fv_sdpa_last_error(), bytes)   # "" until a call of this thread fails


def test_supported_table():
    # rt/attn.rs:932-960
    ok = fv_sdpa.sdpa_supported
    assert ok(1, 40, 38001, 38001, 128) and ok(2, 32, 4097, 1024, 128) and ok(1, 1, 1, 1, 128)
    assert ok(1, 32, 125, 1, 64)
    for d in (32, 80, 96, 256, 384):
        assert not ok(1, 8, 1024, 1024, d)
    assert not ok(1, 8, 0, 1024, 128) and not ok(1, 8, 1024, 0, 128)
    assert not ok(0, 8, 1024, 1024, 128) and not ok(2, 40000, 64, 64, 128)


def test_log2_domain_scale_predicate():
    # scale = ln 2 as f32 times the library's f32 log2(e) rounds to exactly one; its neighbours and the
    # usual 1/sqrt(d) do not
    is_log2 = fv_sdpa.lib().fv_sdpa_is_log2_domain_scale
    ln2 = np.float32(np.log(2.0))
    assert is_log2(float(ln2)) == 1
    assert is_log2(float(np.nextafter(ln2, np.float32(0)))) == 0 and is_log2(float(np.nextafter(ln2, np.float32(1)))) == 0
    for d in (64, 128):
        assert is_log2(1.0 / np.sqrt(d)) == 0
    header = open(os.path.join(ROOT, "include", "fv_sdpa_hip.h")).read()
    m = re.search(r"#define FV_SDPA_SCALE_LOG2_DOMAIN ([0-9.]+)f", header)
    assert m and np.float32(float(m.group(1))) == ln2
    rust = open(os.path.join(ROOT, "rust", "fastvideo-hip-sdpa", "src", "ffi.rs")).read()
    m = re.search(r"FV_SDPA_SCALE_LOG2_DOMAIN: f32 = ([0-9._]+);", rust)
    assert m and np.float32(float(m.group(1).replace("_", ""))) == ln2


@pytest.mark.parametrize("grid", [(4, 4, 4), (33, 28, 52), (3, 5, 7), (1, 1, 1), (1, 1, 5), (21, 30, 52), (32, 32, 32)])
def test_tile_plan_equals_oracle(oracle, grid):
    got, want = fv_sdpa.TilePlan(grid), oracle.TilePlan(grid)
    assert got.tiles == want.tiles and got.seq == want.seq and got.padded == want.padded
    assert np.array_equal(got.slot_src, want.slot_src)
    assert np.array_equal(got.token_slot, want.token_slot)
    assert np.array_equal(got.block_sizes.astype(np.uint32), want.block_sizes)


def test_tile_plan_known_answers():
    p = fv_sdpa.TilePlan((1, 1, 5))
    assert list(p.block_sizes) == [4, 1] and list(p.slot_src[:4]) == [0, 1, 2, 3] and p.slot_src[64] == 4
    assert (p.slot_src[4:64] == -1).all()
    assert fv_sdpa.TilePlan((21, 30, 52)).num_tiles == 624
    with pytest.raises(ValueError):
        fv_sdpa.TilePlan((4, 0, 4))


def test_topk_rule(oracle):
    for sp, n, want in [(0.8, 819, 164), (0.0, 819, 819), (1.0, 819, 1), (0.9, 10, 1), (0.8, 624, 125), (0.875, 512, 64)]:
        assert fv_sdpa.topk_for(sp, n) == want == oracle.topk_for(sp, n)


def test_block_causal_host_helpers(oracle):
    for bt, win, sink in [(5, 2, 1), (1, 0, 0), (7, 0, 2), (4, 1, 0), (0, 0, 0), (60, 3, 1)]:
        assert np.array_equal(fv_sdpa.block_causal_dense_mask(bt, win, sink, 50, 61),
                              oracle.block_causal_dense_mask(bt, win, sink, 50, 61))
    for fpb, las, ft in [(3, -1, 1560), (3, 4, 6), (3, 6, 10), (1, 2, 7), (1, -1, 3), (3, 0, 5)]:
        assert fv_sdpa.block_causal_for(fpb, las, ft) == oracle.block_causal_for(fpb, las, ft)
    assert fv_sdpa.block_causal_for(3, 4, 6) is None
    assert fv_sdpa.block_causal_allows(5, 2, 1, 23, 0) and not fv_sdpa.block_causal_allows(5, 2, 1, 23, 5)


def test_shard_ranges(oracle):
    assert fv_sdpa.shard_ranges(10, 2) == [(0, 5), (5, 5)]
    assert fv_sdpa.shard_ranges(11, 2) == [(0, 6), (6, 5)]
    assert fv_sdpa.shard_ranges(32760, 8) == oracle.shard_ranges(32760, 8)


def test_backend_parses_like_the_reference():
    # rt/sdpa_rule.rs:593-604
    for v in ("dense", "cublas", "flash", "host", "sparse"):
        assert fv_sdpa.parse_backend(v) == v
    for v in ("", "fused", " cublas", "dense "):
        assert fv_sdpa.parse_backend(v) == "dense", v
    assert fv_sdpa.backend() == fv_sdpa.parse_backend(os.environ.get("FASTVIDEO_SDPA", "dense").lower())
    with fv_sdpa.with_backend("cublas"):
        assert fv_sdpa.backend() == "cublas"
    assert fv_sdpa.backend() == fv_sdpa.parse_backend(os.environ.get("FASTVIDEO_SDPA", "dense").lower())


def test_shapes_agree_only_when_k_and_v_match_q():
    # rt/sdpa_rule.rs:624-651
    assert fv_sdpa.shape_of((1, 2, 5, 64), (1, 2, 7, 64), (1, 2, 7, 64)) == (5, 7, (1, 2, 5, 7, 64))
    assert fv_sdpa.shape_of((1, 2, 5, 64), (1, 2, 7, 64), (1, 2, 6, 64))[2] is None
    assert fv_sdpa.shape_of((1, 2, 5, 64), (1, 3, 7, 64), (1, 3, 7, 64))[2] is None
    assert fv_sdpa.shape_of((1, 2, 5, 64), (1, 2, 7, 32), (1, 2, 7, 32))[2] is None


def test_dense_route_collapsed():
    # rt/sdpa_rule.rs:409-437 without the cuDNN / cuBLAS / Sage / f32-flash steps
    s = ((1, 12, 320, 128),) * 3
    assert fv_sdpa.dense_route(*s) == ["fused", "composed"]
    assert fv_sdpa.dense_route(*s, masked=True) == ["composed"]
    for b in ("cublas", "flash"):
        assert fv_sdpa.dense_route(*s, backend_name=b) == ["composed"]
    for b in ("host", "sparse"):
        assert fv_sdpa.dense_route(*s, backend_name=b) == ["retired"]
        assert fv_sdpa.dense_route(*s, masked=True, backend_name=b) == ["composed"]   # masked calls never look


@pytest.mark.parametrize("bt,win,sink,sq,sk", [
    (256, 1, 0, 512, 256),      # the second query tile sees no key at all
    (100, 2, 0, 1000, 300), (100, 2, 1, 1000, 300), (64, 0, 0, 700, 130), (1560, 0, 0, 4680, 4680),
    (1560, 2, 1, 6240, 4680), (7, 3, 2, 900, 200), (300, 1, 0, 2000, 500), (128, 1, 3, 1024, 4096),
    (50, 4, 0, 257, 1), (1000, 1, 0, 513, 64)])
def test_block_causal_tile_walk_covers_every_visible_key(bt, win, sink, sq, sk):
    """The key-tile ranges the fused block-causal kernel walks (the function the kernel itself runs):
    ascending, disjoint, inside the key tiles, and covering every key that rt/attn.rs:449-453 lets any
    query of the tile see; a tile whose walk is empty has no visible key at all."""
    lib = fv_sdpa.lib()
    nkt = (sk + 63) // 64
    q = np.arange(sq)[:, None]
    k = np.arange(sk)[None, :]
    tq, tk = q // bt, k // bt
    vis = (tk < sink) | ((tk <= tq) & ((win == 0) | (tq - tk < win)))
    empty_tiles = 0
    for q0 in range(0, sq, 256):
        out = (ctypes.c_int * 4)()
        assert lib.fv_block_causal_tile_walk(bt, win, sink, sq, sk, q0, out) == 0
        n0, a1, n1, total = list(out)
        assert 0 <= n0 <= a1 and n1 >= 0 and a1 + n1 <= nkt and total == n0 + n1
        walked = np.zeros(nkt, bool)
        walked[:n0] = True
        walked[a1:a1 + n1] = True
        need = vis[q0:q0 + 256].any(axis=0)                       # keys some query of the tile sees
        need_tiles = np.zeros(nkt, bool)
        need_tiles[np.nonzero(need)[0] // 64] = True
        assert not (need_tiles & ~walked).any(), (q0, list(out))
        if total == 0:
            assert not need.any()
            empty_tiles += 1
    if (bt, win, sink, sq, sk) == (256, 1, 0, 512, 256):
        assert empty_tiles == 1
    # parameters the kernel declines
    out = (ctypes.c_int * 4)()
    assert lib.fv_block_causal_tile_walk(0, 0, 0, 256, 256, 0, out) == _lib.FV_DECLINED
    assert lib.fv_block_causal_tile_walk(64, 0, 0, 256, 256, 100, out) == _lib.FV_DECLINED


def _fake_tensor(shape, bf16, addr=0x1000):
    """A descriptor whose pointer is never dereferenced on the host: for calls that must fail before a launch."""
    from fv_sdpa.sdpa import _FvTensor

    t = _FvTensor()
    t.data, t.dtype, t.rank, t.plane_rows = addr, int(bf16), len(shape), 0
    for i, s in enumerate(shape):
        t.shape[i] = s
    return t


def _rt_call(q, k, v, kind=0, mask=None):
    from fv_sdpa.sdpa import _FvPlan, _FvTensor

    lib = fv_sdpa.lib()
    p = _FvPlan()
    p.kind, p.kv_flash = kind, -1
    if mask is not None:
        p.mask = ctypes.pointer(mask)
    out = _FvTensor()
    rc = lib.fv_rt_sdpa(ctypes.byref(q), ctypes.byref(k), ctypes.byref(v), ctypes.byref(p), ctypes.byref(out), None)
    return rc, lib.fv_sdpa_last_error().decode()


def test_rt_sdpa_refuses_before_any_device_work():
    """Argument errors of the one entry are host decisions: they come back as -hipErrorInvalidValue with the
    reference's message and touch no device (rt/sdpa.rs:141-164, rt/tensor.rs:1655-1667)."""
    q = _fake_tensor((1, 2, 8, 128), True)
    rc, msg = _rt_call(_fake_tensor((2, 8, 128), True), q, q)
    assert rc == -1 and msg == "sdpa expects BHSD"
    # a masked composed call with no keys: refused, and the mask's batch count is never divided by sq * sk = 0
    k0 = _fake_tensor((1, 2, 0, 128), False)
    rc, msg = _rt_call(_fake_tensor((1, 2, 8, 128), False), k0, k0, kind=1, mask=_fake_tensor((8, 0), False))
    assert rc == -1 and msg == "sdpa: no keys"
    rc, msg = _rt_call(q, q, q, kind=99)
    assert rc == -1 and "unknown plan kind" in msg


def test_rt_sdpa_reports_an_allocation_failure_with_its_own_code():
    """Without a device the first allocation fails: the entry returns that hipError_t (not the code of a
    refused argument) and the message says which step failed. Skipped where a GPU is present (the
    allocation would succeed and the fake operands must never reach a kernel)."""
    import torch

    if torch.cuda.device_count() > 0:
        pytest.skip("needs a host without a GPU")
    q = _fake_tensor((1, 2, 8, 128), True)
    rc, msg = _rt_call(q, q, q)
    assert rc < -1 and msg.startswith("sdpa: device allocation failed: ")
    # no query rows + a mask: an empty result is allocated (no division by sq * sk = 0 on the way)
    q0 = _fake_tensor((1, 2, 0, 128), False)
    kv = _fake_tensor((1, 2, 8, 128), False)
    rc, msg = _rt_call(q0, kv, kv, kind=1, mask=_fake_tensor((0, 8), False))
    assert rc < -1 and msg.startswith("sdpa: device allocation failed: ")


def test_log_level_parses_like_the_reference():
    # rt/log.rs:17-37
    parse = fv_sdpa.lib().fv_rt_parse_log_level
    for v, want in [(None, 1), (b"", 1), (b"1", 1), (b"info", 1), (b"anything", 1), (b"0", 0), (b"off", 0), (b" OFF ", 0),
                    (b"false", 0), (b"quiet", 0), (b"error", 0), (b"2", 2), (b"debug", 2), (b"Trace", 2), (b"verbose\n", 2)]:
        assert parse(v) == want, v


def _in_subprocess(code, env):
    import subprocess
    import sys

    e = dict(os.environ)
    e.update(env)
    r = subprocess.run([sys.executable, "-c", "import sys; sys.path[:0] = %r; " % [ROOT, os.path.join(ROOT, "fastvideo-rs_amd")]
                        + code], capture_output=True, text=True, env=e, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    return r.stdout.strip()


def test_environment_defaults_are_read_by_the_library():
    code = "import fv_sdpa; l = fv_sdpa.lib(); print(l.fv_rt_log_level(), l.fv_vsa_default_sparsity())"
    assert _in_subprocess(code, {"FASTVIDEO_LOG": "debug", "FASTVIDEO_VSA_SPARSITY": " 0.875 "}) == "2 0.875"
    assert _in_subprocess(code, {"FASTVIDEO_LOG": "0", "FASTVIDEO_VSA_SPARSITY": "sparse"}) == "0 0.8"
    # the reference trims, then parses with Rust's f64 grammar (settings/parse.rs:43-45): a leading '+' and
    # exponents are numbers, hex floats and "nan(...)" (which strtod alone would take) are not
    for text, want in ((" 0.5", "0.5"), ("+0.25", "0.25"), ("5e-1\n", "0.5"), ("0x1p-1", "0.8"), ("nan(1)", "0.8"),
                       ("0.5 0.6", "0.8"), ("", "0.8")):
        assert _in_subprocess(code, {"FASTVIDEO_LOG": "0", "FASTVIDEO_VSA_SPARSITY": text}) == "0 " + want, text
    env = {k: v for k, v in os.environ.items() if k not in ("FASTVIDEO_LOG", "FASTVIDEO_VSA_SPARSITY")}
    import subprocess
    import sys

    r = subprocess.run([sys.executable, "-c", "import sys; sys.path[:0] = %r; " % [ROOT, os.path.join(ROOT, "fastvideo-rs_amd")]
                        + code], capture_output=True, text=True, env=env, timeout=120)
    assert r.stdout.strip() == "1 0.8", r.stderr[-500:]


def test_static_splitkv_never_refuses_its_own_choice():
    """fv_sdpa_dense_bf16_splitkv_static with splits == 0 runs the library's choice stepped down to what its
    32 MiB buffer holds (host arithmetic: fv_sdpa_splitkv_static_splits); only an explicit count that cannot
    fit is refused; absurd counts are settled, not divided by."""
    lib = fv_sdpa.lib()
    cap = lib.fv_sdpa_splitkv_static_bytes()
    assert cap == 32 << 20
    stepped = 0
    for d in (128, 64):
        for bh in (1, 2, 3, 4, 6, 8, 12, 16, 24, 40):
            for sq in (1, 64, 256, 257, 512, 1024, 1560, 2048, 3000, 4096, 4680, 8192):
                for sk in (64, 512, 1560, 4096, 4680, 16384, 32760, 75600):
                    auto = lib.fv_sdpa_splitkv_static_splits(bh, sq, sk, d, 0)
                    chosen = lib.fv_sdpa_splitkv_choose(bh, sq, sk)
                    assert 1 <= auto <= chosen, (bh, sq, sk, d, auto, chosen)
                    assert lib.fv_sdpa_splitkv_workspace_bytes(bh, sq, d, auto) <= cap
                    if auto < chosen:
                        stepped += 1
                        nxt = auto + 1    # the next count that is a real split count does not fit
                        while nxt <= chosen and lib.fv_sdpa_splitkv_static_splits(bh, sq, sk, d, nxt) == auto:
                            nxt += 1
                        assert nxt > chosen or lib.fv_sdpa_splitkv_static_splits(bh, sq, sk, d, nxt) == 0
    assert stepped > 0
    # the three shapes that used to be refused: 16 splits chosen, partials 262 144 bytes over the buffer
    for bh, sq in ((1, 4096), (2, 2048), (4, 1024)):
        assert lib.fv_sdpa_splitkv_choose(bh, sq, 32760) == 16
        assert lib.fv_sdpa_splitkv_workspace_bytes(bh, sq, 128, 16) == 33816576 > cap
        assert lib.fv_sdpa_splitkv_static_splits(bh, sq, 32760, 128, 0) == 15
        assert lib.fv_sdpa_splitkv_static_splits(bh, sq, 32760, 128, 16) == 0     # explicit and too large: refused
    # explicit counts: settled so that no split is empty, never more than the key tiles
    assert lib.fv_sdpa_splitkv_static_splits(12, 256, 32760, 128, 7) == 7
    assert lib.fv_sdpa_splitkv_static_splits(12, 256, 640, 128, 7) == 5            # 10 tiles / ceil(10 / 7) = 2 per split
    assert lib.fv_sdpa_splitkv_static_splits(1, 256, 640, 128, 2 ** 64 - 1) == 10  # no wrap, no division by zero
    assert lib.fv_sdpa_splitkv_static_splits(1, 256, 64, 128, 5) == 1
