"""Repeat-run determinism at size: every kernel whose work order, reduction order or selection could differ
between runs is called three times on the same inputs in one process, and every repeat must equal the first
bit for bit (the reference's `determinism` group, crates/fastvideo-gpucheck/src/kernels/determinism.rs:25-52:
its shapes 8 x 24832^2 and 8 x 9690 x 1024, REPEATS = 3, plus this library's own full-size calls).
Nothing here uses atomics or a data-dependent work order, so the bar is equality, not a tolerance."""
import numpy as np
import pytest

from util import announce

pytestmark = pytest.mark.gpu

REPEATS = 3
D = 128


@pytest.fixture(scope="module")
def fv():
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


def _randn_bf16(seed, *shapes):
    import torch

    g = torch.Generator(device="cuda").manual_seed(seed)
    return [torch.randn(s, generator=g, device="cuda").to(torch.bfloat16) for s in shapes]


def _same(runs):
    import torch

    return all(r.dtype == runs[0].dtype and torch.equal(r, runs[0]) for r in runs[1:])


def _repeat(call):
    """REPEATS results of `call`, with other work (a different launch of the same kernel) between the repeats so
    that the repeats do not run back to back on an undisturbed machine."""
    import torch

    runs = []
    for i in range(REPEATS):
        runs.append(call())
        torch.cuda.synchronize()
        if i + 1 < REPEATS:
            (torch.ones((1 << 20,), device="cuda") * (i + 2)).sum().item()
    return runs


@pytest.mark.parametrize("name,bh,sq,sk", [
    ("reference_self_24k6", 8, 24832, 24832),      # determinism.rs:29
    ("reference_cross", 8, 9690, 1024),            # determinism.rs:30
    ("wan13b_self", 12, 32760, 32760),
    ("wan13b_cross", 12, 32760, 512),
])
def test_dense_repeats_are_bit_identical(fv, name, bh, sq, sk):
    announce(f"determinism dense {name} bh={bh} sq={sq} sk={sk}")
    q, k, v = _randn_bf16(600, (bh, sq, D), (bh, sk, D), (bh, sk, D))
    for out_bf16 in (True, False):
        runs = _repeat(lambda: fv.sdpa_dense_bf16(q, k, v, out_bf16=out_bf16))
        assert _same(runs), (name, out_bf16)
    # the form for a scale folded into Q runs another kernel instantiation
    ln2 = float(np.float32(np.log(2.0)))
    assert _same(_repeat(lambda: fv.sdpa_dense_bf16(q, k, v, scale=ln2, out_bf16=True))), name


@pytest.mark.parametrize("bt,win,sink", [(1560, 0, 0), (4680, 0, 0), (1560, 4, 1)])
def test_block_causal_repeats_are_bit_identical(fv, bt, win, sink):
    bh, s = 12, 32760
    announce(f"determinism block-causal bt={bt} win={win} sink={sink}")
    q, k, v = _randn_bf16(601, (bh, s, D), (bh, s, D), (bh, s, D))
    assert _same(_repeat(lambda: fv.sdpa_block_causal_bf16(q, k, v, bt, win, sink)))


@pytest.mark.parametrize("grid,sparsity", [((32, 32, 32), 0.875), ((21, 30, 52), 0.8)])
def test_vsa_repeats_are_bit_identical(fv, grid, sparsity):
    """The whole VSA op: the output AND the selected block lists (top-k with its tie rule) repeat exactly."""
    import torch

    bh = 12
    announce(f"determinism vsa grid={grid}")
    ctx = fv.VsaCtx(grid, sparsity)
    q, k, v, g = _randn_bf16(602, *[(bh, ctx.seq, D)] * 4)
    scale = float(1.0 / np.sqrt(D))
    outs, sels = [], []
    for i in range(REPEATS):
        out, sel = fv.vsa_attention_device(q, k, v, g, ctx, scale, return_selected=True)
        torch.cuda.synchronize()
        outs.append(out.clone())
        sels.append(sel.clone())
        (torch.ones((1 << 20,), device="cuda") * (i + 2)).sum().item()
    assert _same(sels)
    assert _same(outs)
    # heavily tied coarse scores (identical key tiles): the selection still repeats, and is the lowest indices
    k2 = k.clone()
    k2[:] = k[:, :1]
    sels = []
    for _ in range(REPEATS):
        _, sel = fv.vsa_attention_device(q, k2, v, g, ctx, scale, return_selected=True)
        torch.cuda.synchronize()
        sels.append(sel.clone())
    assert _same(sels)
    if grid == (32, 32, 32):       # full cubes: every key tile has the same mean, so every score of a row ties
        want = torch.arange(ctx.topk, device="cuda", dtype=sels[0].dtype).expand_as(sels[0])
        assert torch.equal(sels[0].sort(-1).values, want)


@pytest.mark.parametrize("bh,sq,sk,splits", [(12, 1560, 32760, 3), (12, 256, 32760, 0), (1, 4096, 32760, 0)])
def test_splitkv_repeats_are_bit_identical(fv, bh, sq, sk, splits):
    """Split-KV: the partials are merged by a second kernel in a fixed order (no arrival order anywhere)."""
    announce(f"determinism split-KV bh={bh} sq={sq} sk={sk} splits={splits}")
    q, k, v = _randn_bf16(603, (bh, sq, D), (bh, sk, D), (bh, sk, D))
    runs = _repeat(lambda: fv.sdpa_dense_bf16_splitkv(q, k, v, splits=splits or None))
    assert _same(runs)


def test_kv_window_and_rt_entry_repeats_are_bit_identical(fv):
    """The one entry (`fv_rt_sdpa`, which picks the route and the split count itself) on a KV-window shape."""
    import torch

    bh, sq, sk = 12, 4680, 32760
    announce("determinism rt sdpa kv-window")
    q, k, v = _randn_bf16(604, (1, bh, sq, D), (1, bh, sk, D), (1, bh, sk, D))
    with fv.with_bf16_act(True):
        runs = _repeat(lambda: fv.sdpa(q, k, v, fv.Plan.kv_window()))
    assert _same(runs) and runs[0].dtype == torch.bfloat16
