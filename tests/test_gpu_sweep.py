"""Seeded sweep of ragged shapes through every fused entry (dense, block-causal incl. more queries than keys,
VDN window, split-KV on row windows, composed f32 with an additive mask, top-k): shapes, mask parameters and
inputs all come from numpy's PCG64 under the case's seed, so a failure names a reproducible case. Every case
is an ordinary parity check against the oracle, to the limits of the per-kernel test files."""
import numpy as np
import pytest

from util import announce, assert_parity, qkv, to_dev_bf16

pytestmark = pytest.mark.gpu

KINDS = ["dense", "block_causal", "vdn_window", "splitkv_window", "composed_masked", "topk"]


@pytest.fixture(scope="module")
def fv():
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


@pytest.mark.parametrize("seed", range(10))
@pytest.mark.parametrize("kind", KINDS)
def test_seeded_case(fv, oracle, kind, seed):
    import torch

    rng = np.random.Generator(np.random.PCG64(1000 * KINDS.index(kind) + seed))
    d = int(rng.choice([64, 128]))
    bh = int(rng.integers(1, 5))
    sq, sk = int(rng.integers(1, 700)), int(rng.integers(1, 900))
    data_seed = int(rng.integers(0, 1 << 30))
    if kind == "dense":
        announce(f"sweep dense bh={bh} sq={sq} sk={sk} d={d} seed={data_seed}")
        q, k, v = qkv(data_seed, bh, sq, sk, d)
        got = fv.sdpa_dense_bf16(*(to_dev_bf16(x) for x in (q, k, v)))
        torch.cuda.synchronize()
        assert_parity(got.cpu().numpy(), oracle.sdpa_composed(q, k, v), f"sweep_dense_{seed}")
    elif kind == "block_causal":
        if seed % 2:
            sk = sq                                   # the reference's own calls are square
        bt = int(rng.integers(1, max(2, max(sq, sk))))
        win, sink = int(rng.integers(0, 4)), int(rng.integers(0, 3))
        announce(f"sweep causal bh={bh} sq={sq} sk={sk} d={d} block={bt} window={win} sink={sink} seed={data_seed}")
        q, k, v = qkv(data_seed, bh, sq, sk, d)
        out = torch.full((bh, sq, d), float("nan"), device="cuda")
        fv.sdpa_block_causal_bf16(*(to_dev_bf16(x) for x in (q, k, v)), bt, win, sink, out=out)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        tq, tk = np.arange(sq)[:, None] // bt, np.arange(sk)[None, :] // bt
        live = ((tk < sink) | ((tk <= tq) & ((win == 0) | (tq - tk < win)))).any(axis=1)
        assert np.isfinite(got).all() and np.all(got[:, ~live] == 0.0)      # rows without a visible key: zeros
        if live.any():
            want = oracle.sdpa_f64(q, k, v, mask_bc=(bt, win, sink), rows=np.nonzero(live)[0])
            assert_parity(got[:, live], want, f"sweep_causal_{seed}")
    elif kind == "vdn_window":
        ft, frames = int(rng.integers(1, 60)), int(rng.integers(1, 12))
        vs, tail = int(rng.integers(0, 50)), int(rng.integers(0, 50))
        s = vs + ft * frames + tail
        chunk, radius = int(rng.integers(0, 4)), int(rng.integers(0, 4))
        announce(f"sweep vdn bh={bh} s={s} d={d} start={vs} ft={ft} frames={frames} chunk={chunk} radius={radius} seed={data_seed}")
        q, k, v = qkv(data_seed, bh, s, s, d)
        got = fv.sdpa_vdn_window_bf16(*(to_dev_bf16(x) for x in (q, k, v)), vs, ft, frames, chunk, radius)
        torch.cuda.synchronize()
        mask = oracle.vdn_window_dense_mask(vs, ft, frames, chunk, radius, s, s)
        assert_parity(got.cpu().numpy(), oracle.sdpa_composed(q, k, v, mask=mask), f"sweep_vdn_{seed}")
    elif kind == "splitkv_window":
        sk2 = sk + 600
        off, splits = int(rng.integers(0, 77)), int(rng.integers(1, 9))
        announce(f"sweep splitkv bh={bh} sq={sq} sk={sk2} d={d} offset={off} splits={splits} seed={data_seed}")
        q, k, v = qkv(data_seed, bh, sq, sk2 + 77, d)
        tk, tv = to_dev_bf16(k), to_dev_bf16(v)
        got = fv.sdpa_dense_bf16_splitkv(to_dev_bf16(q), tk[:, off:off + sk2], tv[:, off:off + sk2], splits=splits)
        torch.cuda.synchronize()
        want = oracle.sdpa_composed(q, np.ascontiguousarray(k[:, off:off + sk2]), np.ascontiguousarray(v[:, off:off + sk2]))
        assert_parity(got.cpu().numpy(), want, f"sweep_splitkv_{seed}")
    elif kind == "composed_masked":
        d = int(rng.choice([32, 48, 64, 96, 128]))     # 48: the scalar kernel; the rest: fp32 MFMA
        announce(f"sweep composed bh={bh} sq={sq} sk={sk} d={d} seed={data_seed}")
        q, k, v = qkv(data_seed, bh, sq, sk, d, round_bf16=False)
        mask = (rng.standard_normal((sq, sk)) * 3).astype(np.float32)
        mask[rng.random((sq, sk)) < 0.2] = -1e9
        mask[:, 0] = 0.0
        tq, tk, tv, tm = (torch.from_numpy(np.ascontiguousarray(x)).cuda() for x in (q, k, v, mask))
        out = torch.empty((bh, sq, d), device="cuda")
        rc = fv.lib().fv_sdpa_composed_f32(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), tm.data_ptr(), 0, out.data_ptr(), bh,
                                           sq, sk, d, float(d) ** -0.5, torch.cuda.current_stream().cuda_stream)
        assert rc == 0, fv.lib().fv_sdpa_last_error().decode()
        torch.cuda.synchronize()
        assert_parity(out.cpu().numpy(), oracle.sdpa_composed(q, k, v, mask=mask), f"sweep_composed_{seed}", max_abs=5e-5)
    else:
        rows, n = int(rng.integers(1, 40)), int(rng.integers(1, 4097))
        kk = int(rng.integers(1, n + 20))
        levels = int(rng.choice([0, 4, 64]))           # 0: distinct values; else heavy ties
        announce(f"sweep topk rows={rows} n={n} k={kk} levels={levels} seed={data_seed}")
        s = np.random.Generator(np.random.PCG64(data_seed)).standard_normal((rows, n)).astype(np.float32)
        if levels:
            s = (np.round(s * levels) / levels).astype(np.float32)
        got = fv.vsa_topk(torch.from_numpy(s).cuda(), kk)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy().view(np.uint32), oracle.topk_device_order(s, kk))


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("kind", KINDS[:4])
def test_seeded_case_log2_domain(fv, oracle, kind, seed):
    """The same sweep through the form for calls at scale ln 2 (softmax scale folded into Q before its rounding)."""
    import math

    import torch

    from util import randn

    rng = np.random.Generator(np.random.PCG64(50000 + 1000 * KINDS.index(kind) + seed))
    d = int(rng.choice([64, 128]))
    bh = int(rng.integers(1, 5))
    sq, sk = int(rng.integers(1, 700)), int(rng.integers(1, 900))
    data_seed = int(rng.integers(0, 1 << 30))
    ln2 = float(np.float32(math.log(2.0)))
    assert fv.lib().fv_sdpa_is_log2_domain_scale(ln2) == 1

    def operands(nq, nk):
        sl2 = np.float32(1.0 / math.sqrt(d)) * np.float32(1.4426950408889634)
        q = oracle.quantize_bf16(randn(data_seed, (bh, nq, d)) * sl2)
        return q, oracle.quantize_bf16(randn(data_seed + 1, (bh, nk, d))), oracle.quantize_bf16(randn(data_seed + 2, (bh, nk, d)))

    if kind == "dense":
        announce(f"sweep log2 dense bh={bh} sq={sq} sk={sk} d={d} seed={data_seed}")
        q, k, v = operands(sq, sk)
        got = fv.sdpa_dense_bf16(*(to_dev_bf16(x) for x in (q, k, v)), scale=ln2)
        torch.cuda.synchronize()
        assert_parity(got.cpu().numpy(), oracle.sdpa_composed(q, k, v, scale=ln2), f"sweep_log2_dense_{seed}")
    elif kind == "block_causal":
        if seed % 2:
            sk = sq
        bt = int(rng.integers(1, max(2, max(sq, sk))))
        win, sink = int(rng.integers(0, 4)), int(rng.integers(0, 3))
        announce(f"sweep log2 causal bh={bh} sq={sq} sk={sk} d={d} block={bt} window={win} sink={sink} seed={data_seed}")
        q, k, v = operands(sq, sk)
        out = torch.full((bh, sq, d), float("nan"), device="cuda")
        fv.sdpa_block_causal_bf16(*(to_dev_bf16(x) for x in (q, k, v)), bt, win, sink, scale=ln2, out=out)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        tq, tk = np.arange(sq)[:, None] // bt, np.arange(sk)[None, :] // bt
        live = ((tk < sink) | ((tk <= tq) & ((win == 0) | (tq - tk < win)))).any(axis=1)
        assert np.isfinite(got).all() and np.all(got[:, ~live] == 0.0)
        if live.any():
            want = oracle.sdpa_f64(q, k, v, scale=ln2, mask_bc=(bt, win, sink), rows=np.nonzero(live)[0])
            assert_parity(got[:, live], want, f"sweep_log2_causal_{seed}")
    elif kind == "vdn_window":
        ft, frames = int(rng.integers(1, 60)), int(rng.integers(1, 12))
        vs, tail = int(rng.integers(0, 50)), int(rng.integers(0, 50))
        s = vs + ft * frames + tail
        chunk, radius = int(rng.integers(0, 4)), int(rng.integers(0, 4))
        announce(f"sweep log2 vdn bh={bh} s={s} d={d} start={vs} ft={ft} frames={frames} chunk={chunk} radius={radius} seed={data_seed}")
        q, k, v = operands(s, s)
        got = fv.sdpa_vdn_window_bf16(*(to_dev_bf16(x) for x in (q, k, v)), vs, ft, frames, chunk, radius, scale=ln2)
        torch.cuda.synchronize()
        mask = oracle.vdn_window_dense_mask(vs, ft, frames, chunk, radius, s, s)
        assert_parity(got.cpu().numpy(), oracle.sdpa_composed(q, k, v, scale=ln2, mask=mask), f"sweep_log2_vdn_{seed}")
    else:
        sk2 = sk + 600
        off, splits = int(rng.integers(0, 77)), int(rng.integers(1, 9))
        announce(f"sweep log2 splitkv bh={bh} sq={sq} sk={sk2} d={d} offset={off} splits={splits} seed={data_seed}")
        q, k, v = operands(sq, sk2 + 77)
        tk, tv = to_dev_bf16(k), to_dev_bf16(v)
        got = fv.sdpa_dense_bf16_splitkv(to_dev_bf16(q), tk[:, off:off + sk2], tv[:, off:off + sk2], splits=splits, scale=ln2)
        torch.cuda.synchronize()
        want = oracle.sdpa_composed(q, np.ascontiguousarray(k[:, off:off + sk2]), np.ascontiguousarray(v[:, off:off + sk2]),
                                    scale=ln2)
        assert_parity(got.cpu().numpy(), want, f"sweep_log2_splitkv_{seed}")
