"""The fused kernels' form for calls whose scale * log2(e) is exactly 1 (scale = ln 2: the caller folded the
softmax scale into Q before Q's one rounding to bf16). The softmax offset then rides in the C operand of the
K Q^T MFMAs and the multiply-add per score is gone; everything else is the same kernel, so the bars are the
same ones, through the C ABI, against the oracle's fp32 composed SDPA on the same bf16-valued operands at the
same scale: max|delta| <= 1e-2, cosine >= 0.9999, rel_l2 <= 2e-3 (only P's rounding is left,
crates/fastvideo-gpucheck/src/kernels.rs:2314-2328), and rel_l2 <= 1e-2 against the f32 math on the unrounded,
unfolded operands at the call's real scale (the fold costs no accuracy: Q is still rounded once).
"""
import math

import numpy as np
import pytest

from util import announce, assert_parity, metrics, randn, to_dev_bf16, assert_bf16_result_matches_f32_result

pytestmark = pytest.mark.gpu

LN2 = float(np.float32(math.log(2.0)))


@pytest.fixture(scope="module")
def fv():
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


def folded_qkv(oracle, seed, bh, sq, sk, d, std=1.0):
    """f32 q, k, v and what a folding caller hands the kernel: bf16(q * scale * log2 e), bf16(k), bf16(v)."""
    q, k, v = randn(seed, (bh, sq, d), std), randn(seed + 1, (bh, sk, d), std), randn(seed + 2, (bh, sk, d))
    sl2 = np.float32(1.0 / math.sqrt(d)) * np.float32(1.4426950408889634)
    qf = oracle.quantize_bf16(q * sl2)
    return (q, k, v), (qf, oracle.quantize_bf16(k), oracle.quantize_bf16(v))


def test_the_predicate_and_the_form_taken(fv, oracle):
    import torch

    lib = fv.lib()
    assert lib.fv_sdpa_is_log2_domain_scale(LN2) == 1
    for d in (64, 128):
        assert lib.fv_sdpa_is_log2_domain_scale(1.0 / math.sqrt(d)) == 0
    assert lib.fv_sdpa_is_log2_domain_scale(1.0) == 0
    # the launch counter moves with calls at scale ln 2, through every fused entry, and with no other call
    _, (qf, kr, vr) = folded_qkv(oracle, 5000, 2, 300, 300, 128)
    qd, kd, vd = (to_dev_bf16(x) for x in (qf, kr, vr))
    n0 = lib.fv_sdpa_log2_domain_launches()
    fv.sdpa_dense_bf16(qd, kd, vd)
    fv.sdpa_block_causal_bf16(qd, kd, vd, 100, 0, 0)
    assert lib.fv_sdpa_log2_domain_launches() == n0
    fv.sdpa_dense_bf16(qd, kd, vd, scale=LN2)
    fv.sdpa_block_causal_bf16(qd, kd, vd, 100, 0, 0, scale=LN2)
    fv.sdpa_vdn_window_bf16(qd, kd, vd, 10, 20, 14, 0, 1, scale=LN2)
    fv.sdpa_dense_bf16_splitkv(qd, kd, vd, splits=2, scale=LN2)
    torch.cuda.synchronize()
    assert lib.fv_sdpa_log2_domain_launches() == n0 + 4


SHAPES = [  # (bh, sq, sk, std, d)
    (1, 1, 1, 1.0, 128),
    (2, 64, 64, 1.0, 128),
    (6, 257, 257, 1.0, 128),
    (4, 300, 512, 1.0, 128),
    (3, 130, 1, 1.0, 128),
    (2, 63, 4097, 1.0, 128),
    (4, 1024, 1024, 2.0, 128),
    (2, 2048, 2048, 1.0, 128),
    (12, 320, 320, 1.0, 128),
    (1, 127, 63, 1.0, 128),
    (2, 70, 70, 1.0, 64),
    (4, 1000, 333, 1.0, 64),
    (3, 259, 129, 1.0, 64),
    (2, 777, 4097, 2.0, 64),
]


@pytest.mark.parametrize("bh,sq,sk,std,d", SHAPES)
def test_dense(fv, oracle, bh, sq, sk, std, d):
    import torch

    seed = 5100 + bh * 7 + sq + d
    announce(f"log2-domain dense bh={bh} sq={sq} sk={sk} d={d} std={std} seed={seed}")
    (q, k, v), (qf, kr, vr) = folded_qkv(oracle, seed, bh, sq, sk, d, std)
    want = oracle.sdpa_composed(qf, kr, vr, scale=LN2)
    qd, kd, vd = (to_dev_bf16(x) for x in (qf, kr, vr))
    got = fv.sdpa_dense_bf16(qd, kd, vd, scale=LN2)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    m = assert_parity(got, want, f"log2_dense_{bh}x{sq}x{sk}x{d}_s{std}", max_abs=1e-2 if std == 1.0 else 5e-2)
    assert m["rel_l2"] <= 2e-3 * (1 if std == 1.0 else 3)
    # against the f32 math on the unrounded, unfolded operands
    assert metrics(got, oracle.sdpa_composed(q, k, v))["rel_l2"] <= 1e-2
    got16 = fv.sdpa_dense_bf16(qd, kd, vd, scale=LN2, out_bf16=True)
    torch.cuda.synchronize()
    assert_bf16_result_matches_f32_result(got16.float().cpu().numpy(), got, f"log2_dense_{bh}x{sq}x{sk}x{d}_s{std}",
                                          1.0 if std == 1.0 else 0.5)
    # the same call one ulp of scale away runs the general form: two roundings of the same numbers apart
    near = fv.sdpa_dense_bf16(qd, kd, vd, scale=float(np.nextafter(np.float32(LN2), np.float32(1.0))))
    torch.cuda.synchronize()
    assert metrics(near.cpu().numpy(), want)["rel_l2"] <= 2e-3 * (1 if std == 1.0 else 3)


def test_scores_that_force_rescales(fv, oracle):
    """Keys ordered so that every query's running max keeps growing by more than the rescale threshold, rows
    that see -inf only at first (tail of a partial tile), and a large common shift of all scores."""
    import torch

    bh, sq, sk, d = 2, 200, 1000, 128
    announce("log2-domain dense, growing maxima")
    g = np.random.Generator(np.random.PCG64(77))
    q = g.standard_normal((bh, sq, d), dtype=np.float32)
    k = g.standard_normal((bh, sk, d), dtype=np.float32) * (0.2 + 3.0 * np.arange(sk, dtype=np.float32)[None, :, None] / sk)
    v = g.standard_normal((bh, sk, d), dtype=np.float32)
    sl2 = np.float32(1.0 / math.sqrt(d)) * np.float32(1.4426950408889634)
    qf, kr, vr = oracle.quantize_bf16(q * sl2 * 4.0), oracle.quantize_bf16(k), oracle.quantize_bf16(v)
    want = oracle.sdpa_f64(qf, kr, vr, scale=LN2)
    got = fv.sdpa_dense_bf16(*(to_dev_bf16(x) for x in (qf, kr, vr)), scale=LN2)
    torch.cuda.synchronize()
    assert_parity(got.cpu().numpy(), want, "log2_growing_maxima", max_abs=2e-2)


CAUSAL = [  # (bh, s, block_tokens, window, sink, d)
    (2, 640, 128, 1, 0, 128),
    (2, 1000, 64, 2, 3, 128),
    (1, 777, 100, 1, 0, 128),
    (2, 1500, 192, 2, 2, 64),
    (1, 900, 300, 0, 0, 128),
]


@pytest.mark.parametrize("bh,s,bt,win,sink,d", CAUSAL)
def test_block_causal(fv, oracle, bh, s, bt, win, sink, d):
    import torch

    announce(f"log2-domain causal bh={bh} s={s} d={d} block={bt} window={win} sink={sink}")
    _, (qf, kr, vr) = folded_qkv(oracle, 5300 + s + d, bh, s, s, d)
    mask = oracle.block_causal_dense_mask(bt, win, sink, s, s)
    want = oracle.sdpa_composed(qf, kr, vr, scale=LN2, mask=mask)
    qd, kd, vd = (to_dev_bf16(x) for x in (qf, kr, vr))
    got = fv.sdpa_block_causal_bf16(qd, kd, vd, bt, win, sink, scale=LN2)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    m = assert_parity(got, want, f"log2_causal_{s}_{bt}_{win}_{sink}")
    assert m["rel_l2"] <= 2e-3


def test_more_queries_than_keys_with_a_window(fv, oracle):
    """Rows and whole tiles without a visible key come out as zeros in this form too."""
    import torch

    bh, sq, sk, bt, win, sink, d = 2, 700, 300, 100, 1, 0, 128
    announce("log2-domain causal, sq > sk with a window")
    _, (qf, kr, vr) = folded_qkv(oracle, 5400, bh, sq, sk, d)
    mask = oracle.block_causal_dense_mask(bt, win, sink, sq, sk)
    want = oracle.sdpa_composed(qf, kr, vr, scale=LN2, mask=mask)
    visible = (mask == 0).any(axis=1)
    want[:, ~visible, :] = 0.0   # the kernel's convention for a row without a visible key
    qd, kd, vd = (to_dev_bf16(x) for x in (qf, kr, vr))
    out = torch.full((bh, sq, d), float("nan"), device="cuda")
    got = fv.sdpa_block_causal_bf16(qd, kd, vd, bt, win, sink, scale=LN2, out=out)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert_parity(got, want, "log2_causal_sq_gt_sk")
    assert not got[:, ~visible, :].any()


def test_vdn_window(fv, oracle):
    import torch

    bh, s, vs, t, frames, chunk, radius, d = 2, 1300, 20, 40, 32, 5, 1, 128
    announce("log2-domain vdn window")
    _, (qf, kr, vr) = folded_qkv(oracle, 5500, bh, s, s, d)
    mask = oracle.vdn_window_dense_mask(vs, t, frames, chunk, radius, s, s)
    want = oracle.sdpa_composed(qf, kr, vr, scale=LN2, mask=mask)
    got = fv.sdpa_vdn_window_bf16(*(to_dev_bf16(x) for x in (qf, kr, vr)), vs, t, frames, chunk, radius, scale=LN2)
    torch.cuda.synchronize()
    m = assert_parity(got.cpu().numpy(), want, "log2_vdn_window")
    assert m["rel_l2"] <= 2e-3


@pytest.mark.parametrize("d", [128, 64])
def test_split_kv(fv, oracle, d):
    import torch

    bh, sq, sk = 3, 257, 2049
    announce(f"log2-domain splitkv d={d}")
    _, (qf, kr, vr) = folded_qkv(oracle, 5600 + d, bh, sq, sk, d)
    want = oracle.sdpa_composed(qf, kr, vr, scale=LN2)
    tq, tk, tv = (to_dev_bf16(x) for x in (qf, kr, vr))
    base = fv.sdpa_dense_bf16(tq, tk, tv, scale=LN2)
    for splits in (1, 2, 5, 1000):
        got = fv.sdpa_dense_bf16_splitkv(tq, tk, tv, splits=splits, scale=LN2)
        torch.cuda.synchronize()
        if splits == 1:
            assert torch.equal(got, base)
        assert (got - base).abs().max().item() <= 2e-3, splits
        assert_parity(got.cpu().numpy(), want, f"log2_splitkv_{splits}_{d}")


def test_headline_shape_sampled_rows(fv, oracle):
    """Wan-1.3B 480p self-attention at full size, folded operands: 512 sampled rows x 12 heads."""
    import torch

    h, s, d = 12, 32760, 128
    announce("log2-domain dense H=12 S=32760, sampled rows")
    g = torch.Generator(device="cuda").manual_seed(5700)
    sl2 = (1.0 / math.sqrt(d)) * 1.4426950408889634
    q = (torch.randn((h, s, d), generator=g, device="cuda") * sl2).to(torch.bfloat16)
    k = torch.randn((h, s, d), generator=g, device="cuda").to(torch.bfloat16)
    v = torch.randn((h, s, d), generator=g, device="cuda").to(torch.bfloat16)
    got = fv.sdpa_dense_bf16(q, k, v, scale=LN2, out_bf16=True)
    torch.cuda.synchronize()
    rows = np.unique(np.concatenate([np.random.Generator(np.random.PCG64(5)).integers(0, s, 500),
                                     [0, 255, 256, 32511, 32512, s - 1]])).astype(np.int64)
    want = oracle.sdpa_composed_rows(q.float().cpu().numpy(), k.float().cpu().numpy(), v.float().cpu().numpy(), rows,
                                     scale=LN2)
    assert_parity(got.float().cpu().numpy()[:, rows, :], want, "log2_headline_rows")


def test_fold_through_the_q_norm_weight(fv, oracle):
    """The caller's recipe end to end: the q RMSNorm weight carries scale * log2 e, the producer's bf16 kernel
    rounds q once as it always does, and the SDPA call passes scale = ln 2. The result meets the bars against
    the oracle on the producer's own output at ln 2, and sits within the fused bar of the unfolded chain
    (weight w, default scale), whose q differs by the rounding noise of one bf16 product."""
    import torch

    batch, seq, heads, d = 1, 700, 4, 128
    announce("fold through q norm weight: prep -> sdpa(ln 2), 1x700x4x128")
    rng = np.random.Generator(np.random.PCG64(5900))
    qkv = oracle.quantize_bf16(rng.standard_normal((batch, seq, 3 * heads * d)).astype(np.float32))
    w = (1.0 + 0.2 * rng.standard_normal(heads * d)).astype(np.float32)
    theta = rng.uniform(-3.0, 3.0, (seq, d // 2))
    cos = np.repeat(np.cos(theta), 2, axis=1).astype(np.float32)
    sin = np.repeat(np.sin(theta), 2, axis=1).astype(np.float32)
    sl2 = np.float32(1.0 / math.sqrt(d)) * np.float32(1.4426950408889634)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    x = dev(qkv).to(torch.bfloat16)
    rope = (dev(cos), dev(sin))
    k = fv.qk_norm_rope_bhsd(x, heads * d, heads, dev(w), rope).reshape(heads, seq, d)
    v = fv.split_heads_bhsd(x, 2 * heads * d, heads, d).reshape(heads, seq, d)
    q_plain = fv.qk_norm_rope_bhsd(x, 0, heads, dev(w), rope).reshape(heads, seq, d)
    q_fold = fv.qk_norm_rope_bhsd(x, 0, heads, dev(w * sl2), rope).reshape(heads, seq, d)
    n0 = fv.lib().fv_sdpa_log2_domain_launches()
    plain = fv.sdpa_dense_bf16(q_plain, k, v)
    assert fv.lib().fv_sdpa_log2_domain_launches() == n0
    got = fv.sdpa_dense_bf16(q_fold, k, v, scale=LN2)
    torch.cuda.synchronize()
    assert fv.lib().fv_sdpa_log2_domain_launches() == n0 + 1
    npy = lambda t: t.float().cpu().numpy()  # noqa: E731
    want = oracle.sdpa_composed(npy(q_fold), npy(k), npy(v), scale=LN2)
    assert_parity(npy(got), want, "log2_fold_norm_weight")
    m = metrics(npy(got), npy(plain))
    assert m["max_abs"] <= 1e-2 and m["cosine"] >= 0.9999, m
