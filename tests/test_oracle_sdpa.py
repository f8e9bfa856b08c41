"""Pins for the CPU oracle's dense path (bf16 rounding, host matmul/softmax,
composed SDPA, f64 checker) — independent of the oracle's own formulas:
torch's bf16 cast and float64 math, closed forms, invariants and brute force.
"""
import numpy as np
import pytest
import torch


def sin_tensor(n, k, shape):
    # C/rt/sdpa.rs:513-519: (i as f32 * k).sin() * 0.9, all in f32
    i = np.arange(n, dtype=np.float32)
    return (np.sin((i * np.float32(k)).astype(np.float32)).astype(np.float32) * np.float32(0.9)).reshape(shape)


def torch_sdpa_f64(q, k, v, scale, add_mask=None):
    q, k, v = (torch.from_numpy(np.asarray(x, dtype=np.float64)) for x in (q, k, v))
    s = torch.matmul(q, k.transpose(-1, -2)) * scale
    if add_mask is not None:
        s = s + torch.from_numpy(np.asarray(add_mask, dtype=np.float64))
    return torch.matmul(torch.softmax(s, dim=-1), v).numpy()


# ---- bf16 ------------------------------------------------------------------------

def test_bf16_rne_matches_torch_on_every_edge_class(oracle):
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2**32, size=200_000, dtype=np.uint64).astype(np.uint32)
    special = np.array([0x00000000, 0x80000000, 0x3F800000, 0x3F808000, 0x3F818000, 0x3F807FFF,
                        0x3F808001, 0x7F7FFFFF, 0x7F7F8000, 0x7F800000, 0xFF800000, 0x00000001,
                        0x00008000, 0x00018000, 0x007FFFFF, 0x7F7F7FFF], dtype=np.uint32)
    bits = np.concatenate([bits, special])
    x = bits.view(np.float32)
    finite_or_inf = ~np.isnan(x)
    got = oracle.to_bf16_bits(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got[finite_or_inf], want[finite_or_inf])
    # NaN stays NaN and quiet (C/rt/kernels/core.cu:9-13)
    nan_bits = got[~finite_or_inf]
    assert np.all((nan_bits & 0x7F80) == 0x7F80) and np.all((nan_bits & 0x0040) != 0)


def test_bf16_known_answers(oracle):
    # ties to even: 1 + 2^-8 is halfway between 1.0 and 1 + 2^-7
    assert oracle.bf16_rne_bits(1.0) == 0x3F80
    assert oracle.bf16_rne_bits(np.float32(1.0 + 2.0**-8)) == 0x3F80
    assert oracle.bf16_rne_bits(np.float32(1.0 + 3 * 2.0**-8)) == 0x3F82
    assert oracle.bf16_rne_bits(np.float32(3.4e38)) == 0x7F80  # past the largest finite bf16 -> inf
    assert oracle.bf16_rne_bits(-0.0) == 0x8000
    x = np.array([0.1, -2.5, 3.14159], dtype=np.float32)
    assert np.array_equal(oracle.from_bf16_bits(oracle.to_bf16_bits(x)), oracle.quantize_bf16(x))


# ---- host ops ----------------------------------------------------------------------

def test_matmul_is_sequential_f32_no_fma(oracle):
    # An input where FMA, pairwise or reversed summation change the f32 result.
    rng = np.random.default_rng(1)
    a = rng.standard_normal((2, 3, 37)).astype(np.float32) * 1e3
    b = rng.standard_normal((2, 37, 5)).astype(np.float32)
    got = oracle.matmul(a, b)
    want = np.zeros((2, 3, 5), dtype=np.float32)
    for bi in range(2):
        for i in range(3):
            for t in range(37):
                want[bi, i] = (want[bi, i] + (a[bi, i, t] * b[bi, t]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(got, want)
    ref64 = np.matmul(a.astype(np.float64), b.astype(np.float64))
    assert np.allclose(got, ref64, rtol=1e-5, atol=1e-2)
    assert np.array_equal(oracle.matmul(a, b, threads=2), got)


def test_matmul_detects_transposed_operand(oracle):
    a = np.arange(6, dtype=np.float32).reshape(1, 2, 3)
    b = np.arange(12, dtype=np.float32).reshape(1, 3, 4)
    assert np.array_equal(oracle.matmul(a, b)[0], a[0] @ b[0])


def test_softmax_rows_sum_to_one_and_match_f64(oracle):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal((7, 333)) * 4).astype(np.float32)
    p = oracle.softmax_last(x)
    assert np.allclose(p.sum(-1), 1.0, atol=2e-6)
    want = torch.softmax(torch.from_numpy(x.astype(np.float64)), -1).numpy()
    assert np.abs(p - want).max() < 1e-6
    # shift invariance (the max subtraction): exact for a power-of-two shift of exact values
    y = np.array([[0.0, 1.0, 2.0, 3.0]], dtype=np.float32)
    assert np.array_equal(oracle.softmax_last(y), oracle.softmax_last(y + 64.0))
    # uniform row -> exactly 1/n when n is a power of two
    assert np.array_equal(oracle.softmax_last(np.zeros((1, 8), np.float32)), np.full((1, 8), 0.125, np.float32))


def test_softmax_with_masked_entries(oracle):
    x = np.array([[0.0, -1e9, 0.0, -1e9]], dtype=np.float32)
    assert np.array_equal(oracle.softmax_last(x), np.array([[0.5, 0.0, 0.5, 0.0]], np.float32))


# ---- composed SDPA --------------------------------------------------------------------

def test_composed_on_the_reference_unit_test_inputs(oracle):
    # C/rt/sdpa.rs:522-542: 1x2x5x7x8, closed-form inputs
    h, sq, sk, d = 2, 5, 7, 8
    q = sin_tensor(h * sq * d, 0.37, (h, sq, d))
    k = sin_tensor(h * sk * d, 0.71, (h, sk, d))
    v = sin_tensor(h * sk * d, 1.13, (h, sk, d))
    got = oracle.sdpa_composed(q, k, v)
    want = torch_sdpa_f64(q, k, v, 1.0 / np.sqrt(8.0))
    assert np.abs(got - want).max() < 1e-6
    # a different scale changes the result (sdpa.rs:540-541)
    assert not np.array_equal(oracle.sdpa_composed(q, k, v, scale=0.5), got)
    # hand-rolled op-by-op restatement in numpy f32 (exp excluded: compare pre-softmax exactly)
    kt = np.ascontiguousarray(np.swapaxes(k, 1, 2))
    scores = oracle.matmul(q, kt) * np.float32(1.0 / np.sqrt(np.float32(8.0)))
    probs = oracle.softmax_last(scores)
    assert np.array_equal(oracle.matmul(probs, v), got)


@pytest.mark.parametrize("bh,sq,sk,d", [(1, 1, 1, 128), (2, 64, 64, 128), (3, 130, 1, 128),
                                        (2, 63, 257, 128), (2, 70, 70, 64), (12, 320, 320, 128)])
def test_composed_vs_f64_and_torch(oracle, bh, sq, sk, d):
    rng = np.random.default_rng(bh * 1000 + sq)
    q = rng.standard_normal((bh, sq, d)).astype(np.float32)
    k = rng.standard_normal((bh, sk, d)).astype(np.float32)
    v = rng.standard_normal((bh, sk, d)).astype(np.float32)
    scale = 1.0 / np.sqrt(d)
    got = oracle.sdpa_composed(q, k, v)
    want = torch_sdpa_f64(q, k, v, scale)
    # the reference measured composed-vs-f64 <= 7.7e-7 on its own cases
    assert np.abs(got - want).max() < 5e-6
    f64 = oracle.sdpa_f64(q, k, v)
    assert np.abs(f64 - want).max() < 1e-6
    # threads split heads only and change nothing
    assert np.array_equal(oracle.sdpa_composed(q, k, v, threads=1), got)


def test_composed_rows_equal_full_bit_for_bit(oracle):
    rng = np.random.default_rng(7)
    bh, sq, sk, d = 3, 97, 211, 128
    q = rng.standard_normal((bh, sq, d)).astype(np.float32)
    k = rng.standard_normal((bh, sk, d)).astype(np.float32)
    v = rng.standard_normal((bh, sk, d)).astype(np.float32)
    full = oracle.sdpa_composed(q, k, v)
    rows = np.array([0, 5, 96, 31, 64])
    assert np.array_equal(oracle.sdpa_composed_rows(q, k, v, rows), full[:, rows])
    f64 = oracle.sdpa_f64(q, k, v)
    assert np.array_equal(oracle.sdpa_f64(q, k, v, rows=rows), f64[:, rows])


def test_composed_with_additive_mask(oracle):
    rng = np.random.default_rng(8)
    bh, s, d = 2, 48, 16
    q = rng.standard_normal((bh, s, d)).astype(np.float32)
    k = rng.standard_normal((bh, s, d)).astype(np.float32)
    v = rng.standard_normal((bh, s, d)).astype(np.float32)
    mask = oracle.block_causal_dense_mask(5, 2, 1, s, s)
    got = oracle.sdpa_composed(q, k, v, mask=mask)
    want = torch_sdpa_f64(q, k, v, 1.0 / np.sqrt(d), add_mask=mask)
    assert np.abs(got - want).max() < 5e-6
    # rows variant applies the same 0 / -1e9 mask from the BlockCausal triple
    rows = np.arange(s)
    assert np.array_equal(oracle.sdpa_composed_rows(q, k, v, rows, mask_bc=(5, 2, 1)), got)
    # -1e9 additive vs -inf in the f64 checker: identical to f32 resolution
    f64 = oracle.sdpa_f64(q, k, v, mask_bc=(5, 2, 1))
    assert np.abs(f64 - want).max() < 1e-6
    # first query (block 0) sees only the first five keys (C/rt/attn.rs:924-929)
    p = torch.softmax(torch.from_numpy((q[0, 0].astype(np.float64) @ k[0, :5].astype(np.float64).T) / np.sqrt(d)), -1).numpy()
    assert np.abs(got[0, 0] - p @ v[0, :5].astype(np.float64)).max() < 5e-6
    assert not np.allclose(got[0, 0], oracle.sdpa_composed(q, k, v)[0, 0])


def test_uniform_values_are_reproduced(oracle):
    # softmax weights sum to one: constant V comes back unchanged
    rng = np.random.default_rng(9)
    q = rng.standard_normal((1, 9, 32)).astype(np.float32)
    k = rng.standard_normal((1, 17, 32)).astype(np.float32)
    v = np.full((1, 17, 32), 0.75, dtype=np.float32)
    assert np.abs(oracle.sdpa_composed(q, k, v) - 0.75).max() < 1e-6
    # one key: output is that key's value row exactly
    v1 = rng.standard_normal((1, 1, 32)).astype(np.float32)
    out = oracle.sdpa_composed(q, k[:, :1], v1)
    assert np.array_equal(out, np.broadcast_to(v1, out.shape))
