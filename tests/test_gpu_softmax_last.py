"""Row softmax entry (`fv_softmax_last`) against the oracle's host form of the reference's
`softmax_last` (crates/fastvideo-cudarc/src/rt/ops.rs:2178-2193; kernels rt/kernels/core.cu:177-252).

Tolerances: the host form sums a row's exponentials one after another in f32; that sum drops the terms
below half a unit of the running total and is off by up to width * 2^-24 relative (5e-5 measured at
width 32760), where the device (like the reference's own kernel) sums a tree. So f32 out is held
within 2^-24 * (8 + width) relative of the oracle, and within 5e-7 relative of the f64 softmax of the
same f32-shifted scores, which is the tight pin of the kernel; rows sum to 1 within 2e-6; bf16 out
within one bf16 step of the rounded f64 value.
"""
import numpy as np
import pytest

from util import announce

pytestmark = pytest.mark.gpu

F64_REL = 5e-7


def oracle_rel(width):
    return 2.0 ** -24 * (8 + width)


def f64_softmax(x):
    # the shifted scores as both forms compute them (one f32 subtraction), everything after in f64
    e = np.exp((x - x.max(-1, keepdims=True)).astype(np.float64))
    return e / e.sum(-1, keepdims=True)


@pytest.fixture(scope="module")
def fv():
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


def dev(x):
    import torch

    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def host(t):
    import torch

    torch.cuda.synchronize()
    return t.float().cpu().numpy()


# one wave per row (<= 1024), four waves per row (<= 4096), sixteen above, with the row in registers up to
# 32768 and a re-read tail beyond; widths off every wave multiple; row counts off the 4-row group
SHAPES = [(1, 1), (3, 7), (5, 64), (9, 333), (13, 624), (6, 1023), (4, 1024), (7, 1025), (3, 4096), (5, 4097),
          (2, 9001), (3, 32760), (2, 32768), (2, 32769), (1, 70001), (12 * 8, 624)]


@pytest.mark.parametrize("rows,width", SHAPES)
def test_f32_rows_match_the_host_form(fv, oracle, rows, width):
    announce(f"softmax_last f32 rows={rows} width={width}")
    rng = np.random.default_rng(rows * 100003 + width)
    x = (rng.standard_normal((rows, width)) * 4).astype(np.float32)
    want = oracle.softmax_last(x)
    got = host(fv.softmax_last(dev(x)))
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= oracle_rel(width) * want + 1e-37)
    exact = f64_softmax(x)
    assert np.all(np.abs(got - exact) <= F64_REL * exact + 1e-37)
    assert np.allclose(got.sum(-1, dtype=np.float64), 1.0, atol=2e-6)


@pytest.mark.parametrize("rows,width", [(3, 7), (9, 333), (13, 624), (7, 1025), (5, 4097), (2, 9001), (2, 40000)])
def test_bf16_rows_are_the_rounded_host_form(fv, oracle, rows, width):
    announce(f"softmax_last bf16 rows={rows} width={width}")
    rng = np.random.default_rng(rows * 7919 + width)
    x = (rng.standard_normal((rows, width)) * 3).astype(np.float32)
    want = f64_softmax(x).astype(np.float32)
    got_bits = fv.softmax_last(dev(x), out_bf16=True)
    import torch

    torch.cuda.synchronize()
    got_bits = got_bits.view(torch.int16).cpu().numpy().view(np.uint16)
    want_bits = oracle.to_bf16_bits(want)
    # positive finite values: bf16 bit patterns are ordered, one step = one unit of the pattern
    step = np.abs(got_bits.astype(np.int32) - want_bits.astype(np.int32))
    assert step.max() <= 1
    assert (step == 0).mean() > 0.99


def test_closed_forms(fv):
    # uniform row -> exactly 1/n for a power-of-two n; shift invariance exact for exact values;
    # masked entries (-1e9 and -inf) get exactly 0
    z = host(fv.softmax_last(dev(np.zeros((5, 2048), np.float32))))
    assert np.array_equal(z, np.full((5, 2048), 1.0 / 2048, np.float32))
    y = np.array([[0.0, 1.0, 2.0, 3.0]], np.float32)
    assert np.array_equal(host(fv.softmax_last(dev(y))), host(fv.softmax_last(dev(y + 64.0))))
    m = np.array([[0.0, -1e9, 0.0, -np.inf]], np.float32)
    assert np.array_equal(host(fv.softmax_last(dev(m))), np.array([[0.5, 0.0, 0.5, 0.0]], np.float32))
    # a one-hot row at a score far above the rest
    w = np.full((2, 5000), -50.0, np.float32)
    w[0, 4999] = 80.0
    w[1, 0] = 80.0
    p = host(fv.softmax_last(dev(w)))
    assert p[0, 4999] == 1.0 and p[1, 0] == 1.0 and p.sum() == 2.0


def test_in_place_and_leading_axes(fv, oracle):
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((2, 3, 5, 700)) * 2).astype(np.float32)
    want = oracle.softmax_last(x)
    t = dev(x)
    r = fv.softmax_last(t, out=t)
    assert r.data_ptr() == t.data_ptr()
    got = host(t)
    assert got.shape == x.shape
    assert np.all(np.abs(got - want) <= oracle_rel(700) * want + 1e-37)
    # the bf16 form would overwrite rows other workgroups have not read yet: refused
    rc = fv.lib().fv_softmax_last(t.data_ptr(), t.data_ptr(), 1, 30, 700, None)
    assert rc < 0 and b"in place" in fv.lib().fv_sdpa_last_error()


def test_empty(fv):
    import torch

    e = fv.softmax_last(torch.empty((0, 16), device="cuda"))
    assert e.shape == (0, 16)
