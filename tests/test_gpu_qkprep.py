"""GPU parity of the producer / consumer either side of the SDPA call, through the C ABI,
against the oracle's restatement of the reference's host forms.

The permutes are bit-exact. The f32 q/k op differs from the host form only by the
summation order of the row's sum of squares (lane-strided + butterfly on the GPU, index
order on the host), so it is compared at 2e-6 relative. The bf16 q/k kernel rounds three
times; a last-bit difference in `inv` can flip the first rounding and that flip can flip
the second, so the bar is: under 0.1 % of the values differ at all, by at most two bf16
ulps without rotation, and by at most 0.03 with it (the rotation can cancel; 0.03 is the
bound of the reference's own host test of this kernel's form, wan/fuse.rs:660-661).
"""
import numpy as np
import pytest

from util import announce

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fv():
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


def _inputs(seed, batch, seq, heads, d, extra, col_off):
    rng = np.random.Generator(np.random.PCG64(seed))
    width = heads * d
    proj = rng.standard_normal((batch, seq, col_off + width + extra)).astype(np.float32)
    w = (1.0 + 0.2 * rng.standard_normal(width)).astype(np.float32)
    theta = rng.uniform(-3.0, 3.0, (seq, d // 2))
    cos = np.repeat(np.cos(theta), 2, axis=1).astype(np.float32)
    sin = np.repeat(np.sin(theta), 2, axis=1).astype(np.float32)
    return proj, w, cos, sin


def _ulps(a, b, oracle):
    ba = oracle.to_bf16_bits(a).astype(np.int32)
    bb = oracle.to_bf16_bits(b).astype(np.int32)
    key = lambda v: np.where(v & 0x8000, 0x8000 - (v & 0x7fff), 0x8000 + (v & 0x7fff))  # noqa: E731
    return np.abs(key(ba) - key(bb))


CASES = [
    # batch, seq, heads, d, extra cols, col_off
    (1, 4, 2, 8, 0, 0),
    (2, 37, 3, 64, 8, 192),       # fused QKV projection, k slice
    (1, 130, 12, 128, 0, 1536),   # Wan-1.3B width, middle slice of a 3x projection
    (1, 65, 40, 128, 0, 0),       # Wan-14B width: more than one chunk pass per lane
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("rope", [False, True])
def test_f32_op(fv, oracle, case, rope):
    import torch

    batch, seq, heads, d, extra, col_off = case
    if col_off and extra == 0:
        extra = 2 * heads * d - col_off if col_off < 2 * heads * d else 0
    announce(f"qk_norm_rope f32 {case} rope={rope}")
    proj, w, cos, sin = _inputs(7, batch, seq, heads, d, extra, col_off)
    want = oracle.qk_norm_rope_bhsd(proj, col_off, heads, w, (cos, sin) if rope else None, 1e-6)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    got = fv.qk_norm_rope_bhsd(dev(proj), col_off, heads, dev(w), (dev(cos), dev(sin)) if rope else None, 1e-6)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert got.shape == want.shape and got.dtype == np.float32
    assert np.abs(got - want).max() <= 2e-6 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("rope", [False, True])
@pytest.mark.parametrize("w16", [False, True])
def test_bf16_kernel_rounding_points(fv, oracle, case, rope, w16):
    import torch

    batch, seq, heads, d, extra, col_off = case
    announce(f"wan_qk_norm_rope16 {case} rope={rope} w16={w16}")
    proj, w, cos, sin = _inputs(8, batch, seq, heads, d, extra, col_off)
    proj = oracle.quantize_bf16(proj)
    if w16:
        w = oracle.quantize_bf16(w)
    want = oracle.wan_qk_norm_rope16(proj, col_off, heads, w, (cos, sin) if rope else None, 1e-6)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    wd = dev(w).to(torch.bfloat16) if w16 else dev(w)
    got = fv.qk_norm_rope_bhsd(dev(proj).to(torch.bfloat16), col_off, heads, wd,
                               (dev(cos), dev(sin)) if rope else None, 1e-6)
    torch.cuda.synchronize()
    assert got.dtype == torch.bfloat16
    got = got.float().cpu().numpy()
    u = _ulps(got, want, oracle)
    assert (u != 0).mean() < 1e-3, f"fraction differing {(u != 0).mean()}"
    if rope:
        assert np.abs(got - want).max() <= 0.03
    else:
        assert u.max() <= 2, f"max ulp {u.max()}"


@pytest.mark.parametrize("case", CASES[1:3])
def test_out_mul_meets_the_values_before_their_one_rounding(fv, oracle, case):
    """`out_mul` (scale * log2(e) for an SDPA call at ln 2): the f32 op's outputs times the factor; the bf16 kernel's
    rotated f32 values times the factor, THEN the one rounding. The expected bf16 values are built here from the
    oracle's un-rotated rows (already bf16 numbers: round_weighted) with numpy's unfused f32 arithmetic; at factor 1
    that construction must be the oracle's own rotated output bit for bit, which pins it. A power-of-two factor
    scales the plain output exactly; 1.0 is the plain output bit for bit."""
    import torch

    batch, seq, heads, d, extra, col_off = case
    announce(f"qk_norm_rope out_mul {case}")
    proj, w, cos, sin = _inputs(18, batch, seq, heads, d, extra, col_off)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    c = np.float32(np.float32(1.0 / np.sqrt(d)) * np.float32(1.4426950408889634))
    # f32 op
    want32 = oracle.qk_norm_rope_bhsd(proj, col_off, heads, w, (cos, sin), 1e-6)
    got32 = fv.qk_norm_rope_bhsd(dev(proj), col_off, heads, dev(w), (dev(cos), dev(sin)), 1e-6, out_mul=float(c))
    plain32 = fv.qk_norm_rope_bhsd(dev(proj), col_off, heads, dev(w), (dev(cos), dev(sin)), 1e-6)
    torch.cuda.synchronize()
    assert torch.equal(got32, plain32 * float(c))               # one f32 multiply of the op's own output
    assert np.abs(got32.cpu().numpy() - want32 * c).max() <= 2e-6 * max(1.0, np.abs(want32).max())
    # bf16 kernel
    p16 = oracle.quantize_bf16(proj)
    n = oracle.wan_qk_norm_rope16(p16, col_off, heads, w, None, 1e-6)          # [b, h, s, d] bf16 numbers
    x1, x2 = n[..., 0::2], n[..., 1::2]
    cv, sv = cos[None, None, :, 0::2], sin[None, None, :, 1::2]

    def expected(f):
        rot = np.empty_like(n)
        rot[..., 0::2] = x1 * cv - x2 * sv                                     # numpy f32: products and sums unfused
        rot[..., 1::2] = x2 * cv + x1 * sv
        return oracle.quantize_bf16(rot * np.float32(f))

    assert np.array_equal(expected(1.0), oracle.wan_qk_norm_rope16(p16, col_off, heads, w, (cos, sin), 1e-6))
    args = (dev(p16).to(torch.bfloat16), col_off, heads, dev(w), (dev(cos), dev(sin)), 1e-6)
    plain = fv.qk_norm_rope_bhsd(*args)
    assert torch.equal(fv.qk_norm_rope_bhsd(*args, out_mul=1.0), plain)
    assert torch.equal(fv.qk_norm_rope_bhsd(*args, out_mul=0.25).float(), plain.float() * 0.25)
    got = fv.qk_norm_rope_bhsd(*args, out_mul=float(c)).float().cpu().numpy()
    want = expected(c)
    u = _ulps(got, want, oracle)
    assert (u != 0).mean() < 1e-3, f"fraction differing {(u != 0).mean()}"
    assert np.abs(got - want).max() <= 0.03 * float(c)
    # and it is NOT the twice-rounded value for a visible share of the elements (the test can tell the two apart)
    twice = oracle.quantize_bf16(plain.float().cpu().numpy() * c)
    assert (_ulps(want, twice, oracle) != 0).mean() > 0.05
    with pytest.raises(fv.FvError):
        fv.qk_norm_rope_bhsd(*args, out_mul=float("nan"))


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_split_and_merge_heads_bit_exact(fv, oracle, dtype):
    import torch

    announce(f"split/merge heads {dtype}")
    rng = np.random.Generator(np.random.PCG64(9))
    batch, seq, heads, d, col_off = 2, 77, 12, 128, 1536 * 2
    proj = rng.standard_normal((batch, seq, 3 * heads * d)).astype(np.float32)
    if dtype == "bf16":
        proj = oracle.quantize_bf16(proj)
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float32
    pd = torch.from_numpy(proj).cuda().to(tdt)
    sp = fv.split_heads_bhsd(pd, col_off, heads, d)
    mg = fv.merge_heads(sp)
    torch.cuda.synchronize()
    want_sp = oracle.split_heads_bhsd(proj, col_off, heads, d)
    assert np.array_equal(sp.float().cpu().numpy(), want_sp)
    assert np.array_equal(mg.float().cpu().numpy(), oracle.merge_heads(want_sp))
    assert np.array_equal(mg.float().cpu().numpy(), proj[:, :, col_off:col_off + heads * d])


def test_declines_and_errors(fv):
    import torch

    x = torch.zeros((1, 2, 36), device="cuda")
    w = torch.ones(12, device="cuda")
    with pytest.raises(fv.FvDeclined):
        fv.qk_norm_rope_bhsd(x, 0, 3, w)          # d = 4: not a multiple of 8
    with pytest.raises(ValueError):
        fv.qk_norm_rope_bhsd(x, 30, 3, w)         # columns outside the projection


def test_producer_feeds_the_attention_kernel(fv, oracle):
    """q/k prepared by the bf16 kernel + split V go straight into the dense kernel, and
    merge_heads brings the result back to [batch, seq, heads*d]."""
    import torch

    announce("qk prep -> sdpa -> merge, 1x300x4x128")
    batch, seq, heads, d = 1, 300, 4, 128
    proj, w, cos, sin = _inputs(10, batch, seq, heads, d, 0, 0)
    rng = np.random.Generator(np.random.PCG64(11))
    qkv = oracle.quantize_bf16(rng.standard_normal((batch, seq, 3 * heads * d)).astype(np.float32))
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    x = dev(qkv).to(torch.bfloat16)
    rope = (dev(cos), dev(sin))
    q = fv.qk_norm_rope_bhsd(x, 0, heads, dev(w), rope)
    k = fv.qk_norm_rope_bhsd(x, heads * d, heads, dev(w), rope)
    v = fv.split_heads_bhsd(x, 2 * heads * d, heads, d)
    o = fv.sdpa_dense_bf16(q.reshape(heads, seq, d), k.reshape(heads, seq, d), v.reshape(heads, seq, d),
                           out_bf16=True)
    merged = fv.merge_heads(o.reshape(batch, heads, seq, d))
    torch.cuda.synchronize()
    want = oracle.sdpa_composed(q.float().cpu().numpy().reshape(heads, seq, d),
                                k.float().cpu().numpy().reshape(heads, seq, d),
                                v.float().cpu().numpy().reshape(heads, seq, d))
    want = oracle.merge_heads(want.reshape(batch, heads, seq, d))
    got = merged.float().cpu().numpy()
    assert got.shape == (batch, seq, heads * d)
    assert np.abs(got - want).max() <= 1e-2


@pytest.mark.parametrize("grid", [(2, 3, 5), (5, 6, 9), (4, 4, 4)])
@pytest.mark.parametrize("out16", [False, True])
def test_tile_ordered_producers_are_the_bhsd_ones_permuted(fv, oracle, grid, out16):
    """qk_norm_rope / split_heads writing VSA's tile-slot order: row token_slot[s] of the padded
    plane holds exactly what row s of the BHSD plane holds, padding rows stay zero."""
    import torch

    ctx = fv.VsaCtx(grid, 0.8)
    batch, heads, d = 2, 3, 128
    announce(f"tile-ordered producers grid={grid} out16={out16}")
    proj, w, cos, sin = _inputs(900 + ctx.seq, batch, ctx.seq, heads, d, 8, 2 * heads * d)
    dt = torch.bfloat16 if out16 else torch.float32
    tp = torch.from_numpy(proj).cuda().to(dt)
    tw = torch.from_numpy(w).cuda().to(dt)
    rope = (torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda())
    col = 2 * heads * d
    slot = torch.from_numpy(ctx.plan.token_slot.astype(np.int64)).cuda()
    pad = torch.from_numpy(ctx.plan.slot_src < 0).cuda()
    for r in (None, rope):
        want = fv.qk_norm_rope_bhsd(tp, col, heads, tw, r, out_bf16=out16)
        got = fv.qk_norm_rope_tiles(tp, col, heads, tw, ctx, r, out_bf16=out16)
        torch.cuda.synchronize()
        assert tuple(got.shape) == (batch, heads, ctx.padded, d) and got.dtype == want.dtype
        assert torch.equal(got[:, :, slot], want)
        assert not got[:, :, pad].any()
    want = fv.split_heads_bhsd(tp, col, heads, d)
    got = fv.split_heads_tiles(tp, col, heads, d, ctx)
    torch.cuda.synchronize()
    assert torch.equal(got[:, :, slot], want) and not got[:, :, pad].any()
    # and against the oracle's own tile permute of the oracle's BHSD result (bf16 permute is exact)
    if out16:
        ref = oracle.split_heads_bhsd(oracle.quantize_bf16(proj), col, heads, d)
        tiles = np.zeros((batch, heads, ctx.padded, d), np.float32)
        tiles[:, :, ctx.plan.token_slot] = ref
        assert np.array_equal(got.float().cpu().numpy(), tiles)
