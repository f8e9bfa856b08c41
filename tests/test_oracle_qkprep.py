"""Oracle pins for the producer / consumer either side of the SDPA call: q/k RMSNorm
(+ RoPE) into BHSD in both of the reference's forms, split_heads_bhsd, merge_heads.

Pinned by the reference's own host test (wan/fuse.rs:627-663: the bf16 twin against the
f32 op within 0.03 on closed-form inputs) and by what the mathematics fixes: a hand
computation without RoPE, unit RMS for w == 1, a rotation keeps each pair's norm, a zero
angle is no rotation, index formulas by brute force, merge(split(x)) == x.
"""
import numpy as np


def vals(n, k):
    # wan/fuse.rs:575-577
    i = np.arange(n, dtype=np.float32)
    return (np.sin(i * np.float32(k)) * np.float32(1.3) + np.float32(0.1)).astype(np.float32)


def test_reference_host_case_bf16_twin_vs_f32_op(oracle):
    # wan/fuse.rs:627-663, same shapes, closed-form inputs and bound
    b, s, heads, d = 1, 4, 2, 4
    width = heads * d
    x = oracle.quantize_bf16(vals(b * s * 3 * width, 0.37)).reshape(b, s, 3 * width)
    w = (1.0 + 0.1 * vals(width, 0.9)).astype(np.float32)
    ang = vals(s * d, 2.1)
    cos, sin = np.cos(ang).reshape(s, d).astype(np.float32), np.sin(ang).reshape(s, d).astype(np.float32)
    got = oracle.wan_qk_norm_rope16(x, width, heads, w, (cos, sin), 1e-6)
    want = oracle.qk_norm_rope_bhsd(x, width, heads, w, (cos, sin), 1e-6)
    assert got.shape == want.shape == (b, heads, s, d)
    assert np.abs(got - want).max() <= 0.03
    assert np.array_equal(got, oracle.quantize_bf16(got))   # bf16 values
    assert np.abs(got - want).max() > 0                      # and the roundings are really there


def test_no_rope_is_x_inv_w_by_hand(oracle):
    rng = np.random.Generator(np.random.PCG64(3))
    b, s, heads, d, off = 2, 3, 3, 4, 5
    width = heads * d
    proj = rng.standard_normal((b, s, off + width + 2)).astype(np.float32)
    w = rng.standard_normal(width).astype(np.float32)
    got = oracle.qk_norm_rope_bhsd(proj, off, heads, w, None, 1e-5)
    for bi in range(b):
        for si in range(s):
            x = proj[bi, si, off:off + width].astype(np.float64)
            inv = 1.0 / np.sqrt((x * x).mean() + 1e-5)
            want = (x * inv * w).reshape(heads, d)
            assert np.allclose(got[bi, :, si, :], want, rtol=2e-6, atol=2e-6)
    # a transposed output (BSHD instead of BHSD) would fail the indexing above; a norm
    # per head instead of across heads fails this:
    one = oracle.qk_norm_rope_bhsd(proj, off, heads, np.ones(width, np.float32), None, 0.0)
    rms = np.sqrt((one.astype(np.float64) ** 2).sum(axis=(1, 3)) / width)
    assert np.allclose(rms, 1.0, atol=1e-5)
    per_head = np.sqrt((one.astype(np.float64) ** 2).mean(axis=3))
    assert np.abs(per_head - 1.0).max() > 1e-2


def test_rope_is_a_rotation_of_interleaved_pairs(oracle):
    rng = np.random.Generator(np.random.PCG64(4))
    b, s, heads, d = 1, 5, 2, 8
    width = heads * d
    proj = rng.standard_normal((b, s, width)).astype(np.float32)
    w = rng.standard_normal(width).astype(np.float32)
    theta = rng.uniform(-3, 3, (s, d // 2))
    # Wan layout: both slots of a pair hold the pair's angle; the op reads cos from the
    # even slot and sin from the odd slot: poison the other two so a swap shows
    cos = np.repeat(np.cos(theta), 2, axis=1).astype(np.float32)
    sin = np.repeat(np.sin(theta), 2, axis=1).astype(np.float32)
    cos_p, sin_p = cos.copy(), sin.copy()
    cos_p[:, 1::2] = 77.0
    sin_p[:, 0::2] = -55.0
    plain = oracle.qk_norm_rope_bhsd(proj, 0, heads, w, None, 1e-6).astype(np.float64)
    rot = oracle.qk_norm_rope_bhsd(proj, 0, heads, w, (cos_p, sin_p), 1e-6).astype(np.float64)
    x1, x2 = plain[..., 0::2], plain[..., 1::2]
    c, sn = np.cos(theta)[None, None], np.sin(theta)[None, None]
    assert np.allclose(rot[..., 0::2], x1 * c - x2 * sn, atol=1e-5)
    assert np.allclose(rot[..., 1::2], x1 * sn + x2 * c, atol=1e-5)
    assert np.allclose(rot[..., 0::2] ** 2 + rot[..., 1::2] ** 2, x1 ** 2 + x2 ** 2, atol=1e-4)
    zero = oracle.qk_norm_rope_bhsd(proj, 0, heads, w, (np.ones((s, d), np.float32), np.zeros((s, d), np.float32)), 1e-6)
    assert np.array_equal(zero, plain.astype(np.float32))


def test_bf16_twin_rounding_points(oracle):
    rng = np.random.Generator(np.random.PCG64(5))
    b, s, heads, d = 1, 3, 2, 4
    width = heads * d
    proj = oracle.quantize_bf16(rng.standard_normal((b, s, width)).astype(np.float32))
    w = rng.standard_normal(width).astype(np.float32)
    got = oracle.wan_qk_norm_rope16(proj, 0, heads, w, None, 1e-6)
    q = oracle.quantize_bf16
    for si in range(s):
        x = proj[0, si]
        ss = np.float32(0)
        for v in x:
            ss = np.float32(ss + np.float32(v * v))
        inv = np.float32(1.0) / np.sqrt(np.float32(ss / np.float32(width) + np.float32(1e-6)), dtype=np.float32)
        want = q(q((x * inv).astype(np.float32)) * w).reshape(heads, d)
        assert np.array_equal(got[0, :, si, :], want)
    ang = rng.uniform(-3, 3, (s, d)).astype(np.float32)
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    rot = oracle.wan_qk_norm_rope16(proj, 0, heads, w, (cos, sin), 1e-6)
    n = got  # the rounded, weighted values the rotation starts from
    x1, x2 = n[..., 0::2], n[..., 1::2]
    c, sn = cos[None, None, :, 0::2], sin[None, None, :, 1::2]
    assert np.array_equal(rot[..., 0::2], q((x1 * c - x2 * sn).astype(np.float32)))
    assert np.array_equal(rot[..., 1::2], q((x2 * c + x1 * sn).astype(np.float32)))


def test_split_and_merge_heads_index_formulas(oracle):
    rng = np.random.Generator(np.random.PCG64(6))
    b, s, heads, d, off = 2, 5, 3, 4, 7
    proj = rng.standard_normal((b, s, off + heads * d + 3)).astype(np.float32)
    sp = oracle.split_heads_bhsd(proj, off, heads, d)
    for bi in range(b):
        for h in range(heads):
            for si in range(s):
                assert np.array_equal(sp[bi, h, si], proj[bi, si, off + h * d: off + (h + 1) * d])
    mg = oracle.merge_heads(sp)
    assert mg.shape == (b, s, heads * d)
    assert np.array_equal(mg, proj[:, :, off:off + heads * d])
    assert np.array_equal(oracle.merge_heads(sp), sp.transpose(0, 2, 1, 3).reshape(b, s, heads * d))
