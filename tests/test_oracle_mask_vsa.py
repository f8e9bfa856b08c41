"""Pins for the oracle's BlockCausal, tiling, top-k and VSA host path: the
reference's own unit-test known answers (C/rt/attn.rs:883-930,
M/wan/family.rs:146-191, C/rt/vsa.rs:480-696, C/rt/sp.rs:66-84) plus brute
force on small inputs.
"""
import numpy as np
import pytest

SF_PATCH = (1, 2, 2)  # WanVideoArchConfig::sf_wan_t2v_1_3b: patch (1,2,2), 3 frames per block, global


# ---- BlockCausal ------------------------------------------------------------------

@pytest.mark.parametrize("window,fpb", [(-1, 3), (3, 3), (6, 3), (-1, 1), (1, 1), (2, 1)])
def test_block_causal_is_the_models_temporal_mask(oracle, window, fpb):
    # C/rt/attn.rs:883-896
    frames, h, w = 9, 6, 4
    want = oracle.causal_temporal_mask(SF_PATCH, fpb, window, frames, h, w)
    spec = oracle.block_causal_for(fpb, window, (h // 2) * (w // 2))
    assert spec is not None
    seq = frames * (h // 2) * (w // 2)
    assert np.array_equal(oracle.block_causal_dense_mask(*spec, seq, seq), want)


def test_partial_block_windows_have_no_block_causal(oracle):
    # C/rt/attn.rs:897-902: 4 frames is not whole 3-frame blocks
    assert oracle.block_causal_for(3, 4, 6) is None
    assert oracle.block_causal_for(3, -1, 1560) == (4680, 0, 0)
    assert oracle.block_causal_for(1, -1, 1560) == (1560, 0, 0)
    assert oracle.block_causal_for(3, 6, 10) == (30, 2, 0)


def test_causal_mask_blocks_future_blocks(oracle):
    # M/wan/family.rs:146-161
    frames, h, w = 4, 4, 4
    mask = oracle.causal_temporal_mask(SF_PATCH, 3, -1, frames, h, w)
    hw = (h // 2) * (w // 2)
    seq = frames * hw
    assert mask.shape == (seq, seq)
    flat = mask.reshape(-1)
    assert flat[2 * hw] == 0.0
    assert flat[3 * hw] < -1e8
    assert flat[3 * hw * seq] == 0.0


def test_token_window_from_the_block_end(oracle):
    # M/wan/family.rs:163-190
    mask = oracle.causal_temporal_mask(SF_PATCH, 3, 4, 9, 4, 4).reshape(-1)
    hw, seq = 4, 36
    q = 6 * hw
    assert mask[q * seq + 5 * hw] == 0.0
    assert mask[q * seq + 5 * hw - 1] < -1e8
    assert mask[q * seq] < -1e8
    assert mask[q * seq + 8 * hw] == 0.0
    mask = oracle.causal_temporal_mask(SF_PATCH, 3, 1, 3, 4, 4).reshape(-1)
    assert mask[0] == 0.0
    assert mask[1] < -1e8


def test_allows_closed_form(oracle):
    # brute-force restatement of the predicate in python ints
    for bt, win, sink in [(5, 2, 1), (1, 0, 0), (7, 0, 2), (4, 1, 0), (0, 0, 0)]:
        b = max(bt, 1)
        for q in range(0, 40, 3):
            for k in range(40):
                tq, tk = q // b, k // b
                want = (tk <= tq and (win == 0 or tq - tk < win)) or tk < sink
                assert oracle.block_causal_allows(bt, win, sink, q, k) == want
    m = oracle.block_causal_dense_mask(5, 2, 1, 24, 24)
    assert set(np.unique(m)) == {np.float32(-1e9), np.float32(0.0)}
    assert m[0, 4] == 0 and m[0, 5] < 0 and m[23, 0] == 0 and m[23, 5] < 0 and m[23, 10] < 0 and m[23, 15] == 0


def test_visible_fraction_of_the_headline_causal_shape(oracle):
    # 21 frame blocks: 231 of 441 block pairs are visible
    vis = sum(oracle.block_causal_allows(1560, 0, 0, q * 1560, k * 1560) for q in range(21) for k in range(21))
    assert vis == 231
    vis3 = sum(oracle.block_causal_allows(4680, 0, 0, q * 4680, k * 4680) for q in range(7) for k in range(7))
    assert vis3 == 28


# ---- tiling / top-k rule ----------------------------------------------------------

@pytest.mark.parametrize("grid", [(4, 4, 4), (33, 28, 52), (3, 5, 7), (1, 1, 1)])
def test_tiling_is_a_permutation_with_padding(oracle, grid):
    p = oracle.TilePlan(grid)
    assert p.seq == grid[0] * grid[1] * grid[2]
    assert p.padded == p.num_tiles * 64
    real = p.slot_src >= 0
    toks = p.slot_src[real]
    assert np.array_equal(np.sort(toks), np.arange(p.seq))
    assert np.array_equal(p.token_slot[toks], np.nonzero(real)[0])
    assert p.block_sizes.sum() == p.seq and p.block_sizes.max() <= 64


def test_tile_plan_known_answers(oracle):
    p = oracle.TilePlan((8, 8, 8))
    assert (p.slot_src >= 0).all() and (p.block_sizes == 64).all()
    p = oracle.TilePlan((1, 1, 5))
    assert p.num_tiles == 2 and list(p.block_sizes) == [4, 1]
    assert list(p.slot_src[:4]) == [0, 1, 2, 3]
    assert (p.slot_src[4:64] == -1).all() and p.slot_src[64] == 4
    p = oracle.TilePlan((21, 30, 52))
    assert p.tiles == (6, 8, 13) and p.num_tiles == 624 and p.padded == 39936
    assert oracle.topk_for(0.8, 624) == 125
    # row-major sub-cube order inside a full tile: slot (z*4+y)*4+x of tile 0
    p = oracle.TilePlan((4, 8, 8))
    assert p.slot_src[1] == 1 and p.slot_src[4] == 8 and p.slot_src[16] == 64 and p.slot_src[64] == 4
    with pytest.raises(ValueError):
        oracle.TilePlan((0, 4, 4))


def test_topk_matches_upstream_rule(oracle):
    assert oracle.topk_for(0.8, 819) == 164
    assert oracle.topk_for(0.0, 819) == 819
    assert oracle.topk_for(1.0, 819) == 1
    assert oracle.topk_for(0.9, 10) == 1
    assert oracle.topk_for(0.875, 512) == 64


def test_shard_ranges(oracle):
    assert oracle.shard_ranges(10, 2) == [(0, 5), (5, 5)]
    assert oracle.shard_ranges(11, 2) == [(0, 6), (6, 5)]
    assert sum(l for _, l in oracle.shard_ranges(32760, 8)) == 32760


# ---- top-k ------------------------------------------------------------------------------

def test_sortable_orders_like_floats(oracle):
    xs = [-np.inf, -3.5, -1e-30, -0.0, 0.0, 1e-30, 2.0, np.inf]
    keys = [oracle.sortable(np.float32(x)) for x in xs]
    assert keys == sorted(keys) and len(set(keys)) == len(keys)


def total_key(x):
    # IEEE total order on non-NaN values: -0.0 sorts just below +0.0
    return (float(x), 0 if np.signbit(x) else 1)


def brute_topk_sets(scores, k):
    out = []
    for row in scores:
        order = sorted(range(len(row)), key=lambda i: (tuple(-c for c in total_key(row[i])), i))
        out.append(order[:k])
    return out


@pytest.mark.parametrize("tied", [False, True])
def test_topk_orders_against_brute_force(oracle, tied):
    rng = np.random.default_rng(11)
    s = rng.standard_normal((13, 97)).astype(np.float32)
    if tied:
        s = (np.round(s * 8) / 8).astype(np.float32)  # heavy ties, as G/kernels/attn3.rs:664-696
        assert np.signbit(s[s == 0]).any() and not np.signbit(s[s == 0]).all()
    for k in (1, 7, 50, 97):
        want = brute_topk_sets(s, k)
        host = oracle.topk_host_order(s, k)
        dev = oracle.topk_device_order(s, k)
        for r in range(s.shape[0]):
            assert list(host[r]) == want[r]
            assert sorted(dev[r]) == sorted(want[r])
            thr = total_key(s[r][want[r][-1]])
            above = [i for i in range(97) if total_key(s[r][i]) > thr]
            equal = [i for i in range(97) if total_key(s[r][i]) == thr]
            assert list(dev[r]) == (above + equal)[:k]


def test_topk_device_order_k_above_n_pads_with_zero(oracle):
    s = np.array([[0.5, -1.0, 2.0]], dtype=np.float32)
    assert list(oracle.topk_device_order(s, 5)[0]) == [0, 1, 2, 0, 0]
    # -0.0 sorts below +0.0 (total order on bits)
    z = np.array([[0.0, -0.0, 0.0, -0.0]], dtype=np.float32)
    assert list(oracle.topk_device_order(z, 2)[0]) == [0, 2]
    assert list(oracle.topk_host_order(z, 3)[0]) == [0, 2, 1]


# ---- tile mean / coarse scores ---------------------------------------------------------

def test_tile_mean_closed_forms(oracle):
    p = oracle.TilePlan((3, 5, 7))
    x = np.full((2, p.seq, 8), 1.25, dtype=np.float32)
    assert np.array_equal(oracle.vsa_tile_mean(x, p), np.full((2, p.num_tiles, 8), 1.25, np.float32))
    # value = token index: mean is the mean of the tile's token ids
    x = np.broadcast_to(np.arange(p.seq, dtype=np.float32)[None, :, None], (1, p.seq, 4)).copy()
    got = oracle.vsa_tile_mean(x, p)
    for tile in range(p.num_tiles):
        n = p.block_sizes[tile]
        toks = p.slot_src[tile * 64: tile * 64 + n]
        assert np.allclose(got[0, tile], toks.mean(), rtol=1e-6)
    # round16 pools bf16-rounded values
    x = np.full((1, p.seq, 4), 1.0 + 2.0**-9, dtype=np.float32)
    assert np.array_equal(oracle.vsa_tile_mean(x, p, round16=True), np.ones((1, p.num_tiles, 4), np.float32))


def test_combine_forms(oracle):
    """kernels/core.cu:803-835: f32 form = numpy's multiply then add; the round16 form is torch's
    own bf16 arithmetic (each bf16 op computes in f32 and rounds once), bf16(bf16(sparse) +
    bf16(bf16(coarse) * bf16(gate))); padding slots and rows outside the tile range are untouched."""
    import torch

    p = oracle.TilePlan((3, 5, 7))
    rng = np.random.default_rng(12)
    bh, dim, nb = 2, 16, p.num_tiles
    sparse = rng.standard_normal((bh, p.padded, dim)).astype(np.float32)
    coarse = rng.standard_normal((bh, nb, dim)).astype(np.float32)
    gate = rng.standard_normal((bh, p.seq, dim)).astype(np.float32)
    real = p.slot_src >= 0
    tok, tile = p.slot_src[real], (np.arange(p.padded) // 64)[real]
    # f32
    want = np.zeros((bh, p.seq, dim), np.float32)
    want[:, tok] = (coarse[:, tile] * gate[:, tok]).astype(np.float32) + sparse[:, real]
    assert np.array_equal(oracle.vsa_combine(sparse, coarse, gate, p, p.seq), want)
    want[:, tok] = coarse[:, tile] + sparse[:, real]
    assert np.array_equal(oracle.vsa_combine(sparse, coarse, None, p, p.seq), want)
    # round16 against torch bf16 tensors
    b16 = lambda x: torch.from_numpy(x).to(torch.bfloat16)
    t = b16(sparse[:, real]) + b16(coarse[:, tile]) * b16(gate[:, tok])
    want = np.zeros((bh, p.seq, dim), np.float32)
    want[:, tok] = t.float().numpy()
    got = oracle.vsa_combine(sparse, coarse, gate, p, p.seq, round16=True)
    assert np.array_equal(got, want)
    assert not np.array_equal(got, oracle.vsa_combine(sparse, coarse, gate, p, p.seq))
    t = b16(sparse[:, real]) + b16(coarse[:, tile])
    want[:, tok] = t.float().numpy()
    assert np.array_equal(oracle.vsa_combine(sparse, coarse, None, p, p.seq, round16=True), want)
    # zero gate: bf16(sparse)
    z = oracle.vsa_combine(sparse, coarse, np.zeros_like(gate), p, p.seq, round16=True)
    assert np.array_equal(z[:, tok], oracle.quantize_bf16(sparse[:, real]))
    # a tile range writes only its tokens
    out = np.full((bh, p.seq, dim), 7.0, np.float32)
    oracle.vsa_combine(sparse[:, 64:192], coarse, gate, p, p.seq, q_base=1, q_tiles=2, out=out)
    inside = np.zeros(p.seq, bool)
    inside[p.slot_src[64:192][p.slot_src[64:192] >= 0]] = True
    assert np.all(out[:, ~inside] == 7.0) and np.all(out[:, inside] != 7.0)


def test_coarse_scores_are_the_sequential_f64_dot(oracle):
    # C/rt/vsa.rs:185-189: f64 products summed in ascending d, times f64(scale), one rounding to f32
    rng = np.random.default_rng(3)
    qc = rng.standard_normal((2, 9, 128)).astype(np.float32)
    kc = rng.standard_normal((2, 9, 128)).astype(np.float32)
    scale = np.float32(0.25 / 3)
    got = oracle.vsa_coarse_scores(qc, kc, scale)
    prod = qc.astype(np.float64)[:, :, None, :] * kc.astype(np.float64)[:, None, :, :]
    dot = np.cumsum(prod, axis=-1)[..., -1]          # cumsum adds strictly left to right
    want = (dot * np.float64(scale)).astype(np.float32)
    assert np.array_equal(got, want)
    # an f32 accumulation of the same products differs in some last bits: the test can tell the two apart
    f32 = np.zeros((2, 9, 9), np.float32)
    for d in range(128):
        f32 = f32 + qc[:, :, None, d] * kc[:, None, :, d]
    assert np.any(f32 * scale != got)


def test_coarse_scores_zero_signs(oracle):
    # the sum starts from -0.0 (Rust's f64 Sum identity): products that are all -0.0 give -0.0,
    # any +0.0 among them gives +0.0
    qc = np.zeros((1, 2, 4), np.float32)
    kc = np.array([[[1, 2, 3, 4], [-1, -2, -3, -4]]], np.float32)
    got = oracle.vsa_coarse_scores(qc, kc, 0.5)
    assert np.all(got == 0) and not np.signbit(got[0, 0, 0]) and np.signbit(got[0, 0, 1])
    kc[0, 1, 2] = 3.0
    assert not np.signbit(oracle.vsa_coarse_scores(qc, kc, 0.5)[0, 0, 1])


def test_coarse_scores_are_what_the_host_oracle_selects_from(oracle):
    # stage 3 of vsa_attention_host sorts exactly these scores (C/rt/vsa.rs:203-212)
    plan = oracle.TilePlan((5, 6, 7))
    rng = np.random.default_rng(8)
    q, k, v = (rng.standard_normal((2, plan.seq, 16)).astype(np.float32) for _ in range(3))
    scale = 0.25
    topk = 3
    _, sel = oracle.vsa_attention_host(q, k, v, None, plan, topk, 1, 2, 16, scale, return_selected=True)
    sc = oracle.vsa_coarse_scores(oracle.vsa_tile_mean(q, plan), oracle.vsa_tile_mean(k, plan), scale)
    assert np.array_equal(sel.reshape(-1, topk), oracle.topk_host_order(sc, topk))


# ---- VSA host oracle -----------------------------------------------------------------------

def lcg(seed, n, inc=1442695040888963407):
    s = seed
    out = np.empty(n, dtype=np.float32)
    for i in range(n):
        s = (s * 6364136223846793005 + inc) & 0xFFFFFFFFFFFFFFFF
        out[i] = np.float32(np.float32(s >> 33) / np.float32(1 << 31)) - np.float32(0.5)
    return out


def test_all_tiles_selected_and_zero_gate_is_dense_attention(oracle):
    # C/rt/vsa.rs:534-597
    b, heads, dim = 1, 2, 8
    plan = oracle.TilePlan((2, 3, 5))
    seq = plan.seq
    n = b * heads * seq * dim
    q, k, v = lcg(1, n), lcg(2, n), lcg(3, n)
    gate = np.zeros(n, dtype=np.float32)
    scale = np.float32(1.0) / np.sqrt(np.float32(dim))
    got = oracle.vsa_attention_host(q, k, v, gate, plan, plan.num_tiles, b, heads, dim, scale)
    qq, kk, vv = (x.reshape(heads, seq, dim).astype(np.float64) for x in (q, k, v))
    s = np.einsum("hqd,hkd->hqk", qq, kk) * float(scale)
    p = np.exp(s - s.max(-1, keepdims=True))
    want = np.einsum("hqk,hkd->hqd", p / p.sum(-1, keepdims=True), vv)
    assert np.abs(got - want).max() < 2e-5


def test_gate_adds_the_coarse_branch(oracle):
    # C/rt/vsa.rs:601-656
    b, heads, dim = 1, 1, 4
    plan = oracle.TilePlan((1, 4, 4))
    n = plan.seq * dim
    i = np.arange(n)
    q = ((i % 7) * 0.1 - 0.3).astype(np.float32)
    k = ((i % 5) * 0.2 - 0.4).astype(np.float32)
    v = ((i % 3) * 0.3 - 0.3).astype(np.float32)
    scale = np.float32(0.5)
    nb = plan.num_tiles
    zero = oracle.vsa_attention_host(q, k, v, np.zeros(n, np.float32), plan, nb, b, heads, dim, scale)
    one = oracle.vsa_attention_host(q, k, v, np.ones(n, np.float32), plan, nb, b, heads, dim, scale)
    none = oracle.vsa_attention_host(q, k, v, None, plan, nb, b, heads, dim, scale)
    assert np.abs(one - none).max() < 1e-6
    assert np.abs(one - zero).max() > 1e-4
    # one - zero is the coarse branch: with a single tile it is the mean value row
    assert np.abs((one - zero) - v.reshape(plan.seq, dim).mean(0)).max() < 1e-6


def test_fewer_tiles_changes_the_result_but_stays_finite(oracle):
    # C/rt/vsa.rs:659-695
    b, heads, dim = 1, 1, 8
    plan = oracle.TilePlan((4, 8, 8))
    n = plan.seq * dim
    r = lcg(99, 3 * n, inc=1)
    q, k, v = r[:n], r[n:2 * n], r[2 * n:]
    scale = np.float32(1.0) / np.sqrt(np.float32(dim))
    nb = plan.num_tiles
    sparse, sel = oracle.vsa_attention_host(q, k, v, None, plan, oracle.topk_for(0.8, nb), b, heads, dim, scale,
                                            return_selected=True)
    dense = oracle.vsa_attention_host(q, k, v, None, plan, nb, b, heads, dim, scale)
    assert np.isfinite(sparse).all() and np.isfinite(dense).all()
    assert np.abs(sparse - dense).max() > 1e-6
    assert sel.shape == (1, nb, oracle.topk_for(0.8, nb))
    assert all(len(set(row)) == len(row) for row in sel[0])


def test_vsa_rejects_wrong_sizes(oracle):
    plan = oracle.TilePlan((1, 4, 4))
    x = np.zeros(plan.seq * 4, np.float32)
    with pytest.raises(ValueError, match="want"):
        oracle.vsa_attention_host(x[:-1], x, x, None, plan, 1, 1, 1, 4, 0.5)
    with pytest.raises(ValueError, match="gate"):
        oracle.vsa_attention_host(x, x, x, x[:-1], plan, 1, 1, 1, 4, 0.5)


def test_vsa_partial_tiles_ignore_padding(oracle):
    # padded slots never enter means or the fine stage: compare with a brute-force
    # f64 block-sparse attention over token sets on a grid with partial tiles
    rng = np.random.default_rng(5)
    plan = oracle.TilePlan((2, 5, 6))
    dim, nb = 16, plan.num_tiles
    q, k, v = (rng.standard_normal((1, plan.seq, dim)).astype(np.float32) for _ in range(3))
    topk = 2
    scale = np.float32(0.25)
    out, sel = oracle.vsa_attention_host(q, k, v, np.zeros_like(q), plan, topk, 1, 1, dim, scale, return_selected=True)
    toks = [plan.slot_src[t * 64: t * 64 + plan.block_sizes[t]] for t in range(nb)]
    for qt in range(nb):
        keys = np.concatenate([toks[kt] for kt in sel[0, qt]])
        for qi in toks[qt]:
            s = (q[0, qi].astype(np.float64) @ k[0, keys].astype(np.float64).T) * float(scale)
            p = np.exp(s - s.max())
            want = (p / p.sum()) @ v[0, keys].astype(np.float64)
            assert np.abs(out[0, qi] - want).max() < 2e-5
