"""Parity of the VSA stages and the whole VSA op (through the C ABI) against
the CPU oracle. Grids and limits follow the reference's vsa / vsa_stages groups
(crates/fastvideo-gpucheck/src/kernels.rs:1577-1816, kernels/attn3.rs:475-766):
whole op rel_l2 <= 2e-2 vs the host oracle (here also max|delta| <= 1e-2), tile
mean exact, top-k bit-exact incl. heavily tied rows, block index lists bit-exact.
"""
import numpy as np
import pytest

from util import announce, assert_parity, metrics, randn

pytestmark = pytest.mark.gpu

GRIDS = [(4, 4, 4), (2, 3, 5), (5, 6, 9), (9, 8, 13)]
D = 128


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


def vsa_inputs(oracle, seed, bh, seq, gate=True):
    q, k, v = (oracle.quantize_bf16(randn(seed + i, (bh, seq, D))) for i in range(3))
    g = oracle.quantize_bf16(randn(seed + 3, (bh, seq, D), 0.5)) if gate else None
    return q, k, v, g


def brute_block_sparse(q, k, v, sel, plan, scale):
    """f64 attention of every real query over the real tokens of its selected tiles."""
    bh, seq, d = q.shape
    out = np.zeros((bh, seq, d))
    toks = [plan.slot_src[t * 64: t * 64 + plan.block_sizes[t]] for t in range(plan.num_tiles)]
    for b in range(bh):
        q64, k64, v64 = (x[b].astype(np.float64) for x in (q, k, v))
        for qt in range(plan.num_tiles):
            keys = np.concatenate([toks[int(kt)] for kt in sel[b, qt]])
            s = (q64[toks[qt]] @ k64[keys].T) * scale
            p = np.exp(s - s.max(-1, keepdims=True))
            out[b, toks[qt]] = (p / p.sum(-1, keepdims=True)) @ v64[keys]
    return out


@pytest.mark.parametrize("grid", GRIDS)
def test_tile_mean_is_exact(fv, oracle, grid):
    import torch

    announce(f"vsa tile_mean grid={grid}")
    ctx = fv.VsaCtx(grid, 0.8)
    oplan = oracle.TilePlan(grid)
    x = randn(11, (3, ctx.seq, D))
    got = fv.vsa_tile_mean(dev(x), ctx)
    got16 = fv.vsa_tile_mean(dev(x), ctx, round16=True)
    gotb = fv.vsa_tile_mean(dev(x).to(torch.bfloat16), ctx)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), oracle.vsa_tile_mean(x, oplan))
    want16 = oracle.vsa_tile_mean(x, oplan, round16=True)
    assert np.array_equal(got16.cpu().numpy(), want16)
    assert np.array_equal(gotb.cpu().numpy(), want16)


@pytest.mark.parametrize("nb", [1, 17, 64, 150, 624])
def test_coarse_scores_bit_exact_and_coarse_output(fv, oracle, nb):
    import torch

    announce(f"vsa coarse nb={nb}")
    bh = 3
    qc, kc, vc = (randn(21 + i, (bh, nb, D), 0.3) for i in range(3))
    scale = np.float32(1.0 / np.sqrt(D))
    scores, coarse = fv.vsa_coarse(dev(qc), dev(kc), dev(vc), float(scale))
    torch.cuda.synchronize()
    want_s = oracle.vsa_coarse_scores(qc, kc, scale)
    assert np.array_equal(scores.cpu().numpy(), want_s)
    s64 = want_s.astype(np.float64)
    p = np.exp(s64 - s64.max(-1, keepdims=True))
    want_c = (p / p.sum(-1, keepdims=True)) @ vc.astype(np.float64)
    assert np.abs(coarse.cpu().numpy() - want_c).max() < 1e-5


@pytest.mark.parametrize("rows,n,k,tied", [(7, 1, 1, False), (13, 97, 7, False), (13, 97, 50, True), (5, 624, 125, False),
                                           (5, 624, 125, True), (3, 4096, 819, True), (4, 512, 64, False),
                                           (2, 300, 300, True), (2, 10, 16, False), (3, 257, 1, True),
                                           # one case per keys-per-lane instantiation boundary (256 .. 4096 wide rows)
                                           (3, 256, 33, True), (3, 700, 140, True), (3, 768, 1, False), (2, 1025, 512, True),
                                           (2, 1536, 300, False), (2, 2049, 2049, True), (2, 3072, 7, True), (2, 3073, 600, False)])
def test_topk_bit_exact(fv, oracle, rows, n, k, tied):
    import torch

    announce(f"vsa topk rows={rows} n={n} k={k} tied={tied}")
    s = randn(31 + n + k, (rows, n))
    if tied:
        s = (np.round(s * 8) / 8).astype(np.float32)   # heavy ties incl. +-0 (G/kernels/attn3.rs:664-696)
    got = fv.vsa_topk(dev(s), k)
    torch.cuda.synchronize()
    got = got.cpu().numpy().view(np.uint32)
    assert np.array_equal(got, oracle.topk_device_order(s, k))
    if k <= n:
        host = oracle.topk_host_order(s, k)
        assert np.array_equal(np.sort(got, axis=-1), np.sort(host, axis=-1))


@pytest.mark.parametrize("grid", GRIDS)
def test_tile_qkv_and_combine_bit_exact(fv, oracle, grid):
    import torch

    announce(f"vsa tile_qkv/combine grid={grid}")
    ctx = fv.VsaCtx(grid, 0.8)
    plan = ctx.plan
    bh, nb = 2, ctx.num_tiles
    x = randn(41, (bh, ctx.seq, D))
    want = np.zeros((bh, plan.padded, D), dtype=np.uint16)
    real = plan.slot_src >= 0
    want[:, real] = oracle.to_bf16_bits(x)[:, plan.slot_src[real]]
    got = fv.vsa_tile_qkv(dev(x), ctx)
    gotb = fv.vsa_tile_qkv(dev(x).to(torch.bfloat16), ctx)
    torch.cuda.synchronize()
    assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want)
    assert np.array_equal(gotb.view(torch.int16).cpu().numpy().view(np.uint16), want)
    # combine: out[token] = coarse[tile] * gate[token] + sparse[slot], f32 mul then add
    sparse, coarse, gate = randn(42, (bh, plan.padded, D)), randn(43, (bh, nb, D)), randn(44, (bh, ctx.seq, D))
    tile_of_slot = np.arange(plan.padded) // 64
    for g in (gate, None):
        wantc = np.zeros((bh, ctx.seq, D), dtype=np.float32)
        c = coarse[:, tile_of_slot[real]]
        gg = g[:, plan.slot_src[real]] if g is not None else np.float32(1.0)
        wantc[:, plan.slot_src[real]] = (c * gg).astype(np.float32) + sparse[:, real]
        gotc = fv.vsa_combine(dev(sparse), dev(coarse), dev(g) if g is not None else None, ctx)
        torch.cuda.synchronize()
        assert np.array_equal(gotc.cpu().numpy(), wantc)
    g16 = oracle.quantize_bf16(gate)
    a = fv.vsa_combine(dev(sparse), dev(coarse), dev(g16), ctx)
    b = fv.vsa_combine(dev(sparse), dev(coarse), dev(g16).to(torch.bfloat16), ctx)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    # the H3 family's bf16 combine (round16): f32 gate, bf16 gate (same bits), no gate, a tile range
    for g in (gate, None):
        wantr = oracle.vsa_combine(sparse, coarse, g, plan, ctx.seq, round16=True)
        gotr = fv.vsa_combine(dev(sparse), dev(coarse), dev(g) if g is not None else None, ctx, round16=True)
        torch.cuda.synchronize()
        assert np.array_equal(gotr.cpu().numpy(), wantr)
    gotr16 = fv.vsa_combine(dev(sparse), dev(coarse), dev(g16).to(torch.bfloat16), ctx, round16=True)
    torch.cuda.synchronize()
    assert np.array_equal(gotr16.cpu().numpy(), oracle.vsa_combine(sparse, coarse, gate, plan, ctx.seq, round16=True))
    if nb >= 3:
        part = fv.vsa_combine(dev(sparse[:, 64:(nb * 64)]), dev(coarse), dev(gate), ctx, q_base=1, q_tiles=nb - 1,
                              round16=True)
        torch.cuda.synchronize()
        wantp = oracle.vsa_combine(sparse[:, 64:(nb * 64)], coarse, gate, plan, ctx.seq, round16=True, q_base=1,
                                   q_tiles=nb - 1)
        assert np.array_equal(part.cpu().numpy(), wantp)


@pytest.mark.parametrize("grid", GRIDS)
def test_fine_stage_vs_f64_block_sparse(fv, oracle, grid):
    import torch

    announce(f"vsa fine grid={grid}")
    ctx = fv.VsaCtx(grid, 0.8)
    plan, nb, bh = ctx.plan, ctx.num_tiles, 3
    topk = max(1, min(nb, 5))
    q, k, v, _ = vsa_inputs(oracle, 51, bh, ctx.seq, gate=False)
    # distinct lists ((i + h*7 + j) mod nb), as G/kernels_attn.rs:199-208
    sel = np.array([[[(i + h * 7 + j) % nb for j in range(topk)] for i in range(nb)] for h in range(bh)], dtype=np.int32)
    scale = 1.0 / np.sqrt(D)
    qt, kt, vt = (fv.vsa_tile_qkv(dev(x), ctx) for x in (q, k, v))
    sparse = fv.vsa_fine(qt, kt, vt, dev(sel), ctx, scale)
    torch.cuda.synchronize()
    sparse = sparse.cpu().numpy()
    want = brute_block_sparse(q, k, v, sel, plan, scale)
    real = plan.slot_src >= 0
    got_tok = np.zeros_like(want)
    got_tok[:, plan.slot_src[real]] = sparse[:, real]
    assert_parity(got_tok, want, f"vsa_fine_{grid}")
    # a group launch (q_base, q_tiles) writes the same rows
    if nb >= 3:
        part = fv.vsa_fine(qt, kt, vt, dev(sel), ctx, scale, q_base=1, q_tiles=nb - 2)
        torch.cuda.synchronize()
        assert np.array_equal(part.cpu().numpy(), sparse[:, 64:(nb - 1) * 64])


def test_whole_op_folds_the_scale_into_the_one_rounding_of_f32_queries(fv, oracle):
    """f32 q gets its one rounding to bf16 in the whole op's tile pass: with the fold switch on (opt-in) that is the
    rounding of q * scale * log2(e), and the fine kernel runs its form without the per-score multiply. On a q that
    is NOT made of bf16 numbers both orders are equally close to the host oracle, the selection (which never sees
    the rounded copy) is the same list for list, and bf16 operands, which are already rounded, are left alone."""
    import torch

    grid = (5, 6, 9)
    announce(f"vsa whole op, scale folded into f32 q, grid={grid}")
    ctx = fv.VsaCtx(grid, 0.8)
    oplan = oracle.TilePlan(grid)
    q, k, v, g = vsa_inputs(oracle, 67, 2, ctx.seq)
    q = randn(670, q.shape)                                    # f32 values off the bf16 grid
    scale = np.float32(1.0 / np.sqrt(D))
    want = oracle.vsa_attention_host(q, k, v, g, oplan, ctx.topk, 1, 2, D, scale)
    args = [dev(x) for x in (q, k, v, g)]
    assert not fv.fold_scale()                                  # the default is the reference's order
    plain, sel_p = fv.vsa_attention_device(*args, ctx, float(scale), return_selected=True)
    with fv.with_fold_scale(True):
        folded, sel_f = fv.vsa_attention_device(*args, ctx, float(scale), return_selected=True)
    torch.cuda.synchronize()
    assert torch.equal(sel_f, sel_p) and not torch.equal(folded, plain)
    mf = assert_parity(folded.cpu().numpy(), want, "vsa_op_f32_folded")
    mp = assert_parity(plain.cpu().numpy(), want, "vsa_op_f32_unfolded")
    assert mf["rel_l2"] <= 1.1 * mp["rel_l2"] and mf["rel_l2"] <= 2e-2
    b16 = [x.to(torch.bfloat16) for x in args]
    a = fv.vsa_attention_device(*b16, ctx, float(scale))
    with fv.with_fold_scale(True):
        b = fv.vsa_attention_device(*b16, ctx, float(scale))
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.mark.parametrize("grid", GRIDS)
@pytest.mark.parametrize("in_bf16", [False, True])
def test_whole_op_vs_host_oracle(fv, oracle, grid, in_bf16):
    import torch

    announce(f"vsa whole op grid={grid} bf16_in={in_bf16}")
    ctx = fv.VsaCtx(grid, 0.8)
    oplan = oracle.TilePlan(grid)
    b, heads = 1, 2
    q, k, v, g = vsa_inputs(oracle, 61, heads, ctx.seq)
    scale = np.float32(1.0 / np.sqrt(D))
    want, want_sel = oracle.vsa_attention_host(q, k, v, g, oplan, ctx.topk, b, heads, D, scale, return_selected=True)
    cast = (lambda x: dev(x).to(torch.bfloat16)) if in_bf16 else dev
    got, sel = fv.vsa_attention_device(cast(q), cast(k), cast(v), cast(g), ctx, float(scale), return_selected=True)
    torch.cuda.synchronize()
    got, sel = got.cpu().numpy(), sel.cpu().numpy().view(np.uint32)
    # block index lists: the device computes the host oracle's own scores (f64 dot, rt/vsa.rs:185-189),
    # so it selects the host oracle's tiles, row for row; its list order is the device contract
    # (above the threshold ascending, then ties ascending; kernels/core.cu:580-618)
    assert np.array_equal(np.sort(sel, -1), np.sort(want_sel.reshape(sel.shape), -1))
    qc, kc = oracle.vsa_tile_mean(q, oplan), oracle.vsa_tile_mean(k, oplan)
    scores = oracle.vsa_coarse_scores(qc, kc, scale)
    assert np.array_equal(sel, oracle.topk_device_order(scores, ctx.topk).reshape(sel.shape))
    m = assert_parity(got, want, f"vsa_op_{grid}_{'bf16' if in_bf16 else 'f32'}")
    assert m["rel_l2"] <= 2e-2
    # gate None == gate of ones
    ones = np.ones_like(q)
    a = fv.vsa_attention_device(cast(q), cast(k), cast(v), None, ctx, float(scale))
    bb = fv.vsa_attention_device(cast(q), cast(k), cast(v), cast(ones), ctx, float(scale))
    torch.cuda.synchronize()
    assert torch.equal(a, bb)


@pytest.mark.parametrize("grid", GRIDS + [(21, 30, 52)])
def test_whole_op_on_tile_ordered_operands_is_bit_identical(fv, oracle, grid):
    """fv_vsa_attention_tiled (q/k/v already in tile-slot order, as the tile-ordered producers write
    them) == fv_vsa_attention on the token-ordered bf16 tensors: output and block lists bit for bit."""
    import torch

    announce(f"vsa tiled whole op grid={grid}")
    ctx = fv.VsaCtx(grid, 0.8)
    heads = 2
    g = torch.Generator(device="cuda").manual_seed(71)
    q, k, v, gate = (torch.randn((heads, ctx.seq, D), generator=g, device="cuda").to(torch.bfloat16) for _ in range(4))
    scale = float(1.0 / np.sqrt(D))
    slot = torch.from_numpy(ctx.plan.token_slot.astype(np.int64)).cuda()

    def tiled(x):
        t = torch.zeros((heads, ctx.padded, D), device="cuda", dtype=torch.bfloat16)
        t[:, slot] = x
        return t

    for gt in (gate, None):
        want, want_sel = fv.vsa_attention_device(q, k, v, gt, ctx, scale, return_selected=True)
        got, sel = fv.vsa_attention_tiled(tiled(q), tiled(k), tiled(v), gt, ctx, scale, return_selected=True)
        torch.cuda.synchronize()
        assert torch.equal(sel, want_sel)
        assert torch.equal(got, want)
    # the stage entry reads tile-ordered input when slot_src is NULL
    qc = fv.vsa_tile_mean(q, ctx)
    qc_t = fv.vsa_tile_mean(tiled(q), ctx, tiled=True)
    torch.cuda.synchronize()
    assert torch.equal(qc, qc_t)


def test_all_tiles_and_zero_gate_is_dense_attention(fv, oracle):
    """C/rt/vsa.rs:534-597 on the device: every tile selected + zero gate == dense SDPA."""
    import torch

    grid = (3, 5, 7)
    announce(f"vsa all-tiles == dense grid={grid}")
    ctx = fv.VsaCtx(grid, 0.0)
    assert ctx.topk == ctx.num_tiles
    q, k, v, _ = vsa_inputs(oracle, 71, 2, ctx.seq, gate=False)
    zero = np.zeros_like(q)
    got = fv.vsa_attention_device(dev(q), dev(k), dev(v), dev(zero), ctx, 1.0 / np.sqrt(D))
    dense = fv.sdpa_dense_bf16(*(dev(x).to(torch.bfloat16) for x in (q, k, v)))
    torch.cuda.synchronize()
    want = oracle.sdpa_composed(q, k, v)
    assert_parity(got.cpu().numpy(), want, "vsa_all_tiles_vs_composed")
    assert metrics(got.cpu().numpy(), dense.cpu().numpy())["max_abs"] < 5e-3


def test_declines_and_errors(fv):
    import torch

    ctx = fv.VsaCtx((4, 4, 4), 0.8)
    x = torch.zeros((1, 64, 64), device="cuda")
    with pytest.raises(fv.FvDeclined):
        fv.vsa_attention_device(x, x, x, None, ctx, 0.1)     # dim 64
    y = torch.zeros((1, 64, 128), device="cuda")
    with pytest.raises(ValueError, match="gate"):
        fv.vsa_attention_device(y, y, y, y[:, :32].contiguous(), ctx, 0.1)
    s = torch.zeros((2, 5000), device="cuda")
    with pytest.raises(fv.FvDeclined):
        fv.vsa_topk(s, 4)                                   # n > 4096


@pytest.mark.parametrize("grid,topk", [((32, 32, 32), 64), ((21, 30, 52), 125)])
def test_headline_vsa_shapes(fv, oracle, grid, topk):
    """The synthetic VSA benchmark geometry (512 full cubes, top-k 64 of 512) and the reference's own Wan
    480p geometry (624 tiles, top-k 125), H = 12, bf16: block index lists equal to the host oracle's at
    full size (every row of every head); fine + combine output checked on sampled query tiles."""
    import torch

    bh = 12
    announce(f"vsa headline grid={grid} topk={topk} bh={bh}")
    ctx = fv.VsaCtx(grid, 0.8)
    oplan = oracle.TilePlan(grid)
    nb = ctx.num_tiles
    qn, kn, vn, gn = (oracle.quantize_bf16(randn(990 + i, (bh, ctx.seq, D))) for i in range(4))
    q, k, v, g = (dev(x).to(torch.bfloat16) for x in (qn, kn, vn, gn))
    scale = np.float32(1.0 / np.sqrt(D))
    out, sel = fv.vsa_attention_device(q, k, v, g, ctx, float(scale), topk=topk, return_selected=True)
    torch.cuda.synchronize()
    sel = sel.cpu().numpy().view(np.uint32)
    # stages 1-3 of the host oracle (rt/vsa.rs:151-212) at full size: tile means, f64-dot scores, top-k
    scores = oracle.vsa_coarse_scores(oracle.vsa_tile_mean(qn, oplan), oracle.vsa_tile_mean(kn, oplan), scale)
    host_sel = oracle.topk_host_order(scores, topk).reshape(sel.shape)
    assert np.array_equal(np.sort(sel, -1), np.sort(host_sel, -1))          # the reference's block lists, as sets
    assert np.array_equal(sel, oracle.topk_device_order(scores, topk).reshape(sel.shape))   # in the device order
    # sampled query tiles: f64 fine attention over the selected tiles + coarse branch
    vc = oracle.vsa_tile_mean(vn, oplan).astype(np.float64)
    rng = np.random.Generator(np.random.PCG64(5))
    toks = [oplan.slot_src[t * 64: t * 64 + oplan.block_sizes[t]] for t in range(nb)]
    outn = out.cpu().numpy()
    got_rows, want_rows = [], []
    for b in (0, bh - 1):
        for qt in list(rng.choice(nb, size=3, replace=False)) + [nb - 1]:
            keys = np.concatenate([toks[int(kt)] for kt in sel[b, qt]])
            s = (qn[b, toks[qt]].astype(np.float64) @ kn[b, keys].astype(np.float64).T) * float(scale)
            p = np.exp(s - s.max(-1, keepdims=True))
            sparse = (p / p.sum(-1, keepdims=True)) @ vn[b, keys].astype(np.float64)
            cs = scores[b, qt].astype(np.float64)
            cp = np.exp(cs - cs.max())
            coarse = (cp / cp.sum()) @ vc[b]
            want_rows.append(coarse[None, :] * gn[b, toks[qt]] + sparse)
            got_rows.append(outn[b, toks[qt]])
    assert_parity(np.concatenate(got_rows), np.concatenate(want_rows), f"vsa_headline_{grid}")


@pytest.mark.parametrize("grid,sparsity", [((21, 30, 52), 0.8), ((32, 32, 32), 0.875)])
def test_full_size_rows_of_ones(fv, grid, sparsity):
    """V = 1 and a zero gate at the two full-size geometries: the fine stage's softmax over the selected
    tiles' real tokens sums to one, so every real token's output is 1 (partial tiles, padding slots and
    the scatter back to token order included); with gate = 1 the coarse branch adds its own 1."""
    import torch

    announce(f"vsa rows-of-ones grid={grid}")
    ctx = fv.VsaCtx(grid, sparsity)
    heads = 12
    g = torch.Generator(device="cuda").manual_seed(13)
    q, k = (torch.randn((heads, ctx.seq, D), generator=g, device="cuda").to(torch.bfloat16) for _ in range(2))
    v = torch.ones((heads, ctx.seq, D), device="cuda", dtype=torch.bfloat16)
    scale = float(1.0 / np.sqrt(D))
    out0 = fv.vsa_attention_device(q, k, v, torch.zeros_like(v), ctx, scale)
    out1 = fv.vsa_attention_device(q, k, v, None, ctx, scale)
    torch.cuda.synchronize()
    e0, e1 = (out0 - 1.0).abs().max().item(), (out1 - 2.0).abs().max().item()
    print(f"max |out - 1| = {e0:.3e} (zero gate), max |out - 2| = {e1:.3e} (gate of one)")
    assert e0 <= 4e-3 and e1 <= 4e-3


@pytest.mark.parametrize("grid", GRIDS)
def test_log2_domain_form_of_the_fine_stage_and_the_whole_op(fv, oracle, grid):
    """Calls at scale ln 2 (softmax scale folded into Q before its rounding) run the fine kernel's form without the
    per-score multiply-add: same bars against the f64 block-sparse attention and the host oracle at the same
    operands and scale; the block lists stay the host oracle's."""
    import math

    import torch

    ln2 = float(np.float32(math.log(2.0)))
    assert fv.lib().fv_sdpa_is_log2_domain_scale(ln2) == 1
    announce(f"vsa log2-domain grid={grid}")
    ctx = fv.VsaCtx(grid, 0.8)
    plan, nb = ctx.plan, ctx.num_tiles
    oplan = oracle.TilePlan(grid)
    sl2 = np.float32(1.0 / np.sqrt(D)) * np.float32(1.4426950408889634)
    bh = 2
    q = oracle.quantize_bf16(randn(71, (bh, ctx.seq, D)) * sl2)
    k, v = (oracle.quantize_bf16(randn(71 + i, (bh, ctx.seq, D))) for i in (1, 2))
    g = oracle.quantize_bf16(randn(74, (bh, ctx.seq, D), 0.5))
    # fine stage alone, distinct lists
    topk = max(1, min(nb, 5))
    sel = np.array([[[(i + h * 7 + j) % nb for j in range(topk)] for i in range(nb)] for h in range(bh)], dtype=np.int32)
    qt, kt, vt = (fv.vsa_tile_qkv(dev(x), ctx) for x in (q, k, v))
    sparse = fv.vsa_fine(qt, kt, vt, dev(sel), ctx, ln2)
    torch.cuda.synchronize()
    sparse = sparse.cpu().numpy()
    want = brute_block_sparse(q, k, v, sel, plan, ln2)
    real = plan.slot_src >= 0
    got_tok = np.zeros_like(want)
    got_tok[:, plan.slot_src[real]] = sparse[:, real]
    assert_parity(got_tok, want, f"vsa_fine_log2_{grid}")
    # whole op
    want, want_sel = oracle.vsa_attention_host(q, k, v, g, oplan, ctx.topk, 1, bh, D, np.float32(ln2), return_selected=True)
    got, sel = fv.vsa_attention_device(dev(q), dev(k), dev(v), dev(g), ctx, ln2, return_selected=True)
    torch.cuda.synchronize()
    got, sel = got.cpu().numpy(), sel.cpu().numpy().view(np.uint32)
    assert np.array_equal(np.sort(sel, -1), np.sort(want_sel.reshape(sel.shape), -1))
    m = assert_parity(got, want, f"vsa_op_log2_{grid}")
    assert m["rel_l2"] <= 2e-2
