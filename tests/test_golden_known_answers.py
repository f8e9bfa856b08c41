"""The reference's own known answers (tests/golden/reference_known_answers.json: data transcribed from
its unit tests and run artifacts) against the oracle and against the library's host logic. No GPU."""
import json
import os

import numpy as np
import pytest

import util  # noqa: F401
import fv_sdpa

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")))


def test_topk_rule_and_wan_grid(oracle):
    for sparsity, n, want in G["topk_for"]["cases"]:
        assert oracle.topk_for(sparsity, n) == want and fv_sdpa.topk_for(sparsity, n) == want
    w = G["wan_480p_grid"]
    for mod in (oracle, fv_sdpa):
        p = mod.TilePlan(tuple(w["grid"]))
        assert p.num_tiles == w["num_tiles"] and mod.topk_for(w["sparsity"], p.num_tiles) == w["topk"]


def test_tile_plans(oracle):
    t = G["tile_plan"]
    for mod in (oracle, fv_sdpa):
        for grid in t["permutation_grids"]:
            p = mod.TilePlan(tuple(grid))
            assert p.seq == grid[0] * grid[1] * grid[2] and p.padded == p.num_tiles * 64
            real = p.slot_src >= 0
            assert sorted(p.slot_src[real].tolist()) == list(range(p.seq))
            assert np.array_equal(np.asarray(p.token_slot)[p.slot_src[real]], np.nonzero(real)[0])
            assert int(np.sum(p.block_sizes)) == p.seq and int(np.max(p.block_sizes)) <= 64
        full = mod.TilePlan(tuple(t["full_tiles_grid"]))
        assert (full.slot_src >= 0).all() and (np.asarray(full.block_sizes) == 64).all()
        part = mod.TilePlan(tuple(t["partial"]["grid"]))
        assert part.num_tiles == t["partial"]["num_tiles"]
        assert np.asarray(part.block_sizes).tolist() == t["partial"]["block_sizes"]
        assert part.slot_src[:4].tolist() == t["partial"]["first_slots"] and (part.slot_src[4:64] == -1).all()
        assert part.slot_src[64] == t["partial"]["slot_64"]


def test_shard_ranges(oracle):
    for seq, world, want in G["shard_ranges"]["cases"]:
        want = [tuple(x) for x in want]
        assert oracle.shard_ranges(seq, world) == want and fv_sdpa.shard_ranges(seq, world) == want


def test_block_causal_for(oracle):
    b = G["block_causal_for"]
    frame_tokens = (b["h"] // b["patch"][1]) * (b["w"] // b["patch"][2])
    s = b["frames"] * frame_tokens
    for window, fpb in b["equal_to_causal_temporal_mask"]:
        bc = oracle.block_causal_for(fpb, window, frame_tokens)
        assert bc is not None and fv_sdpa.block_causal_for(fpb, window, frame_tokens) == bc
        want = oracle.causal_temporal_mask(tuple(b["patch"]), fpb, window, b["frames"], b["h"], b["w"])
        assert np.array_equal(oracle.block_causal_dense_mask(*bc, s, s), want)
        assert np.array_equal(fv_sdpa.block_causal_dense_mask(*bc, s, s), want)
    for window, fpb in b["none"]:
        assert oracle.block_causal_for(fpb, window, frame_tokens) is None
        assert fv_sdpa.block_causal_for(fpb, window, frame_tokens) is None


def test_kv_plan(oracle):
    for name in ("global_21_frames_of_10", "rolling_6_frames_sink_1"):
        blk = G["kv_plan"][name]
        sp = blk["spec"]
        args5 = (sp["frame_tokens"], sp["capacity"], sp["sink"], sp["max_attention"], sp["rolling"])
        o, l = oracle.KvSpecO(*args5), fv_sdpa.KvSpec(*args5)
        for c in blk["cases"]:
            if c.get("error"):
                with pytest.raises(oracle.KvError):
                    o.plan(*c["args"])
                with pytest.raises(fv_sdpa.TensorError):
                    l.plan(*c["args"])
                continue
            got_o = dict(zip(("evicted", "local_start", "local_end", "window_start"), o.plan(*c["args"])))
            m = l.plan(*c["args"])
            got_l = {"evicted": m.evicted, "local_start": m.local_start, "local_end": m.local_end, "window_start": m.window_start}
            for key in ("evicted", "local_start", "local_end", "window_start"):
                if key in c:
                    assert got_o[key] == c[key] and got_l[key] == c[key], (name, c, key)


def test_kv_update_sequence(oracle):
    u = G["kv_update"]
    sp = u["spec"]
    c = oracle.CausalKvCacheO(oracle.KvSpecO(sp["frame_tokens"], sp["capacity"], sp["sink"], sp["max_attention"], sp["rolling"]), 1)
    for step in u["steps"]:
        blk = (step["base"] + np.arange(4, dtype=np.float32)).reshape(1, 1, 4, 1)
        kw, vw = c.update(0, blk, blk, step["current_start"])
        if "window" in step:
            assert kw.reshape(-1).tolist() == step["window"] and vw.reshape(-1).tolist() == step["window"]
        else:
            assert kw.shape[2] == step["window_len"]


def test_backend_parse():
    b = G["backend_parse"]
    for name in b["named"]:
        assert fv_sdpa.parse_backend(name) == name
    for v in b["dense_default"]:
        assert fv_sdpa.parse_backend(v) == "dense"


def test_composed_plans_on_the_closed_form_inputs(oracle):
    c = G["composed_plans_closed_form_inputs"]["shape"]
    n_q, n_k = c["b"] * c["h"] * c["sq"] * c["d"], c["b"] * c["h"] * c["sk"] * c["d"]
    mk = lambda n, k, shape: (np.sin(np.arange(n, dtype=np.float32) * np.float32(k)) * np.float32(0.9)).astype(np.float32).reshape(shape)  # noqa: E731
    q = mk(n_q, 0.37, (c["b"] * c["h"], c["sq"], c["d"]))
    k = mk(n_k, 0.71, (c["b"] * c["h"], c["sk"], c["d"]))
    v = mk(n_k, 1.13, (c["b"] * c["h"], c["sk"], c["d"]))
    base = oracle.sdpa_composed(q, k, v)
    assert np.isfinite(base).all() and base.shape == q.shape
    assert np.array_equal(base, oracle.sdpa_composed(q, k, v, scale=1.0 / np.sqrt(c["d"])))
    assert not np.array_equal(base, oracle.sdpa_composed(q, k, v, scale=0.5))
