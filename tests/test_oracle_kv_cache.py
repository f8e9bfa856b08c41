"""Pins for the oracle's KV-cache restatement and, side by side, for the library's host arithmetic
(`fv_kv_plan`): the reference's known answers (crates/fastvideo-cudarc/src/wan/causal.rs:872-910)
and hand-built roll sequences. No GPU calls.
"""
import numpy as np
import pytest

import util  # noqa: F401  (puts the package on sys.path)
import fv_sdpa


def both(o, frame_tokens, capacity, sink, max_attention, rolling):
    return (o.KvSpecO(frame_tokens, capacity, sink, max_attention, rolling),
            fv_sdpa.KvSpec(frame_tokens, capacity, sink, max_attention, rolling))


def plan_both(specs, *args):
    want = specs[0].plan(*args)
    m = specs[1].plan(*args)
    assert (m.evicted, m.local_start, m.local_end, m.window_start) == want
    return want


def test_blocks_append_and_steps_overwrite(oracle):
    # causal.rs:872-886: a global 21-frame window of 10-token frames
    s = both(oracle, 10, 210, 0, 210, False)
    assert plan_both(s, 0, 0, 0, 30)[1:] == (0, 30, 0)
    assert plan_both(s, 30, 30, 0, 30)[1:3] == (0, 30)           # the next denoising step: same slots
    assert plan_both(s, 30, 30, 30, 30)[1:] == (30, 60, 0)       # block 1 appends, reads blocks 0 and 1
    with pytest.raises(oracle.KvError):
        s[0].plan(210, 210, 210, 10)                             # a 22nd frame is refused
    with pytest.raises(fv_sdpa.TensorError, match="local_attn_size=-1 keeps a 21-frame KV window"):
        s[1].plan(210, 210, 210, 10)


def test_rolling_cache_keeps_the_sink(oracle):
    # causal.rs:888-910: local_attn_size 6 frames, sink 1 frame, 3-frame blocks of 10 tokens
    s = both(oracle, 10, 60, 10, 60, True)
    assert plan_both(s, 0, 0, 0, 30)[2] == 30
    assert plan_both(s, 30, 30, 30, 30)[2] == 60
    assert plan_both(s, 60, 60, 60, 30) == (30, 30, 60, 0)       # 30 tokens evicted after the sink
    assert plan_both(s, 90, 60, 60, 30)[:3] == (0, 30, 60)       # the next step overwrites in place


def test_plan_errors(oracle):
    s = both(oracle, 10, 60, 10, 60, True)
    for args, text in (((100, 20, 10, 10), "block before the cache start"),
                       ((0, 0, 0, 70), "block longer than the cache")):   # 10 evicted, write end 60 < 70
        with pytest.raises(oracle.KvError, match=text):
            s[0].plan(*args)
        with pytest.raises(fv_sdpa.TensorError, match=text):
            s[1].plan(*args)
    with pytest.raises(fv_sdpa.TensorError, match="sink 6 frames must be below the window"):
        fv_sdpa.KvSpec.rolling_window(10, 6, 6)
    r = fv_sdpa.KvSpec.rolling_window(10, 6, 1)
    assert (r.capacity, r.sink, r.max_attention, r.rolling, r.window_frames()) == (60, 10, 60, True, 6)


def test_plan_sweep_matches(oracle):
    """Every (state, write) of small caches: the library's plan == the oracle's, errors included."""
    rng = np.random.default_rng(5)
    n_ok = n_err = 0
    for _ in range(4000):
        ft = int(rng.integers(1, 5))
        cap = ft * int(rng.integers(1, 8))
        spec = (ft, cap, ft * int(rng.integers(0, 3)), ft * int(rng.integers(1, 9)), bool(rng.integers(0, 2)))
        args = tuple(int(x) for x in (rng.integers(0, 40), rng.integers(0, cap + 1), rng.integers(0, 40), rng.integers(0, 12)))
        s = both(oracle, *spec)
        try:
            want = s[0].plan(*args)
        except oracle.KvError:
            with pytest.raises(fv_sdpa.TensorError):
                s[1].plan(*args)
            n_err += 1
            continue
        m = s[1].plan(*args)
        assert (m.evicted, m.local_start, m.local_end, m.window_start) == want, (spec, args)
        n_ok += 1
    assert n_ok > 300 and n_err > 300


def test_oracle_cache_rolls_by_hand(oracle):
    """Tokens numbered by their absolute position: after every write the window holds the sink and the
    newest tokens, in order."""
    spec = oracle.KvSpecO(2, 8, 2, 8, True)      # 4-frame window of 2-token frames, sink 1 frame
    c = oracle.CausalKvCacheO(spec, 1)
    tok = lambda a, b: np.arange(a, b, dtype=np.float32).reshape(1, 1, -1, 1) * np.ones((1, 2, 1, 3), np.float32)  # noqa: E731
    seen = lambda w: w[0, 0, :, 0].astype(int).tolist()  # noqa: E731
    kw, vw = c.update(0, tok(0, 4), -tok(0, 4), 0)
    assert seen(kw) == [0, 1, 2, 3] and seen(-vw) == [0, 1, 2, 3]
    kw, _ = c.update(0, tok(4, 8), -tok(4, 8), 4)
    assert seen(kw) == list(range(8))
    kw, _ = c.update(0, tok(8, 12), -tok(8, 12), 8)          # rolls: sink 0,1 stays, 2..5 dropped
    assert seen(kw) == [0, 1, 6, 7, 8, 9, 10, 11]
    kw, _ = c.update(0, 100 + tok(8, 12), -tok(8, 12), 8)    # same block again: overwritten in place
    assert seen(kw) == [0, 1, 6, 7, 108, 109, 110, 111]
    kw, _ = c.update(0, tok(12, 14), -tok(12, 14), 12)       # a shorter block
    assert seen(kw) == [0, 1, 108, 109, 110, 111, 12, 13]
    # the sink guard: a recompute of cached frames that would land on the sink leaves it alone
    c2 = oracle.CausalKvCacheO(oracle.KvSpecO(2, 8, 2, 8, True), 1)
    c2.update(0, tok(0, 4), tok(0, 4), 0)
    c2.update(0, tok(4, 8), tok(4, 8), 4)
    c2.sink_guard = True
    kw, _ = c2.update(0, 50 + tok(0, 4), tok(0, 4), 0)        # current_start == 0: not a recompute, lands whole
    assert seen(kw)[:4] == [50, 51, 52, 53]


def test_update_keeps_prefix_and_window(oracle):
    """The reference's known answers, causal.rs:1111-1152 (2-token frames, capacity 8, sink 2)."""
    c = oracle.CausalKvCacheO(oracle.KvSpecO(2, 8, 2, 8, True), 1)
    blk = lambda base: (base + np.arange(4, dtype=np.float32)).reshape(1, 1, 4, 1)  # noqa: E731
    flat = lambda w: w.reshape(-1).tolist()  # noqa: E731
    assert flat(c.update(0, blk(0.0), blk(0.0), 0)[0]) == [0.0, 1.0, 2.0, 3.0]
    assert flat(c.update(0, blk(10.0), blk(10.0), 0)[0]) == [10.0, 11.0, 12.0, 13.0]      # next step: overwritten
    assert c.update(0, blk(20.0), blk(20.0), 4)[0].shape[2] == 8
    assert flat(c.update(0, blk(30.0), blk(30.0), 8)[0]) == [10.0, 11.0, 22.0, 23.0, 30.0, 31.0, 32.0, 33.0]
    assert c.layers[0].local_end == 8
    assert flat(c.update(0, blk(40.0), blk(40.0), 12)[0]) == [10.0, 11.0, 32.0, 33.0, 40.0, 41.0, 42.0, 43.0]


def _tables(seed, s, d, frame0=0.0):
    rng = np.random.Generator(np.random.PCG64(seed))
    theta = (rng.uniform(0.01, 1.0, (1, d // 2)) * (np.arange(s)[:, None] + frame0)).astype(np.float64)
    return (np.repeat(np.cos(theta), 2, axis=1).astype(np.float32), np.repeat(np.sin(theta), 2, axis=1).astype(np.float32), theta)


def test_rope_bhsd_is_a_rotation_of_pairs(oracle):
    """causal.rs:250-262: against the complex-number closed form in f64, norm of every pair kept, the
    inverse rotation (sin negated) undoes it, angle 0 is the identity, tables read from the EVEN slot."""
    rng = np.random.Generator(np.random.PCG64(9))
    b, h, s, d = 2, 3, 7, 16
    x = rng.standard_normal((b, h, s, d)).astype(np.float32)
    cos, sin, theta = _tables(1, s, d)
    got = oracle.rope_bhsd_f32(x, cos, sin)
    z = (x[..., 0::2].astype(np.float64) + 1j * x[..., 1::2].astype(np.float64)) * np.exp(1j * theta)[None, None]
    assert np.abs(got[..., 0::2] - z.real).max() < 1e-6 and np.abs(got[..., 1::2] - z.imag).max() < 1e-6
    n_in = x[..., 0::2] ** 2 + x[..., 1::2] ** 2
    n_out = got[..., 0::2] ** 2 + got[..., 1::2] ** 2
    assert np.allclose(n_in, n_out, rtol=1e-5)
    back = oracle.rope_bhsd_f32(got, cos, -sin)
    assert np.abs(back - x).max() < 1e-6
    assert np.array_equal(oracle.rope_bhsd_f32(x, np.ones_like(cos), np.zeros_like(sin)), x)
    # the odd slots of the tables are never read
    cos2, sin2 = cos.copy(), sin.copy()
    cos2[:, 1::2], sin2[:, 1::2] = 123.0, -7.0
    assert np.array_equal(oracle.rope_bhsd_f32(x, cos2, sin2), got)


def test_rebased_sink_lands_where_roping_there_directly_would(oracle):
    """causal.rs:733-808: the sink keys, roped at frames [0, sink), are re-roped to frames
    [target, target + sink) through an un-roped f32 copy taken once: equal (to rounding) to roping the
    raw keys at the target frames directly, and moving twice does not compound error."""
    rng = np.random.Generator(np.random.PCG64(10))
    b, h, d, ft = 1, 2, 16, 3
    spec = oracle.KvSpecO(ft, 6 * ft, 2 * ft, 6 * ft, True, rebase_sink=True)
    raw = rng.standard_normal((b, h, 6 * ft, d)).astype(np.float32)
    cos0, sin0, _ = _tables(2, 6 * ft, d)                       # positions 0 .. 6*ft of the clip
    c = oracle.CausalKvCacheO(spec, 1)
    c.update(0, oracle.rope_bhsd_f32(raw, cos0, sin0), raw, 0)
    sink = spec.sink
    assert spec.sink_target(9) == 3 and spec.sink_target(5) == 0
    for target in (3, 7, 3):
        cosn, sinn, _ = _tables(2, sink, d, frame0=float(target * ft))
        c.rebase_sink(target, (cos0[:sink], sin0[:sink]), (cosn, sinn))
        want = oracle.rope_bhsd_f32(raw[:, :, :sink], cosn, sinn)
        assert np.abs(c.layers[0].k[:, :, :sink] - want).max() < 2e-6
        assert np.array_equal(c.layers[0].k[:, :, sink:], oracle.rope_bhsd_f32(raw, cos0, sin0)[:, :, sink:])
        assert c.layers[0].sink_at == target
    before = c.layers[0].k.copy()
    c.rebase_sink(3, (cos0[:sink], sin0[:sink]), (cosn, sinn))   # already there: untouched
    assert np.array_equal(c.layers[0].k, before)
