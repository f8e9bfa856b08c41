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
