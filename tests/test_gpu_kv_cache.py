"""The causal-Wan KV cache on the device, through the C ABI: token copies and the in-place roll are
bit-exact against numpy; a cache driven block by block holds, after every write, exactly the window
the oracle's restatement of the reference holds (crates/fastvideo-cudarc/src/wan/causal.rs:540-706);
the fused kernel reading that window in place is bit-identical to the same kernel on a contiguous
copy; and block by block through the cache equals the whole clip under the block-causal mask
(the reference's own invariant, causal.rs:916-1000) within the kernel tolerance.
"""
import numpy as np
import pytest

from util import announce, assert_parity, qkv, to_dev_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fv():
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


@pytest.mark.parametrize("bf16", [True, False])
def test_copy_and_shift_tokens_bit_exact(fv, bf16):
    import torch

    announce(f"kv copy/shift bf16={bf16}")
    dt = torch.bfloat16 if bf16 else torch.float32
    bh, rows, d = 5, 37, 64
    g = torch.Generator(device="cuda").manual_seed(3)
    dst = torch.randn((bh, rows, d), generator=g, device="cuda").to(dt)
    src = torch.randn((bh, 11, d), generator=g, device="cuda").to(dt)
    want = dst.clone()
    want[:, 20:27] = src[:, 3:10]
    fv.kv_copy_tokens(dst, 20, src, 3, 7)
    torch.cuda.synchronize()
    assert torch.equal(dst, want)
    # a shift shorter than the moved range: source and destination overlap, chunks must not
    for frm, to, n in ((9, 4, 25), (30, 0, 7), (5, 4, 32), (12, 12, 3)):
        t = torch.randn((bh, rows, d), generator=g, device="cuda").to(dt)
        want = t.clone()
        want[:, to:to + n] = t[:, frm:frm + n].clone()
        fv.kv_shift_tokens_down(t, frm, to, n)
        torch.cuda.synchronize()
        assert torch.equal(t, want), (frm, to, n)
    with pytest.raises(fv.FvError):
        fv.kv_copy_tokens(dst, 35, src, 0, 7)          # past the destination
    with pytest.raises(fv.FvError):
        fv.kv_shift_tokens_down(dst, 3, 9, 4)          # tokens only move down


@pytest.mark.parametrize("d", [128, 64])
def test_row_windows_are_read_in_place_bit_identically(fv, d):
    import torch

    announce(f"strided dense d={d}")
    bh, rows_q, rows_kv = 3, 400, 1000
    g = torch.Generator(device="cuda").manual_seed(5)
    Q = torch.randn((bh, rows_q, d), generator=g, device="cuda").to(torch.bfloat16)
    K = torch.randn((bh, rows_kv, d), generator=g, device="cuda").to(torch.bfloat16)
    V = torch.randn((bh, rows_kv, d), generator=g, device="cuda").to(torch.bfloat16)
    for (q0, q1), (k0, k1) in (((0, 400), (0, 1000)), ((17, 300), (130, 899)), ((399, 400), (0, 1)), ((5, 261), (936, 1000))):
        q, k, v = Q[:, q0:q1], K[:, k0:k1], V[:, k0:k1]
        want = fv.sdpa_dense_bf16(q.contiguous(), k.contiguous(), v.contiguous())
        got = fv.sdpa_dense_bf16_windows(q, k, v)
        torch.cuda.synchronize()
        assert torch.equal(got, want), ((q0, q1), (k0, k1))
    with pytest.raises(ValueError):
        fv.sdpa_dense_bf16_windows(Q[:, ::2], K, V)


def _blocks(seed, b, h, n, d, count):
    rng = np.random.Generator(np.random.PCG64(seed))
    return [(rng.standard_normal((b, h, n, d)).astype(np.float32), rng.standard_normal((b, h, n, d)).astype(np.float32))
            for _ in range(count)]


CACHES = [
    # frame_tokens, capacity frames, sink frames, rolling, block frames, blocks
    (6, 7, 0, False, 2, 3),      # global window, appends only
    (6, 6, 1, True, 3, 5),       # the reference's rolling example geometry (causal.rs:888-910)
    (5, 8, 2, True, 3, 6),       # capacity not a multiple of the block: partial evictions
    (4, 5, 0, True, 2, 6),       # no sink
]


@pytest.mark.parametrize("static", [True, False])
@pytest.mark.parametrize("case", CACHES)
@pytest.mark.parametrize("bf16", [True, False])
def test_cache_windows_equal_the_oracles(fv, oracle, case, bf16, static):
    """Static mode (persistent buffers, wan/causal.rs:386-391) and the tensor-per-write mode
    (wan/causal.rs:379-385, 556-624) return the same windows: the oracle's, bit for bit."""
    import torch

    ft, cap_f, sink_f, rolling, blk_f, count = case
    announce(f"kv cache {case} bf16={bf16} static={static}")
    b, h, d, layers = 2, 3, 64, 2
    n = blk_f * ft
    spec = fv.KvSpec(ft, cap_f * ft, sink_f * ft, cap_f * ft, rolling)
    ospec = oracle.KvSpecO(ft, cap_f * ft, sink_f * ft, cap_f * ft, rolling)
    cache, ocache = fv.CausalKvCache(spec, layers, static=static), oracle.CausalKvCacheO(ospec, layers)
    assert cache.is_static() == static
    dt = torch.bfloat16 if bf16 else torch.float32
    rnd = (lambda x: oracle.quantize_bf16(x)) if bf16 else (lambda x: x)
    dev = lambda x: torch.from_numpy(x).cuda().to(dt)  # noqa: E731
    for layer in range(layers):
        for i, (k, v) in enumerate(_blocks(100 * layer + ft, b, h, n, d, count)):
            k, v = rnd(k), rnd(v)
            for step in range(2):    # every block runs twice: an append, then an overwrite in place
                kk = k if step == 0 else rnd(k * 0.5)
                want_k, want_v = ocache.update(layer, kk, v, i * n)
                kw, vw = cache.update(layer, dev(kk), dev(v), i * n)
                torch.cuda.synchronize()
                assert tuple(kw.shape) == want_k.shape and kw.dtype == dt
                assert np.array_equal(kw.float().cpu().numpy(), want_k), (layer, i, step)
                assert np.array_equal(vw.float().cpu().numpy(), want_v), (layer, i, step)
                o = ocache.layers[layer]
                assert cache.pointers(layer) == (o.global_end, o.local_end)
    if static:
        assert cache.bytes() == layers * 2 * b * h * max(cap_f * ft, n) * d * (2 if bf16 else 4)
    else:   # exactly the cached tokens
        assert cache.bytes() == sum(2 * b * h * cache.pointers(layer)[1] * d * (2 if bf16 else 4) for layer in range(layers))
        with pytest.raises(fv.TensorError, match="needs a static cache"):
            cache.advance(0, n)
    # a new rollout keeps the buffers and starts from empty pointers
    cache.reset()
    ocache.reset()
    assert cache.pointers(0) == (0, 0)
    k, v = _blocks(7, b, h, n, d, 1)[0]
    kw, _ = cache.update(0, dev(rnd(k)), dev(rnd(v)), 0)
    torch.cuda.synchronize()
    assert np.array_equal(kw.float().cpu().numpy(), ocache.update(0, rnd(k), rnd(v), 0)[0])


@pytest.mark.parametrize("static", [True, False])
def test_update_keeps_prefix_and_window(fv, static):
    """The reference's known answers for `update` (causal.rs:1111-1152), each token's value repeated
    over a 4-wide head dim (the device copies move 16-byte units)."""
    import torch

    announce(f"kv cache known answers static={static}")
    cache = fv.CausalKvCache(fv.KvSpec(2, 8, 2, 8, True), 1, static=static)
    blk = lambda base: (base + torch.arange(4, dtype=torch.float32, device="cuda")).reshape(1, 1, 4, 1).repeat(1, 1, 1, 4)  # noqa: E731

    def flat(w):
        torch.cuda.synchronize()
        assert torch.equal(w, w[..., :1].expand_as(w))
        return w[0, 0, :, 0].tolist()

    assert flat(cache.update(0, blk(0.0), blk(0.0), 0)[0]) == [0.0, 1.0, 2.0, 3.0]
    assert flat(cache.update(0, blk(10.0), blk(10.0), 0)[0]) == [10.0, 11.0, 12.0, 13.0]
    assert cache.update(0, blk(20.0), blk(20.0), 4)[0].shape[2] == 8
    assert flat(cache.update(0, blk(30.0), blk(30.0), 8)[0]) == [10.0, 11.0, 22.0, 23.0, 30.0, 31.0, 32.0, 33.0]
    assert cache.pointers(0)[1] == 8
    kw, vw = cache.update(0, blk(40.0), blk(40.0), 12)        # 1-token... the roll moves 2 tokens by 4
    assert flat(kw) == [10.0, 11.0, 32.0, 33.0, 40.0, 41.0, 42.0, 43.0] and flat(vw) == flat(kw)


def test_cache_errors_and_sink_guard(fv, oracle):
    import torch

    announce("kv cache errors / sink guard")
    b, h, d, ft = 1, 2, 64, 4
    dev = lambda x: torch.from_numpy(x).cuda().to(torch.bfloat16)  # noqa: E731
    glob = fv.CausalKvCache(fv.KvSpec.global_window(ft, 3), 1)
    blk = _blocks(1, b, h, 2 * ft, d, 1)[0]
    glob.update(0, dev(blk[0]), dev(blk[1]), 0)
    with pytest.raises(fv.TensorError, match="local_attn_size=-1 keeps a 3-frame KV window"):
        glob.update(0, dev(blk[0]), dev(blk[1]), 2 * ft)
    with pytest.raises(fv.TensorError, match="no layer 4"):
        glob.update(4, dev(blk[0]), dev(blk[1]), 0)
    with pytest.raises(fv.TensorError, match="do not fit these keys"):
        glob.update(0, dev(blk[0][:, :1]), dev(blk[1][:, :1]), 0)
    # sink guard (causal.rs:396-418): a recompute of cached frames leaves the sink slots as they are
    spec, ospec = fv.KvSpec(ft, 6 * ft, ft, 6 * ft, True), oracle.KvSpecO(ft, 6 * ft, ft, 6 * ft, True)
    cache, ocache = fv.CausalKvCache(spec, 1), oracle.CausalKvCacheO(ospec, 1)
    q16 = oracle.quantize_bf16
    for i, (k, v) in enumerate(_blocks(2, b, h, 3 * ft, d, 2)):
        cache.update(0, dev(k), dev(v), i * 3 * ft)
        ocache.update(0, q16(k), q16(v), i * 3 * ft)
    cache.set_sink_guard(True)
    ocache.sink_guard = True
    k, v = _blocks(3, b, h, 6 * ft, d, 1)[0]
    # frames [0, 6) again from current_start 0 is not a recompute; from a later start it is
    for start, kk, vv in ((0, k, v), (3 * ft, k[:, :, :3 * ft], v[:, :, :3 * ft])):
        want_k, want_v = ocache.update(0, q16(kk), q16(vv), start)
        kw, vw = cache.update(0, dev(kk), dev(vv), start)
        torch.cuda.synchronize()
        assert np.array_equal(kw.float().cpu().numpy(), want_k) and np.array_equal(vw.float().cpu().numpy(), want_v)


@pytest.mark.parametrize("act16", [True, False])
def test_kv_window_plan_reads_the_cache_in_place(fv, oracle, act16):
    """sdpa(q, kw, vw, Plan::kv_window()) (wan/transformer.rs:292-294) on the windows of a rolling
    cache: bit-identical to the fused kernel on contiguous copies, and within tolerance of the
    fp32 oracle on the window."""
    import torch

    b, h, d, ft = 1, 3, 128, 40
    n, layers = 3 * ft, 1
    announce(f"kv window plan act16={act16}")
    spec = fv.KvSpec.rolling_window(ft, 9, 1)
    cache = fv.CausalKvCache(spec, layers)
    ocache = oracle.CausalKvCacheO(oracle.KvSpecO(ft, 9 * ft, ft, 9 * ft, True), layers)
    with fv.with_bf16_act(act16):
        for i in range(5):
            q, k, v = (x.reshape(b, h, n, d) for x in qkv(500 + i, b * h, n, n, d))
            kw, vw = cache.update(0, to_dev_bf16(k), to_dev_bf16(v), i * n)
            want_k, want_v = ocache.update(0, oracle.quantize_bf16(k), oracle.quantize_bf16(v), i * n)
            assert not kw.is_contiguous() or kw.shape[2] == spec.capacity
            before = fv.rt_stats()
            got = fv.sdpa(to_dev_bf16(q), kw, vw, fv.Plan.kv_window())
            after = fv.rt_stats()
            assert after["fused"] == before["fused"] + 1 and after["composed"] == before["composed"]
            assert got.dtype == (torch.bfloat16 if act16 else torch.float32)
            direct = fv.sdpa_dense_bf16(to_dev_bf16(q).reshape(b * h, n, d), kw.reshape(b * h, -1, d).contiguous(),
                                        vw.reshape(b * h, -1, d).contiguous(), out_bf16=act16)
            torch.cuda.synchronize()
            assert torch.equal(got.reshape(b * h, n, d), direct)
            sk = want_k.shape[2]
            want = oracle.sdpa_composed(q.reshape(b * h, n, d), want_k.reshape(b * h, sk, d), want_v.reshape(b * h, sk, d))
            assert_parity(got.float().cpu().numpy().reshape(b * h, n, d), want, f"kv_window_block{i}",
                          max_abs=2e-2 if act16 else 1e-2)
        # the composed route (FASTVIDEO_WAN_CAUSAL_FLASH=0) takes contiguous copies of the windows
        got_c = fv.sdpa(to_dev_bf16(q), kw, vw, fv.Plan.kv_window_with(False))
        torch.cuda.synchronize()
        assert_parity(got_c.float().cpu().numpy().reshape(b * h, n, d), want, "kv_window_composed",
                      max_abs=2e-2 if act16 else 1e-5)


def test_cached_blocks_equal_the_masked_whole_clip(fv, oracle):
    """causal.rs:916-1000: block by block through a global-window cache is the whole clip under the
    block-causal mask: every query meets the same keys."""
    import torch

    bh, d, ft, fpb, frames = 4, 128, 90, 3, 9
    n, s = fpb * ft, frames * ft
    announce("kv cache blocks == block-causal whole clip")
    q, k, v = qkv(77, bh, s, s, d)
    whole = fv.sdpa_block_causal_bf16(to_dev_bf16(q), to_dev_bf16(k), to_dev_bf16(v), n, 0, 0)
    cache = fv.CausalKvCache(fv.KvSpec.global_window(ft, frames), 1)
    r4 = lambda x, a, bnd: to_dev_bf16(x[:, a:bnd]).reshape(1, bh, bnd - a, d)  # noqa: E731
    parts = []
    with fv.with_bf16_act(False):
        for i in range(frames // fpb):
            kw, vw = cache.update(0, r4(k, i * n, (i + 1) * n), r4(v, i * n, (i + 1) * n), i * n)
            parts.append(fv.sdpa(r4(q, i * n, (i + 1) * n), kw, vw, fv.Plan.kv_window()))
    torch.cuda.synchronize()
    blocks = torch.cat(parts, dim=2).reshape(bh, s, d)
    assert_parity(blocks.cpu().numpy(), whole.cpu().numpy(), "kv_blocks_vs_block_causal", max_abs=2e-3)
    want = oracle.sdpa_composed(q, k, v, mask=oracle.block_causal_dense_mask(n, 0, 0, s, s))
    assert_parity(blocks.cpu().numpy(), want, "kv_blocks_vs_oracle")


def _rope_tables(seed, s, d, frame0=0.0):
    rng = np.random.Generator(np.random.PCG64(seed))
    theta = rng.uniform(0.01, 1.0, (1, d // 2)) * (np.arange(s)[:, None] + frame0)
    return (np.repeat(np.cos(theta), 2, axis=1).astype(np.float32), np.repeat(np.sin(theta), 2, axis=1).astype(np.float32))


@pytest.mark.parametrize("in16", [False, True])
@pytest.mark.parametrize("out16", [False, True])
def test_rope_bhsd_bit_exact(fv, oracle, in16, out16):
    import torch

    announce(f"rope_bhsd in16={in16} out16={out16}")
    b, h, s, d = 2, 3, 37, 64
    rng = np.random.Generator(np.random.PCG64(21))
    x = rng.standard_normal((b, h, s, d)).astype(np.float32)
    if in16:
        x = oracle.quantize_bf16(x)
    cos, sin = _rope_tables(22, s, d)
    tx = torch.from_numpy(x).cuda().to(torch.bfloat16 if in16 else torch.float32)
    tc, ts = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    for neg in (False, True):
        want = oracle.rope_bhsd_f32(x, cos, -sin if neg else sin)
        if out16:
            want = oracle.quantize_bf16(want)
        got = fv.rope_bhsd(tx, tc, ts, negate_sin=neg, out_bf16=out16)
        torch.cuda.synchronize()
        assert got.dtype == (torch.bfloat16 if out16 else torch.float32)
        assert np.array_equal(got.float().cpu().numpy(), want)


def test_rebased_sink_in_the_tensor_per_write_mode(fv, oracle):
    """The rebased-sink policy on a cache that is not static: same contents as the oracle's after every roll."""
    import torch

    announce("kv rebased sink, tensor-per-write mode")
    b, h, d, ft = 1, 2, 64, 4
    win_f, sink_f, blk_f = 6, 2, 2
    n, sink = blk_f * ft, sink_f * ft
    spec = fv.KvSpec.rolling_window(ft, win_f, sink_f, fv.KvRope.REBASED_SINK)
    ospec = oracle.KvSpecO(ft, win_f * ft, sink, win_f * ft, True, rebase_sink=True)
    cache, ocache = fv.CausalKvCache(spec, 1, static=False), oracle.CausalKvCacheO(ospec, 1)
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
    cos_o, sin_o = _rope_tables(30, sink, d)
    for blk in range(6):
        target = spec.sink_target((blk + 1) * blk_f)
        if target > 0:
            cos_n, sin_n = _rope_tables(30, sink, d, frame0=float(target * ft))
            cache.rebase_sink(target, (dev(cos_o), dev(sin_o)), (dev(cos_n), dev(sin_n)))
            ocache.rebase_sink(target, (cos_o, sin_o), (cos_n, sin_n), quantize=None)
        k, v = _blocks(140 + blk, b, h, n, d, 1)[0]
        want_k, want_v = ocache.update(0, k, v, blk * n)
        kw, vw = cache.update(0, dev(k), dev(v), blk * n)
        torch.cuda.synchronize()
        assert np.array_equal(kw.cpu().numpy(), want_k) and np.array_equal(vw.cpu().numpy(), want_v), blk


@pytest.mark.parametrize("bf16", [True, False])
def test_rebased_sink_policy_equals_the_oracles(fv, oracle, bf16):
    """A rolling cache under the rebased-sink RoPE policy (causal.rs:733-776): after every roll the
    sink is re-roped to the frames just before the rolled part; cache contents equal the oracle's bit
    for bit (the rope is elementwise f32), pointers follow, advance / set_pointers move host state only."""
    import torch

    announce(f"kv rebased sink bf16={bf16}")
    b, h, d, ft, layers = 1, 2, 64, 4, 2
    win_f, sink_f, blk_f = 6, 2, 2
    n, sink = blk_f * ft, sink_f * ft
    spec = fv.KvSpec.rolling_window(ft, win_f, sink_f, fv.KvRope.REBASED_SINK)
    ospec = oracle.KvSpecO(ft, win_f * ft, sink, win_f * ft, True, rebase_sink=True)
    cache, ocache = fv.CausalKvCache(spec, layers), oracle.CausalKvCacheO(ospec, layers)
    dt = torch.bfloat16 if bf16 else torch.float32
    rnd = oracle.quantize_bf16 if bf16 else (lambda x: x)
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x)).cuda()  # noqa: E731
    cos_o, sin_o = _rope_tables(30, sink, d)
    for blk in range(6):
        end_frame = (blk + 1) * blk_f
        target = spec.sink_target(end_frame)
        assert target == ospec.sink_target(end_frame)
        if target > 0:
            cos_n, sin_n = _rope_tables(30, sink, d, frame0=float(target * ft))
            cache.rebase_sink(target, (dev(cos_o), dev(sin_o)), (dev(cos_n), dev(sin_n)))
            ocache.rebase_sink(target, (cos_o, sin_o), (cos_n, sin_n), quantize=rnd if bf16 else None)
        for layer in range(layers):
            k, v = _blocks(40 + 10 * layer + blk, b, h, n, d, 1)[0]
            k, v = rnd(k), rnd(v)
            want_k, want_v = ocache.update(layer, k, v, blk * n)
            kw, vw = cache.update(layer, dev(k).to(dt), dev(v).to(dt), blk * n)
            torch.cuda.synchronize()
            assert np.array_equal(kw.float().cpu().numpy(), want_k), (blk, layer)
            assert np.array_equal(vw.float().cpu().numpy(), want_v), (blk, layer)
            o = ocache.layers[layer]
            # a layer's sink moves at the first rebase after it holds the sink
            assert cache.pointers4(layer)[:3] == (o.global_end, o.local_end, o.sink_at)
    assert cache.pointers4(0)[3] is True
    # advance == update's bookkeeping without device work; set_pointers puts a state back
    state = [cache.pointers4(layer) for layer in range(layers)]
    cache.advance(6 * n, n, spec.sink_target(7 * blk_f))
    moved = cache.pointers4(0)
    assert moved[0] == 7 * n and moved[2] == spec.sink_target(7 * blk_f)
    cache.set_pointers(state)
    assert [cache.pointers4(layer) for layer in range(layers)] == state
    with pytest.raises(fv.TensorError, match="one entry per layer"):
        cache.set_pointers(state[:1])
    plain = fv.CausalKvCache(fv.KvSpec.rolling_window(ft, win_f, sink_f), 1)
    with pytest.raises(fv.TensorError, match="rebased-sink RoPE policy"):
        plain.rebase_sink(1, (dev(cos_o), dev(sin_o)), (dev(cos_o), dev(sin_o)))
    with pytest.raises(fv.TensorError, match="advance over an unwritten cache"):
        plain.advance(0, n)


def test_block_keys_settle_once_the_window_is_full(fv):
    """The reference's known answers for `block_key` (causal.rs:1196-1232; head dim 8 here instead of 2,
    the rope kernel rotates 8 elements per thread): keys follow the fill — appends while the window fills, the first roll
    takes the un-roped sink, then every block has the same key; an in-place re-run of a block neither
    appends, rebases nor evicts."""
    import torch

    spec = fv.KvSpec.rolling_window(10, 6, 2, fv.KvRope.REBASED_SINK)
    cache = fv.CausalKvCache(spec, 1)
    blk = lambda start: (start + torch.arange(160, dtype=torch.float32, device="cuda")).reshape(1, 1, 20, 8)  # noqa: E731
    tab = torch.ones((20, 8), device="cuda")
    zero = torch.zeros((20, 8), device="cuda")
    keys = []
    for b in range(6):
        start = b * 20
        target = spec.sink_target(b * 2 + 2)
        key = cache.block_key(start, 20, target)
        keys.append(key)
        if key.rebase:
            cache.rebase_sink(target, (tab, zero), (tab, zero))
        cache.update(0, blk(start), blk(start), start)
        again = cache.block_key(start, 20, target)      # the in-place re-run of the same block (next step)
        assert not again.appends and not again.rebase and again.evicted == 0
    torch.cuda.synchronize()
    assert keys[0].local_end == 0
    assert keys[1].appends and keys[1].evicted == 0 and not keys[1].rebase
    assert keys[3].rebase and keys[3].take_raw and keys[3].evicted == 20
    assert keys[4].rebase and not keys[4].take_raw
    assert keys[4] == keys[5]
    p = [cache.pointers4(0)]
    cache.set_pointers(p)
    assert [cache.pointers4(0)] == p
    # a block the cache cannot take is refused with the plan's message
    with pytest.raises(fv.TensorError):
        cache.block_key(1000, 20, 0)
