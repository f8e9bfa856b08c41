"""The `sdpa(q, k, v, &Plan)` entry on the device, read like the reference's own unit
tests (crates/fastvideo-cudarc/src/rt/sdpa.rs:508-575, rt/attn.rs:905-1002): plan
equivalences, refusals, the block-causal fallback, dtype rules under bf16 activations —
plus parity of the device composed path against the fp32 oracle.
"""
import numpy as np
import pytest

from util import announce, assert_parity, metrics, qkv, randn
from test_oracle_sdpa import sin_tensor

pytestmark = pytest.mark.gpu


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


def test_dense_plans_without_a_fused_kernel_are_the_composed_reference(fv, oracle):
    # rt/sdpa.rs:522-542: 1x2x5x7x8 (d = 8: the fused kernel declines, every plan is composed)
    announce("rt plans == composed, 1x2x5x7x8")
    b, h, sq, sk, d = 1, 2, 5, 7, 8
    q = sin_tensor(b * h * sq * d, 0.37, (b, h, sq, d))
    k = sin_tensor(b * h * sk * d, 0.71, (b, h, sk, d))
    v = sin_tensor(b * h * sk * d, 1.13, (b, h, sk, d))
    P = fv.Plan
    with fv.with_bf16_act(False):
        want = host(fv.sdpa(dev(q), dev(k), dev(v), P.composed(None, None)))
        for plan in (P.dense(None), P.dense(None).fp8_first(), P.masked(None, None), P.composed(None, None),
                     P.kv_window_with(True), P.kv_window_with(False)):
            got = fv.sdpa(dev(q), dev(k), dev(v), plan)
            assert got.dtype.is_floating_point and got.element_size() == 4
            assert np.array_equal(host(got), want)
        scaled = host(fv.sdpa(dev(q), dev(k), dev(v), P.dense(0.5)))
        assert not np.array_equal(scaled, want)
    ref = oracle.sdpa_composed(q.reshape(h, sq, d), k.reshape(h, sk, d), v.reshape(h, sk, d))
    assert np.abs(want.reshape(h, sq, d) - ref).max() < 2e-6


def test_non_bhsd_operands_are_refused(fv):
    q = dev(np.zeros((2, 4), np.float32))
    with pytest.raises(fv.TensorError, match="BHSD"):
        fv.sdpa(q, q, q, fv.Plan.dense(None))


def test_vdn_window_of_no_frames_is_dense(fv, oracle):
    """A window without video rows masks nothing (rt/attn.rs:497-501): the kernel declines it
    (frames == 0) and the masked fallback runs with an all-visible mask."""
    import torch

    q, k, v = qkv(73, 2, 40, 40, 128)
    qd, kd, vd = (dev(x.reshape(1, 2, 40, 128)) for x in (q, k, v))
    with fv.with_bf16_act(False):
        out = fv.sdpa(qd, kd, vd, fv.Plan.vdn_window(None, fv.VdnWindow(5, 0, 0)))
    torch.cuda.synchronize()
    want = oracle.sdpa_composed(q, k, v)
    assert np.abs(out.cpu().numpy().reshape(2, 40, 128) - want).max() <= 1e-5


def test_block_causal_fallback_matches_the_masked_composed_sdpa(fv, oracle):
    # rt/attn.rs:905-930: S = 24, d = 8, BlockCausal{5, 2, 1}
    announce("rt block-causal fallback 1x2x24x8")
    b, h, s, d = 1, 2, 24, 8
    q = sin_tensor(b * h * s * d, 0.37, (b, h, s, d))
    k = sin_tensor(b * h * s * d, 0.71, (b, h, s, d))
    v = sin_tensor(b * h * s * d, 1.13, (b, h, s, d))
    spec = fv.BlockCausal(5, 2, 1)
    before = fv.rt_stats()
    with fv.with_bf16_act(False):
        got = host(fv.sdpa(dev(q), dev(k), dev(v), fv.Plan.block_causal(None, spec)))
        mask = dev(spec.dense_mask(s, s).reshape(1, 1, s, s))
        want = host(fv.sdpa(dev(q), dev(k), dev(v), fv.Plan.masked(None, mask)))
        dense = host(fv.sdpa(dev(q), dev(k), dev(v), fv.Plan.dense(None)))
    assert np.array_equal(got, want)
    assert not np.array_equal(got[0, 0, 0], dense[0, 0, 0])
    after = fv.rt_stats()
    assert after["masks"] == before["masks"] + 1 and after["composed"] == before["composed"] + 3
    ref = oracle.sdpa_composed(q.reshape(h, s, d), k.reshape(h, s, d), v.reshape(h, s, d),
                               mask=oracle.block_causal_dense_mask(5, 2, 1, s, s))
    assert np.abs(got.reshape(h, s, d) - ref).max() < 2e-6


def test_dense_bf16_act_psnr_vs_f32(fv):
    # rt/attn.rs:986-1002
    import torch

    q = dev(((np.arange(24, dtype=np.float32) * np.float32(0.13)) - np.float32(0.8)).reshape(1, 2, 3, 4))
    with fv.with_bf16_act(False):
        f32_out = fv.sdpa(q, q, q, fv.Plan.dense(None))
    with fv.with_bf16_act(True):
        bf16_out = fv.sdpa(q, q, q, fv.Plan.dense(None))
    assert f32_out.dtype == torch.float32 and bf16_out.dtype == torch.bfloat16
    a, r = host(bf16_out).astype(np.float64), host(f32_out).astype(np.float64)
    rng_ = 2.0 * max(np.abs(r).max(), 1.0)
    psnr = 10 * np.log10(rng_ * rng_ / np.mean((a - r) ** 2))
    assert psnr >= 35.0


@pytest.mark.parametrize("act16", [False, True])
@pytest.mark.parametrize("f32_in", [False, True])
def test_dense_plan_reaches_the_fused_kernel(fv, oracle, act16, f32_in):
    import torch

    b, h, sq, sk, d = 1, 3, 200, 300, 128
    announce(f"rt dense fused act16={act16} f32_in={f32_in}")
    q, k, v = qkv(300, b * h, sq, sk, d)
    shape = lambda x, s: x.reshape(b, h, s, d)
    mk = (lambda x: dev(x)) if f32_in else (lambda x: dev(x).to(torch.bfloat16))
    tq, tk, tv = mk(shape(q, sq)), mk(shape(k, sk)), mk(shape(v, sk))
    before = fv.rt_stats()
    # (fold off: the reference's order for f32 operands, round then scale; bf16 operands never see the switch)
    with fv.with_bf16_act(act16), fv.with_fold_scale(False):
        got = fv.sdpa(tq, tk, tv, fv.Plan.dense(None))
    after = fv.rt_stats()
    assert after["fused"] == before["fused"] + 1 and after["composed"] == before["composed"]
    assert got.dtype == (torch.bfloat16 if act16 else torch.float32) and tuple(got.shape) == (b, h, sq, d)
    # bit-identical to the direct kernel call (G/kernels.rs "default dispatch" check)
    direct = fv.sdpa_dense_bf16(dev(q).to(torch.bfloat16), dev(k).to(torch.bfloat16), dev(v).to(torch.bfloat16),
                                out_bf16=act16)
    torch.cuda.synchronize()
    assert torch.equal(got.reshape(b * h, sq, d), direct)
    assert_parity(host(got).reshape(b * h, sq, d), oracle.sdpa_composed(q, k, v), "rt_dense_fused",
                  max_abs=2e-2 if act16 else 1e-2)


REFERENCE_SHAPES = [  # (b, h, sq, sk, d, std): gpucheck/src/kernels.rs:2287-2298
    (1, 1, 1, 1, 128, 1.0), (1, 2, 64, 64, 128, 1.0), (1, 2, 70, 70, 64, 1.0), (2, 3, 257, 257, 128, 1.0),
    (1, 4, 300, 512, 128, 1.0), (2, 2, 1000, 333, 64, 1.0), (1, 3, 130, 1, 128, 1.0), (1, 2, 63, 4097, 128, 1.0),
    (2, 2, 1024, 1024, 128, 2.0), (1, 2, 2048, 2048, 128, 1.0),
]


@pytest.mark.parametrize("b,h,sq,sk,d,std", REFERENCE_SHAPES)
def test_f32_operands_meet_the_reference_bars_in_the_default_order(fv, oracle, b, h, sq, sk, d, std):
    """The reference's own check of its fused kernel (gpucheck/src/kernels.rs:2286-2328), as it would run against this
    library: f32 tensors of N(0, std) go to the one entry, which rounds them to bf16 itself; the f32 result is
    compared with the host math on the f32 operands (rel_l2 <= 1e-2) AND on the operands rounded to bf16 the plain
    way (<= 2e-3), the bf16 result with the former (<= 1e-2). The default (round, then scale) meets all three; with
    the scale folded into q's rounding the first and third hold as well, the second cannot (a different rounding of
    q than the one it assumes) and is only reported."""
    import torch

    announce(f"rt sdpa on f32 operands, reference bars, {b}x{h}x{sq}x{sk}x{d} std={std}")
    rng = np.random.Generator(np.random.PCG64(2286 + sq + d))
    q = rng.standard_normal((b * h, sq, d), dtype=np.float32) * np.float32(std)
    k = rng.standard_normal((b * h, sk, d), dtype=np.float32) * np.float32(std)
    v = rng.standard_normal((b * h, sk, d), dtype=np.float32)
    want = oracle.sdpa_f64(q, k, v)
    want_rounded = oracle.sdpa_f64(*(oracle.quantize_bf16(x) for x in (q, k, v)))
    tq, tk, tv = (dev(x.reshape(b, h, -1, d)) for x in (q, k, v))
    host = lambda t: t.float().cpu().numpy().reshape(b * h, sq, d)
    assert not fv.fold_scale()
    with fv.with_bf16_act(False):
        got = host(fv.sdpa(tq, tk, tv, fv.Plan.dense(None)))
        with fv.with_fold_scale(True):
            folded = host(fv.sdpa(tq, tk, tv, fv.Plan.dense(None)))
    with fv.with_bf16_act(True):
        got16 = host(fv.sdpa(tq, tk, tv, fv.Plan.dense(None)))
    torch.cuda.synchronize()
    m_f32, m_rounded, m16 = metrics(got, want), metrics(got, want_rounded), metrics(got16, want)
    f_f32, f_rounded = metrics(folded, want), metrics(folded, want_rounded)
    print(f"[reference bars] vs f32 operands {m_f32['rel_l2']:.3e} (folded {f_f32['rel_l2']:.3e}), vs rounded operands "
          f"{m_rounded['rel_l2']:.3e} (folded {f_rounded['rel_l2']:.3e}), bf16 result {m16['rel_l2']:.3e}", flush=True)
    assert m_f32["rel_l2"] <= 1e-2 and m_rounded["rel_l2"] <= 2e-3 and m16["rel_l2"] <= 1e-2
    assert f_f32["rel_l2"] <= 1e-2


@pytest.mark.parametrize("kind", ["dense", "dense_scale", "block_causal", "kv_window"])
def test_f32_queries_take_the_scale_into_their_one_rounding(fv, oracle, kind):
    """An f32 q is rounded to bf16 by the library itself (rt/sdpa.rs:167-181): with the fold switch on (opt-in) that
    one rounding is of q * scale * log2(e) and the kernel runs its form for scale = ln 2. Checked: the launch counter
    of that form moves; the result IS the kernel-level call on bf16(q * c) at ln 2, bit for bit; against the fp32
    host math on the UNROUNDED q at the plan's scale it is inside the tolerance and as close as the unfolded order
    (round, then scale) is; bf16 queries give the same bits whatever the switch says."""
    import torch

    b, h, sq, sk, d = 1, 4, 700, 1100, 128
    announce(f"rt fold scale into f32 q, {kind}")
    rng = np.random.Generator(np.random.PCG64(4100))
    qn = rng.standard_normal((b * h, sq, d), dtype=np.float32)                 # NOT bf16 numbers
    kn, vn = (oracle.quantize_bf16(rng.standard_normal((b * h, sk, d), dtype=np.float32)) for _ in range(2))
    if kind in ("block_causal", "kv_window"):
        sk = sq if kind == "block_causal" else sk
        kn, vn = kn[:, :sk].copy(), vn[:, :sk].copy()
    scale = 0.11 if kind == "dense_scale" else None
    sc = np.float32(scale if scale is not None else 1.0 / np.sqrt(d))
    bc = fv.BlockCausal(100, 3, 1)
    plan = {"dense": fv.Plan.dense(None), "dense_scale": fv.Plan.dense(scale), "block_causal": fv.Plan.block_causal(None, bc),
            "kv_window": fv.Plan.kv_window()}[kind]
    tq = dev(qn.reshape(b, h, sq, d))
    tk, tv = (dev(x.reshape(b, h, sk, d)).to(torch.bfloat16) for x in (kn, vn))
    lib = fv.lib()
    with fv.with_bf16_act(False):
        n0 = lib.fv_sdpa_log2_domain_launches()
        with fv.with_fold_scale(True):
            folded = fv.sdpa(tq, tk, tv, plan)
        assert lib.fv_sdpa_log2_domain_launches() == n0 + 1
        with fv.with_fold_scale(False):
            plain = fv.sdpa(tq, tk, tv, plan)
        assert lib.fv_sdpa_log2_domain_launches() == n0 + 1
        assert not fv.fold_scale()                                            # the default is the reference's order
        # bf16 queries: the switch changes nothing
        q16 = tq.to(torch.bfloat16)
        with fv.with_fold_scale(True):
            a = fv.sdpa(q16, tk, tv, plan)
        with fv.with_fold_scale(False):
            c = fv.sdpa(q16, tk, tv, plan)
        assert torch.equal(a, c) and torch.equal(c, plain)                    # ... and is the unfolded f32-q call
        assert lib.fv_sdpa_log2_domain_launches() == n0 + 1
    # the kernel-level call the folded route makes
    cmul = float(np.float32(sc * np.float32(1.4426950408889634)))
    qc = fv.cast_f32_bf16(tq.reshape(b * h, sq, d), mul=cmul)
    assert torch.equal(qc, (tq.reshape(b * h, sq, d) * cmul).to(torch.bfloat16))   # one product in f32, one rounding
    ln2 = float(np.float32(np.log(2.0)))
    k3, v3 = tk.reshape(b * h, sk, d), tv.reshape(b * h, sk, d)
    # (dense routes split the keys when the query tiles alone do not fill the GPU: the same choice here)
    direct = (fv.sdpa_block_causal_bf16(qc, k3, v3, 100, 3, 1, scale=ln2) if kind == "block_causal"
              else fv.sdpa_dense_bf16_splitkv(qc, k3, v3, splits=None, scale=ln2))
    torch.cuda.synchronize()
    assert torch.equal(folded.reshape(b * h, sq, d), direct)
    # against the host math on the f32 q
    want = oracle.sdpa_composed_rows(qn, kn, vn, np.arange(sq), scale=float(sc),
                                     mask_bc=(100, 3, 1) if kind == "block_causal" else None)
    mf = assert_parity(host(folded).reshape(b * h, sq, d), want, f"rt_fold_{kind}", max_rel_l2=1e-2)
    mp = assert_parity(host(plain).reshape(b * h, sq, d), want, f"rt_unfolded_{kind}", max_rel_l2=1e-2)
    assert mf["rel_l2"] <= 1.1 * mp["rel_l2"], (mf, mp)


def test_backend_setting_steers_the_dense_route(fv, oracle):
    """FASTVIDEO_SDPA (rt/sdpa_rule.rs:199-219, 409-437; rt/sdpa.rs:225-246): cublas / flash take the
    f32-score kernel instead of the fused one, host / sparse are retired and refuse the call."""
    import torch

    b, h, sq, sk, d = 1, 2, 130, 190, 128
    announce("rt backend routes")
    q, k, v = qkv(310, b * h, sq, sk, d)
    tq, tk, tv = (dev(x.reshape(b, h, -1, d)).to(torch.bfloat16) for x in (q, k, v))
    want = oracle.sdpa_composed(q, k, v)
    for name in ("cublas", "flash"):
        before = fv.rt_stats()
        with fv.with_backend(name), fv.with_bf16_act(False):
            got = fv.sdpa(tq, tk, tv, fv.Plan.dense(None))
        after = fv.rt_stats()
        assert after["fused"] == before["fused"] and after["composed"] == before["composed"] + 1
        assert_parity(host(got).reshape(b * h, sq, d), want, f"rt_backend_{name}", max_abs=1e-5)
    for name, needle in (("host", "retired"), ("sparse", "FASTVIDEO_VSA=1")):
        with fv.with_backend(name), pytest.raises(fv.TensorError, match=needle):
            fv.sdpa(tq, tk, tv, fv.Plan.dense(None))
    before = fv.rt_stats()
    fv.sdpa(tq, tk, tv, fv.Plan.dense(None))
    assert fv.rt_stats()["fused"] == before["fused"] + 1


@pytest.mark.parametrize("b,h,sq,sk,d", [(1, 4, 256, 256, 128), (1, 4, 256, 77, 128), (2, 2, 130, 130, 64), (1, 2, 96, 96, 80)])
@pytest.mark.parametrize("act16", [False, True])
def test_every_plan_the_families_call_runs_on_the_device(fv, oracle, b, h, sq, sk, d, act16):
    """gpucheck/src/kernels.rs:2813-2897, as it would run against this library: every plan the model families build
    (dense, dense with fp8_first, masked with a zero mask, both KV-window forms, block-causal and the VDN window where
    the shape allows), f32 tensors in, f32 and bf16 activations, the fused head dims and one the fused kernels
    decline (d = 80): each call succeeds with a device-resident result of the context's dtype; here the values are
    checked too, against the host math under the plan's mask."""
    import torch

    announce(f"rt every plan {b}x{h}x{sq}x{sk}x{d} act16={act16}")
    q, k, v = qkv(2813 + sq + sk + d, b * h, sq, sk, d, round_bf16=False)
    t4 = lambda x, s: dev(x.reshape(b, h, s, d))
    tq, tk, tv = t4(q, sq), t4(k, sk), t4(v, sk)
    zero_mask = torch.zeros((1, 1, sq, sk), device="cuda", dtype=torch.float32)
    plans = [("dense", fv.Plan.dense(None), None), ("dense_fp8_first", fv.Plan.dense(None).fp8_first(), None),
             ("masked", fv.Plan.masked(None, zero_mask), None), ("kv_window", fv.Plan.kv_window(), None),
             ("kv_window_reference", fv.Plan.kv_window_with(False), None)]
    if sq == sk:
        plans.append(("block_causal", fv.Plan.block_causal(None, fv.BlockCausal(64, 0, 0)),
                      oracle.block_causal_dense_mask(64, 0, 0, sq, sk)))
    if sq == sk and d == 128:
        plans.append(("vdn_window", fv.Plan.vdn_window(None, fv.VdnWindow(16, 16, 15, 0, 1)),
                      oracle.vdn_window_dense_mask(16, 16, 15, 0, 1, sq, sk)))
    for name, plan, mask in plans:
        with fv.with_bf16_act(act16):
            out = fv.sdpa(tq, tk, tv, plan)
        torch.cuda.synchronize()
        assert out.is_cuda and tuple(out.shape) == (b, h, sq, d), name
        assert out.dtype == (torch.bfloat16 if act16 else torch.float32), name
        want = oracle.sdpa_composed(q, k, v, mask=mask)
        m = metrics(out.float().cpu().numpy().reshape(b * h, sq, d), want)
        print(f"[every plan] {name}: rel_l2 {m['rel_l2']:.3e} max_abs {m['max_abs']:.2e}", flush=True)
        assert m["rel_l2"] <= 1e-2 and m["cosine"] >= 0.9999, (name, m)


def test_block_causal_and_kv_window_plans_at_d128(fv, oracle):
    import torch

    b, h, s, d, bt = 1, 2, 384, 128, 96
    announce("rt block-causal / kv-window d128")
    q, k, v = qkv(400, b * h, s, s, d)
    t4 = lambda x: dev(x.reshape(b, h, s, d)).to(torch.bfloat16)
    before = fv.rt_stats()
    with fv.with_bf16_act(False):
        got = fv.sdpa(t4(q), t4(k), t4(v), fv.Plan.block_causal(None, fv.BlockCausal(bt, 0, 0)))
        kvw = fv.sdpa(t4(q)[:, :, :100].contiguous(), t4(k), t4(v), fv.Plan.kv_window())
        kvc = fv.sdpa(t4(q)[:, :, :100].contiguous(), t4(k), t4(v), fv.Plan.kv_window_with(False))
    after = fv.rt_stats()
    assert after["causal"] == before["causal"] + 1 and after["masks"] == before["masks"]
    want = oracle.sdpa_composed(q, k, v, mask=oracle.block_causal_dense_mask(bt, 0, 0, s, s))
    assert_parity(host(got).reshape(b * h, s, d), want, "rt_block_causal")
    wantw = oracle.sdpa_composed(q[:, :100], k, v)
    assert_parity(host(kvw).reshape(b * h, 100, d), wantw, "rt_kv_window_flash")
    assert np.abs(host(kvc).reshape(b * h, 100, d) - wantw).max() < 1e-5


@pytest.mark.parametrize("bh,sq,sk,d,mask_kind", [(2, 5, 7, 8, None), (3, 33, 300, 64, "shared"), (2, 40, 257, 128, "per_bh"),
                                                  (1, 3, 1000, 256, None), (2, 64, 64, 128, "shared"), (1, 2, 1, 128, None),
                                                  # the f32 matrix-core kernel: every head dim it takes, query / key tails,
                                                  # one and many key tiles, more than one workgroup per head
                                                  (2, 300, 515, 32, "shared"), (3, 129, 31, 96, None), (2, 257, 1025, 96, "per_bh"),
                                                  (1, 128, 32, 128, None), (2, 700, 333, 128, "shared"), (4, 1, 65, 64, "per_bh"),
                                                  (1, 384, 2048, 128, None)])
def test_composed_kernel_vs_oracle(fv, oracle, bh, sq, sk, d, mask_kind):
    import ctypes
    import torch

    announce(f"composed f32 bh={bh} sq={sq} sk={sk} d={d} mask={mask_kind}")
    q, k, v = qkv(500 + sq, bh, sq, sk, d, round_bf16=False)
    mask = None
    if mask_kind == "shared":
        mask = oracle.block_causal_dense_mask(max(sk // 5, 1), 0, 1, sq, sk)
    elif mask_kind == "per_bh":
        mask = (randn(7, (bh, sq, sk)) * 2).astype(np.float32)
    tq, tk, tv = dev(q), dev(k), dev(v)
    tm = dev(mask) if mask is not None else None
    out = torch.empty((bh, sq, d), device="cuda", dtype=torch.float32)
    scale = 1.0 / np.sqrt(d)
    rc = fv.lib().fv_sdpa_composed_f32(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), tm.data_ptr() if tm is not None else None,
                                       int(mask_kind == "per_bh"), out.data_ptr(), bh, sq, sk, d, scale,
                                       torch.cuda.current_stream().cuda_stream)
    assert rc == 0, fv.lib().fv_sdpa_last_error()
    if mask_kind == "per_bh":
        want = np.stack([oracle.sdpa_composed(q[i:i + 1], k[i:i + 1], v[i:i + 1], mask=mask[i])[0] for i in range(bh)])
    else:
        want = oracle.sdpa_composed(q, k, v, mask=mask)
    m = metrics(host(out), want)
    print(m)
    assert m["max_abs"] < 2e-5


def test_allocation_failure_is_reported_with_its_own_code_and_leaves_the_device_usable(fv):
    """A result larger than the device's memory: `sdpa` fails at its first allocation, before any
    launch (the operand descriptors claim 130 M query rows; nothing ever reads them), with the
    out-of-memory code rather than the code of a refused argument, and the next call works."""
    import ctypes
    import torch

    from fv_sdpa.sdpa import _FvPlan, _FvTensor

    announce("rt allocation failure, 12 x 130e6 x 128 bf16 result (400 GB)")
    buf = torch.zeros((1, 12, 256, 128), device="cuda", dtype=torch.bfloat16)

    def desc(rows):
        t = _FvTensor()
        t.data, t.dtype, t.rank, t.plane_rows = buf.data_ptr(), 1, 4, 0
        for i, s in enumerate((1, 12, rows, 128)):
            t.shape[i] = s
        return t

    lib = fv.lib()
    p = _FvPlan()
    p.kind, p.kv_flash = 0, -1
    out = _FvTensor()
    q, kv = desc(130_000_000), desc(256)
    rc = lib.fv_rt_sdpa(ctypes.byref(q), ctypes.byref(kv), ctypes.byref(kv), ctypes.byref(p), ctypes.byref(out),
                        torch.cuda.current_stream().cuda_stream)
    msg = lib.fv_sdpa_last_error().decode()
    print(f"rc={rc} message={msg!r}")
    assert rc == -2 and msg.startswith("sdpa: device allocation failed: ")      # hipErrorOutOfMemory
    got = fv.sdpa(buf, buf, buf, fv.Plan.dense(None))
    torch.cuda.synchronize()
    assert got.shape == buf.shape and torch.isfinite(got.float()).all()


def test_first_use_of_a_kernel_on_a_shape_is_logged_once():
    """rt/attn.rs:306-310 + rt/log.rs: at FASTVIDEO_LOG=info the entry names the kernel it launched, once per
    (kernel, shape); FASTVIDEO_LOG=0 is quiet. Run in child processes (the level is read once per process)."""
    import os
    import subprocess
    import sys

    from util import PKG, ROOT

    announce("rt first-use log lines")
    code = (
        "import sys; sys.path[:0] = %r\n"
        "import torch, fv_sdpa\n"
        "x = torch.randn((1, 2, 300, 128), device='cuda').to(torch.bfloat16)\n"
        "y = torch.randn((1, 2, 200, 128), device='cuda').to(torch.bfloat16)\n"
        "z = torch.randn((1, 2, 40, 48), device='cuda')\n"
        "for _ in range(3):\n"
        "    fv_sdpa.sdpa(x, x, x, fv_sdpa.Plan.dense(None))\n"
        "    fv_sdpa.sdpa(x, y, y, fv_sdpa.Plan.dense(None))\n"
        "    fv_sdpa.sdpa(x, x, x, fv_sdpa.Plan.block_causal(None, fv_sdpa.BlockCausal(100, 0, 0)))\n"
        "    fv_sdpa.sdpa(z, z, z, fv_sdpa.Plan.dense(None))\n"
        "torch.cuda.synchronize()\n" % [ROOT, PKG])

    def run(level):
        env = dict(os.environ)
        env["FASTVIDEO_LOG"] = level
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        return [ln for ln in r.stderr.splitlines() if ln.startswith("[fastvideo] sdpa:")]

    lines = run("info")
    assert lines == ["[fastvideo] sdpa: fused mma B=1 H=2 Sq=300 Sk=300 D=128",
                     "[fastvideo] sdpa: fused mma B=1 H=2 Sq=300 Sk=200 D=128",
                     "[fastvideo] sdpa: fused mma block-causal B=1 H=2 Sq=300 Sk=300 D=128",
                     "[fastvideo] sdpa: composed f32 B=1 H=2 Sq=40 Sk=40 D=48"], lines
    assert run("0") == []
