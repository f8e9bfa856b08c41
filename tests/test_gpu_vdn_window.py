"""Parity of the flash kernel under the VDN-H3 window mask (through the C ABI and through
Plan::vdn_window) against the oracle's masked composed fp32 SDPA on identical bf16-valued
inputs: max|delta| <= 1e-2, cosine >= 0.9999. Cases cover both window forms (chunk-aligned,
centred), videos that start and end inside / at the ends of the sequence, frames that do and
do not align with the 64-key tiles and the 256-query workgroups, windows that merge with the
anchor ranges, and the degenerate clips (1-2 frames, radius past the clip) that are dense.
"""
import numpy as np
import pytest

from util import announce, assert_bf16_result_matches_f32_result, assert_parity, qkv, to_dev_bf16

pytestmark = pytest.mark.gpu

CASES = [  # (bh, s, video_start, frame_tokens, frames, chunk, radius, d)
    (4, 256, 16, 16, 15, 0, 1, 128),      # the reference's own plan case (gpucheck kernels.rs:2860-2868)
    (2, 1300, 20, 40, 32, 5, 1, 128),     # chunk 5 / radius 1, text rows on both sides
    (2, 2048, 0, 64, 32, 5, 1, 128),      # frames = tiles, video fills the sequence
    (1, 2100, 52, 128, 16, 0, 2, 128),    # frames of two tiles, centred window
    (2, 1536, 0, 256, 6, 0, 1, 128),      # frame = workgroup: inner query tiles walk 3 ranges
    (1, 3000, 100, 100, 29, 4, 0, 128),   # radius 0: own chunk only
    (2, 900, 7, 33, 27, 3, 1, 64),        # ragged everything, head dim 64
    (1, 4200, 64, 192, 21, 5, 1, 128),    # detached window, anchors and tail all separate ranges
    (2, 700, 10, 50, 2, 5, 1, 128),       # two frames: both anchors, dense
    (2, 700, 10, 50, 13, 2, 40, 128),     # radius past the clip: every frame visible
    (1, 515, 3, 1, 500, 7, 2, 128),       # one-token frames
]


@pytest.fixture(scope="module")
def fv():
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


@pytest.mark.parametrize("bh,s,vs,t,frames,chunk,radius,d", CASES)
def test_vdn_window_matches_masked_oracle(fv, oracle, bh, s, vs, t, frames, chunk, radius, d):
    import torch

    announce(f"vdn window bh={bh} s={s} video={vs}+{frames}x{t} chunk={chunk} radius={radius} d={d}")
    q, k, v = qkv(7000 + s + chunk, bh, s, s, d)
    mask = oracle.vdn_window_dense_mask(vs, t, frames, chunk, radius, s, s)
    want = oracle.sdpa_composed(q, k, v, mask=mask)
    qd, kd, vd = (to_dev_bf16(x) for x in (q, k, v))
    got = fv.sdpa_vdn_window_bf16(qd, kd, vd, vs, t, frames, chunk, radius)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert_parity(got, want, f"vdn_{s}_{vs}_{t}x{frames}_c{chunk}_r{radius}")
    got16 = fv.sdpa_vdn_window_bf16(qd, kd, vd, vs, t, frames, chunk, radius, out_bf16=True)
    torch.cuda.synchronize()
    # (the bf16 launch keeps its softmax offset fixed after the first 128 keys, the f32 one follows the running max)
    assert_bf16_result_matches_f32_result(got16.float().cpu().numpy(), got, f"vdn_{s}_{vs}_{t}x{frames}", exact_share=0.999)


def test_fixed_offset_pass_under_the_window_and_its_rerun(fv, oracle):
    """Every query sees key 0 under this mask (rows before the video and frame 0 are visible to all), so launches
    that write bf16 fix each query's softmax offset at the largest score of its walk's first 128 keys and redo the
    pass with the running max where a row outgrew it. Head 0's scores climb by hundreds of base-2 units along the
    keys: its workgroups take the second pass (counted), every row matches the masked f32 host math, and the other
    head is the bits of a launch on its own."""
    import torch

    bh, s, d = 2, 1300, 128
    vs, t, frames, chunk, radius = 20, 40, 32, 5, 1
    announce("vdn window fixed-offset pass and its rerun")
    rng = np.random.Generator(np.random.PCG64(909))
    q = rng.standard_normal((bh, s, d)).astype(np.float32)
    k = rng.standard_normal((bh, s, d)).astype(np.float32)
    v = oracle.quantize_bf16(rng.standard_normal((bh, s, d)).astype(np.float32))
    q[0] = np.abs(q[0]) + 2.0
    k[0, :128] = -0.5
    k[0, 128:] = np.linspace(1.0, 30.0, s - 128, dtype=np.float32)[:, None]
    q, k = oracle.quantize_bf16(q), oracle.quantize_bf16(k)
    tq, tk, tv = (to_dev_bf16(x) for x in (q, k, v))
    lib = fv.lib()
    n0 = lib.fv_sdpa_exact_pass_reruns()
    got = fv.sdpa_vdn_window_bf16(tq, tk, tv, vs, t, frames, chunk, radius, out_bf16=True)
    torch.cuda.synchronize()
    n1 = lib.fv_sdpa_exact_pass_reruns()
    assert n1 - n0 == (s + 255) // 256, (n0, n1)       # every query tile of head 0 sees keys past its first 128
    mask = oracle.vdn_window_dense_mask(vs, t, frames, chunk, radius, s, s)
    want = oracle.sdpa_composed(q, k, v, mask=mask)
    assert_parity(got.float().cpu().numpy(), want, "vdn_rerun", max_abs=2e-2)
    rest = fv.sdpa_vdn_window_bf16(tq[1:].contiguous(), tk[1:].contiguous(), tv[1:].contiguous(), vs, t, frames, chunk,
                                   radius, out_bf16=True)
    got32 = fv.sdpa_vdn_window_bf16(tq, tk, tv, vs, t, frames, chunk, radius)
    torch.cuda.synchronize()
    assert lib.fv_sdpa_exact_pass_reruns() == n1 and torch.equal(rest, got[1:])   # f32 results keep the running max
    assert_parity(got32.cpu().numpy(), want, "vdn_running_max")


def test_masked_rows_really_differ_from_dense(fv, oracle):
    import torch

    bh, s, d = 1, 1024, 128
    announce("vdn window vs dense, 1x1024")
    q, k, v = (to_dev_bf16(x) for x in qkv(71, bh, s, s, d))
    dense = fv.sdpa_dense_bf16(q, k, v)
    win = fv.sdpa_vdn_window_bf16(q, k, v, 0, 64, 16, 0, 1)
    torch.cuda.synchronize()
    diff = (dense - win).abs().amax(dim=-1)[0].cpu().numpy()
    assert diff[:64].max() == 0 and diff[-64:].max() == 0      # anchor frames: dense rows, bit for bit
    assert diff[64:-64].min() > 0                               # every inner row lost keys


def test_plan_vdn_window_kernel_and_fallback(fv, oracle):
    import torch

    b, h, s, d = 1, 4, 256, 128
    announce("Plan::vdn_window 1x4x256x128 (reference plan case) and the masked fallback")
    w = fv.VdnWindow(16, 16, 15, 0, 1)
    q, k, v = qkv(72, b * h, s, s, d)
    mask = oracle.vdn_window_dense_mask(16, 16, 15, 0, 1, s, s)
    want = oracle.sdpa_composed(q, k, v, mask=mask)
    qd, kd, vd = (to_dev_bf16(x).reshape(b, h, s, d) for x in (q, k, v))
    before = fv.rt_stats()
    out = fv.sdpa(qd, kd, vd, fv.Plan.vdn_window(None, w))
    torch.cuda.synchronize()
    after = fv.rt_stats()
    assert out.dtype == torch.bfloat16 and tuple(out.shape) == (b, h, s, d)
    assert after["causal"] == before["causal"] + 1
    assert after["composed"] == before["composed"]
    assert_parity(out.float().cpu().numpy().reshape(b * h, s, d), want, "plan_vdn_window", max_abs=2e-2)
    # sq != sk: the kernel declines and the plan falls back to the masked composed path
    qs = qd[:, :, :100].contiguous()
    before = fv.rt_stats()
    out2 = fv.sdpa(qs, kd, vd, fv.Plan.vdn_window(None, w))
    torch.cuda.synchronize()
    after = fv.rt_stats()
    assert after["composed"] == before["composed"] + 1
    assert after["masks"] == before["masks"] + 1
    want2 = oracle.sdpa_composed(q[:, :100], k, v, mask=oracle.vdn_window_dense_mask(16, 16, 15, 0, 1, 100, s))
    assert_parity(out2.float().cpu().numpy().reshape(b * h, 100, d), want2, "plan_vdn_window_fallback", max_abs=2e-2)


def test_declines(fv):
    import torch

    x = torch.zeros((1, 300, 128), device="cuda", dtype=torch.bfloat16)
    y = torch.zeros((1, 200, 128), device="cuda", dtype=torch.bfloat16)
    with pytest.raises(fv.FvDeclined):
        fv.sdpa_vdn_window_bf16(y, x, x, 0, 10, 10)        # sq != sk
    with pytest.raises(fv.FvDeclined):
        fv.sdpa_vdn_window_bf16(x, x, x, 0, 10, 31)        # video past the sequence
    with pytest.raises(fv.FvDeclined):
        fv.sdpa_vdn_window_bf16(x, x, x, 0, 0, 3)          # no frame tokens
