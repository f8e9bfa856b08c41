"""Split-KV form of the dense kernel (few query tiles, many keys): every split count gives the unsplit
kernel's result to rounding (each split normalises by its own row sum, the merge re-weights by the
base-2 log-sum-exp), parity against the fp32 oracle, row windows read in place, the library's own
choice of the split count, and the `fv_rt_sdpa` entry applying it by itself.
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


@pytest.mark.parametrize("d", [128, 64])
@pytest.mark.parametrize("bh,sq,sk", [(2, 100, 3000), (3, 257, 2049), (1, 1, 4096), (4, 300, 1000)])
def test_every_split_count_matches_the_unsplit_kernel(fv, oracle, bh, sq, sk, d):
    import torch

    announce(f"splitkv bh={bh} sq={sq} sk={sk} d={d}")
    q, k, v = qkv(900 + sk + d, bh, sq, sk, d)
    tq, tk, tv = (to_dev_bf16(x) for x in (q, k, v))
    base = fv.sdpa_dense_bf16(tq, tk, tv)
    want = oracle.sdpa_composed(q, k, v)
    for splits in (1, 2, 3, 5, 16, 1000):
        got = fv.sdpa_dense_bf16_splitkv(tq, tk, tv, splits=splits)
        torch.cuda.synchronize()
        if splits == 1:
            assert torch.equal(got, base)
        assert (got - base).abs().max().item() <= 2e-3, splits
        assert_parity(got.cpu().numpy(), want, f"splitkv_{splits}_{bh}_{sq}_{sk}_{d}")
    got16 = fv.sdpa_dense_bf16_splitkv(tq, tk, tv, splits=4, out_bf16=True)
    torch.cuda.synchronize()
    assert (got16.float() - base).abs().max().item() <= 2e-2


def test_many_split_items(fv, oracle):
    """40 heads x 2 query tiles x 8 splits = 640 workgroups of 4 key tiles (several rounds of short
    items), against the unsplit kernel, the oracle, and the same heads in smaller calls."""
    import torch

    bh, sq, sk, d = 40, 300, 2000, 128
    announce(f"splitkv many items bh={bh} sq={sq} sk={sk}")
    q, k, v = qkv(4242, bh, sq, sk, d)
    tq, tk, tv = (to_dev_bf16(x) for x in (q, k, v))
    got = fv.sdpa_dense_bf16_splitkv(tq, tk, tv, splits=8)
    base = fv.sdpa_dense_bf16(tq, tk, tv)
    torch.cuda.synchronize()
    assert (got - base).abs().max().item() <= 2e-3
    heads = np.array([0, 1, 20, 38, 39])
    assert_parity(got[torch.from_numpy(heads).cuda()].cpu().numpy(), oracle.sdpa_composed(q[heads], k[heads], v[heads]),
                  "splitkv_many_items")
    # the same heads in smaller calls: bit-identical partials and merge
    for lo in range(0, bh, 10):
        part = fv.sdpa_dense_bf16_splitkv(tq[lo:lo + 10].contiguous(), tk[lo:lo + 10].contiguous(),
                                          tv[lo:lo + 10].contiguous(), splits=8)
        assert torch.equal(part, got[lo:lo + 10])


def test_choice_and_windows(fv, oracle):
    import torch

    # a one-frame block of Self-Forcing generation against a 21-frame cache: 7 query tiles x 12 heads
    bh, sq, sk, d = 12, 1560, 32760, 128
    splits = fv.splitkv_choose(bh, sq, sk)
    announce(f"splitkv choice bh={bh} sq={sq} sk={sk}: {splits}")
    assert 2 <= splits <= 16
    assert fv.splitkv_choose(12, 32760, 32760) == 1 and fv.splitkv_choose(12, 4680, 32760) == 1
    assert fv.splitkv_choose(12, 1560, 512) == 1          # too few key tiles to share out
    g = torch.Generator(device="cuda").manual_seed(4)
    cache_k = torch.randn((bh, sk + 500, d), generator=g, device="cuda").to(torch.bfloat16)
    cache_v = torch.randn((bh, sk + 500, d), generator=g, device="cuda").to(torch.bfloat16)
    q = torch.randn((bh, sq, d), generator=g, device="cuda").to(torch.bfloat16)
    kw, vw = cache_k[:, 100:100 + sk], cache_v[:, 100:100 + sk]      # row windows, read in place
    got = fv.sdpa_dense_bf16_splitkv(q, kw, vw)
    base = fv.sdpa_dense_bf16_windows(q, kw, vw)
    torch.cuda.synchronize()
    assert (got - base).abs().max().item() <= 2e-3
    # the plan entry picks the split form by itself for such a shape, and stays within the kernel bar
    t4 = lambda x: x.reshape(1, *x.shape)  # noqa: E731
    with fv.with_bf16_act(False):
        via_plan = fv.sdpa(t4(q), t4(cache_k)[:, :, 100:100 + sk], t4(cache_v)[:, :, 100:100 + sk], fv.Plan.kv_window())
    torch.cuda.synchronize()
    assert torch.equal(via_plan.reshape(bh, sq, d), got)
    with pytest.raises(fv.FvError):
        ws = torch.empty(256, device="cuda", dtype=torch.uint8)
        fv.lib().fv_sdpa_dense_bf16_splitkv.restype  # noqa: B018
        fv._lib.check(fv.lib().fv_sdpa_dense_bf16_splitkv(q.data_ptr(), kw.data_ptr(), vw.data_ptr(), got.data_ptr(), 0, bh, sq,
                                                          sk, d, 0.088, 0, sk + 500, sk + 500, 4, ws.data_ptr(), 256,
                                                          torch.cuda.current_stream().cuda_stream))
