"""The split-KV entry that allocates nothing (`fv_sdpa_dense_bf16_splitkv_static`: partials in a buffer inside
the library's code object) against the entry it is a variant of (`fv_sdpa_dense_bf16_splitkv`, partials in a
caller workspace): same kernels, same split count, so the outputs are bit-identical. Two calls in a row share
the one buffer, the second on a smaller input; then the refusals."""
import numpy as np
import pytest

from util import announce, assert_parity, qkv, to_dev_bf16

pytestmark = pytest.mark.gpu


def _both(lib, torch, q, k, v, splits, out_bf16):
    """(static entry's output, workspace entry's output) on contiguous [bh, s, d] bf16 operands."""
    bh, sq, d = q.shape
    sk = k.shape[1]
    stream = torch.cuda.current_stream().cuda_stream
    dt = torch.bfloat16 if out_bf16 else torch.float32
    got = torch.full((bh, sq, d), float("nan"), device="cuda", dtype=dt)
    want = torch.full((bh, sq, d), float("nan"), device="cuda", dtype=dt)
    nbytes = int(lib.fv_sdpa_splitkv_workspace_bytes(bh, sq, d, splits))
    ws = torch.empty(max(nbytes, 256), device="cuda", dtype=torch.uint8)
    scale = float(d) ** -0.5
    rc = lib.fv_sdpa_dense_bf16_splitkv_static(q.data_ptr(), k.data_ptr(), v.data_ptr(), got.data_ptr(), int(out_bf16), bh,
                                               sq, sk, d, scale, 0, 0, 0, splits, stream)
    assert rc == 0, lib.fv_sdpa_last_error().decode()
    rc = lib.fv_sdpa_dense_bf16_splitkv(q.data_ptr(), k.data_ptr(), v.data_ptr(), want.data_ptr(), int(out_bf16), bh, sq,
                                        sk, d, scale, 0, 0, 0, splits, ws.data_ptr(), nbytes, stream)
    assert rc == 0, lib.fv_sdpa_last_error().decode()
    torch.cuda.synchronize()
    return got, want


def test_static_buffer_entry_equals_the_workspace_entry_on_two_calls_in_a_row(oracle):
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    lib = fv_sdpa.lib()
    assert lib.fv_sdpa_init() == 0
    cap = int(lib.fv_sdpa_splitkv_static_bytes())
    assert cap == 32 << 20
    # first call: a one-frame block of causal generation against a long cache (the shape the entry is for),
    # 3 splits: 29 MB of the 32 MiB buffer
    bh, sq, sk, d, splits = 12, 1560, 8192, 128, 3
    assert int(lib.fv_sdpa_splitkv_workspace_bytes(bh, sq, d, splits)) <= cap
    announce(f"no-alloc splitkv first call bh={bh} sq={sq} sk={sk} splits={splits} seed=5100")
    q, k, v = qkv(5100, bh, sq, sk, d)
    tq, tk, tv = (to_dev_bf16(x) for x in (q, k, v))
    got, want = _both(lib, torch, tq, tk, tv, splits, False)
    assert torch.isfinite(got).all() and torch.equal(got, want)
    rows = np.array([0, 255, 256, 777, sq - 1])
    assert_parity(got[:, torch.from_numpy(rows).cuda()].cpu().numpy(), oracle.sdpa_composed_rows(q, k, v, rows),
                  "no_alloc_first_call")
    # second call, smaller: the buffer still holds the first call's partials beyond what this one writes
    bh2, sq2, sk2, splits2 = 3, 257, 2049, 5
    announce(f"no-alloc splitkv second call bh={bh2} sq={sq2} sk={sk2} splits={splits2} seed=5200")
    q2, k2, v2 = qkv(5200, bh2, sq2, sk2, d)
    t2 = [to_dev_bf16(x) for x in (q2, k2, v2)]
    for out_bf16 in (False, True):
        got2, want2 = _both(lib, torch, *t2, splits2, out_bf16)
        assert torch.isfinite(got2.float()).all() and torch.equal(got2, want2)
    got2, _ = _both(lib, torch, *t2, splits2, False)
    assert_parity(got2.cpu().numpy(), oracle.sdpa_composed(q2, k2, v2), "no_alloc_second_call")
    # the library's own choice of the split count (splits = 0), head dim 64, and the unsplit route (splits = 1)
    q3, k3, v3 = qkv(5300, 2, 100, 3000, 64)
    t3 = [to_dev_bf16(x) for x in (q3, k3, v3)]
    for splits3 in (0, 1, 4):
        stream = torch.cuda.current_stream().cuda_stream
        got3 = torch.full((2, 100, 64), float("nan"), device="cuda")
        rc = lib.fv_sdpa_dense_bf16_splitkv_static(t3[0].data_ptr(), t3[1].data_ptr(), t3[2].data_ptr(), got3.data_ptr(), 0,
                                                   2, 100, 3000, 64, 0.125, 0, 0, 0, splits3, stream)
        assert rc == 0, lib.fv_sdpa_last_error().decode()
        torch.cuda.synchronize()
        assert_parity(got3.cpu().numpy(), oracle.sdpa_composed(q3, k3, v3), f"no_alloc_d64_splits{splits3}")


def test_static_buffer_entry_steps_its_own_choice_down_to_what_fits(oracle):
    """splits == 0 at a shape whose chosen count (16) would need 262 144 bytes more than the buffer holds:
    the entry runs 15 splits instead of refusing, bit-identical to the workspace entry at 15."""
    import torch

    import fv_sdpa

    lib = fv_sdpa.lib()
    bh, sq, sk, d = 1, 4096, 32760, 128
    assert int(lib.fv_sdpa_splitkv_choose(bh, sq, sk)) == 16
    assert int(lib.fv_sdpa_splitkv_workspace_bytes(bh, sq, d, 16)) > int(lib.fv_sdpa_splitkv_static_bytes())
    assert int(lib.fv_sdpa_splitkv_static_splits(bh, sq, sk, d, 0)) == 15
    announce(f"no-alloc splitkv stepped-down choice bh={bh} sq={sq} sk={sk} seed=5400")
    q, k, v = qkv(5400, bh, sq, sk, d)
    tq, tk, tv = (to_dev_bf16(x) for x in (q, k, v))
    stream = torch.cuda.current_stream().cuda_stream
    got = torch.full((bh, sq, d), float("nan"), device="cuda")
    rc = lib.fv_sdpa_dense_bf16_splitkv_static(tq.data_ptr(), tk.data_ptr(), tv.data_ptr(), got.data_ptr(), 0, bh, sq, sk, d,
                                               float(d) ** -0.5, 0, 0, 0, 0, stream)
    assert rc == 0, lib.fv_sdpa_last_error().decode()
    _, want = _both(lib, torch, tq, tk, tv, 15, False)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    rows = np.array([0, 1, 255, 256, 2047, sq - 1])
    assert_parity(got[:, torch.from_numpy(rows).cuda()].cpu().numpy(), oracle.sdpa_composed_rows(q, k, v, rows),
                  "no_alloc_stepped_down")


def test_static_buffer_entry_refuses_what_does_not_fit():
    import torch

    import fv_sdpa

    lib = fv_sdpa.lib()
    cap = int(lib.fv_sdpa_splitkv_static_bytes())
    bh, sq, sk, d, splits = 12, 1560, 8192, 128, 4           # 38 MB of partials
    assert int(lib.fv_sdpa_splitkv_workspace_bytes(bh, sq, d, splits)) > cap
    x = torch.zeros((bh, sk, d), device="cuda", dtype=torch.bfloat16)
    out = torch.full((bh, sq, d), 7.0, device="cuda")
    rc = lib.fv_sdpa_dense_bf16_splitkv_static(x.data_ptr(), x.data_ptr(), x.data_ptr(), out.data_ptr(), 0, bh, sq, sk, d,
                                               0.088, 0, 0, 0, splits, torch.cuda.current_stream().cuda_stream)
    msg = lib.fv_sdpa_last_error().decode()
    torch.cuda.synchronize()
    assert rc == -1 and "static buffer holds 33554432" in msg, (rc, msg)
    assert (out == 7.0).all()                                 # nothing was launched
    rc = lib.fv_sdpa_dense_bf16_splitkv_static(x.data_ptr(), x.data_ptr(), x.data_ptr(), out.data_ptr(), 0, bh, sq, sk, 96,
                                               0.088, 0, 0, 0, 2, torch.cuda.current_stream().cuda_stream)
    assert rc == 1                                            # declined: head dim 96
