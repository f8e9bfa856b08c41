"""The library is driven from several host threads at once, each on its own HIP stream (the reference
spawns one thread per rank, rt/device.rs:65-71): results equal the single-threaded ones bit for bit,
and a failing call's message stays with the thread that made it."""
import threading

import pytest

from util import announce

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fv():
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    fv_sdpa.lib()
    return fv_sdpa


def test_concurrent_threads_on_their_own_streams(fv):
    import torch

    announce("threads x streams")
    shapes = [(3, 700, 900, 128, 0), (2, 513, 513, 64, 0), (4, 300, 1200, 128, 100), (2, 1024, 1024, 128, 256)]
    g = torch.Generator(device="cuda").manual_seed(8)
    data, want = [], []
    for bh, sq, sk, d, bt in shapes:
        q = torch.randn((bh, sq, d), generator=g, device="cuda").to(torch.bfloat16)
        k = torch.randn((bh, sk, d), generator=g, device="cuda").to(torch.bfloat16)
        v = torch.randn((bh, sk, d), generator=g, device="cuda").to(torch.bfloat16)
        data.append((q, k, v, bt))
        want.append(fv.sdpa_block_causal_bf16(q, k, v, bt, 0, 0) if bt else fv.sdpa_dense_bf16(q, k, v))
    torch.cuda.synchronize()
    errors, msgs = [], {}

    def worker(i):
        try:
            q, k, v, bt = data[i]
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for rep in range(20):
                    got = fv.sdpa_block_causal_bf16(q, k, v, bt, 0, 0) if bt else fv.sdpa_dense_bf16(q, k, v)
                    if rep % 5 == i:      # a declined call in between: its message belongs to this thread
                        try:
                            fv.sdpa_dense_bf16(q, k, v, scale=-1.0 - i)
                        except fv.FvDeclined as e:
                            msgs[i] = str(e)
                stream.synchronize()
            if not torch.equal(got, want[i]):
                errors.append(f"thread {i}: result differs")
            if fv.lib().fv_sdpa_last_error() != b"sdpa: the fused kernel needs a finite scale > 0":
                errors.append(f"thread {i}: last error {fv.lib().fv_sdpa_last_error()!r}")
        except Exception as e:  # noqa: BLE001
            errors.append(f"thread {i}: {type(e).__name__}: {e}")

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(shapes))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads)
    assert not errors, errors
    assert len(msgs) == len(shapes)
