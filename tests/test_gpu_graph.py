"""HIP-graph capture of the library's entry points: every call is stream-ordered and allocates
nothing, so a captured call replays on new data in the same buffers. Each graph is replayed several
times with eager work and synchronisations of the program's own in between, and every replay is
checked bit for bit against the eager call on the same inputs. (`fv_sdpa_init` sets the once-per-device
LDS attributes of the kernels up front, so that no capture has to.)
"""
import numpy as np
import pytest

from util import announce

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def fv():
    import torch

    assert torch.cuda.is_available()
    import fv_sdpa

    assert fv_sdpa.lib().fv_sdpa_init() == 0   # per-device kernel attributes, before any capture
    assert fv_sdpa.lib().fv_sdpa_init() == 0   # idempotent
    return fv_sdpa


def _fill(g, *tensors):
    import torch

    for t in tensors:
        t.copy_(torch.randn(t.shape, generator=g, device="cuda").to(t.dtype))


@pytest.mark.parametrize("form", ["exact", "log2_domain"])
def test_dense_and_block_causal_replay(fv, form):
    """Both forms of the fused kernel (the second is taken at scale = ln 2, operands as they are)."""
    import torch

    announce(f"graph: dense + block-causal, {form}")
    bh, s, d = 4, 700, 128
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v = (torch.empty((bh, s, d), device="cuda", dtype=torch.bfloat16) for _ in range(3))
    _fill(g, q, k, v)
    lib = fv.lib()
    out_d = torch.empty((bh, s, d), device="cuda", dtype=torch.bfloat16)
    out_c = torch.empty((bh, s, d), device="cuda", dtype=torch.float32)
    scale = 1.0 / d ** 0.5 if form == "exact" else float(np.float32(np.log(2.0)))
    assert lib.fv_sdpa_is_log2_domain_scale(scale) == (form == "log2_domain")

    def run():
        st = torch.cuda.current_stream().cuda_stream
        assert lib.fv_sdpa_dense_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out_d.data_ptr(), 1, bh, s, s, d, scale, st) == 0
        assert lib.fv_sdpa_block_causal_bf16(q.data_ptr(), k.data_ptr(), v.data_ptr(), out_c.data_ptr(), 0, bh, s, s, d,
                                             scale, 100, 2, 1, st) == 0

    run()                                   # eager first: per-device kernel attributes
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for i in range(4):
        _fill(g, q, k, v)
        want_d = fv.sdpa_dense_bf16(q, k, v, out_bf16=True, scale=scale)
        want_c = fv.sdpa_block_causal_bf16(q, k, v, 100, 2, 1, scale=scale)
        torch.cuda.synchronize()
        out_d.zero_()
        out_c.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_d, want_d) and torch.equal(out_c, want_c), i


def test_vsa_whole_op_replay(fv):
    import torch

    announce("graph: VSA whole op")
    grid, heads, d = (5, 6, 9), 3, 128
    ctx = fv.VsaCtx(grid, 0.8)
    g = torch.Generator(device="cuda").manual_seed(2)
    q, k, v, gate = (torch.empty((heads, ctx.seq, d), device="cuda", dtype=torch.bfloat16) for _ in range(4))
    _fill(g, q, k, v, gate)
    lib = fv.lib()
    nb, topk = ctx.num_tiles, ctx.topk
    nbytes = int(lib.fv_vsa_workspace_bytes(heads, nb, topk, d))
    ws = torch.empty(nbytes, device="cuda", dtype=torch.uint8)
    out = torch.empty((heads, ctx.seq, d), device="cuda", dtype=torch.float32)
    sel = torch.empty((heads, nb, topk), device="cuda", dtype=torch.int32)
    scale = 1.0 / d ** 0.5

    def run():
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.fv_vsa_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), 1, gate.data_ptr(), 1, ctx.slot_src.data_ptr(),
                                  ctx.block_sizes.data_ptr(), out.data_ptr(), ws.data_ptr(), nbytes, sel.data_ptr(), heads,
                                  ctx.seq, nb, topk, d, scale, st)
        assert rc == 0

    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for i in range(3):
        _fill(g, q, k, v, gate)
        want, want_sel = fv.vsa_attention_device(q, k, v, gate, ctx, scale, return_selected=True)
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(sel, want_sel) and torch.equal(out, want), i


def test_kv_cache_block_forward_replay(fv):
    """One block forward through a static KV cache (roll + write + attention on the window in place)
    captured once and replayed for later blocks of the same shape: the buffers' addresses never
    change, the host pointers move with `advance` (wan/causal.rs:503-536)."""
    import torch

    announce("graph: kv cache block forward")
    b, h, d, ft = 1, 3, 128, 40
    n = 2 * ft
    spec = fv.KvSpec.rolling_window(ft, 6, 1)
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v = (torch.empty((b, h, n, d), device="cuda", dtype=torch.bfloat16) for _ in range(3))
    cache, ref = fv.CausalKvCache(spec, 1), fv.CausalKvCache(spec, 1)
    lib = fv.lib()
    out = torch.empty((b * h, n, d), device="cuda", dtype=torch.bfloat16)

    def forward(c, start, dst):
        kw, vw = c.update(0, k, v, start)
        rows = kw.stride(1) // d
        st = torch.cuda.current_stream().cuda_stream
        assert lib.fv_sdpa_dense_bf16_strided(q.data_ptr(), kw.data_ptr(), vw.data_ptr(), dst.data_ptr(), 1, b * h, n,
                                              kw.shape[2], d, 1.0 / d ** 0.5, 0, rows, rows, st) == 0

    # fill the window eagerly on both caches (blocks 0..2), then block 3 rolls: steady state
    for blk in range(3):
        _fill(g, q, k, v)
        forward(cache, blk * n, out)
        forward(ref, blk * n, torch.empty_like(out))
    torch.cuda.synchronize()
    state = [cache.pointers4(0)]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        forward(cache, 3 * n, out)          # capture: the device work is recorded, not run
    cache.set_pointers(state)               # the capture moved host state only; put it back
    for blk in range(3, 7):
        _fill(g, q, k, v)
        want = torch.empty_like(out)
        forward(ref, blk * n, want)
        torch.cuda.synchronize()
        out.zero_()
        graph.replay()
        cache.advance(blk * n, n)
        torch.cuda.synchronize()
        assert cache.pointers(0) == ref.pointers(0)
        assert torch.equal(out, want), blk
