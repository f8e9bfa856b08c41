"""Oracle pins for the VDN-H3 window mask (rt/attn.rs:469-524): hand-counted visible sets
for the reference's two window forms, the anchor / global rules, and the library's host
helper against the oracle."""
import numpy as np

import util  # noqa: F401  (puts the package directory on sys.path)

import fv_sdpa  # noqa: E402


def frames_seen(oracle, w, qf):
    vs, t, frames, chunk, radius = w
    q = vs + qf * t
    return [kf for kf in range(frames) if oracle.vdn_window_allows(vs, t, frames, chunk, radius, q, vs + kf * t)]


def test_chunk_aligned_window_sees_10_to_15_frames(oracle):
    # chunk 5, radius 1 (the shipped transform, docs/ports/vdn-h3.md:103-105): a query frame sees
    # its own chunk and one chunk each side, clamped to the clip, plus the two anchor frames
    w = (7, 3, 32, 5, 1)
    assert frames_seen(oracle, w, 12) == [0] + list(range(5, 20)) + [31]      # chunk 2: chunks 1..3
    assert frames_seen(oracle, w, 2) == list(range(0, 10)) + [31]             # chunk 0: clamped, 10 frames
    assert frames_seen(oracle, w, 27) == [0] + list(range(20, 32))            # chunk 5: frames 20..34 -> ..31
    assert frames_seen(oracle, w, 29) == frames_seen(oracle, w, 25)           # same chunk, same window
    assert frames_seen(oracle, w, 0) == list(range(32)) == frames_seen(oracle, w, 31)   # anchors: dense


def test_centred_window(oracle):
    # gpucheck kernels.rs:2860-2868: video_start 16, frame_tokens 16, frames 15, chunk 0, radius 1
    w = (16, 16, 15, 0, 1)
    assert frames_seen(oracle, w, 5) == [0, 4, 5, 6, 14]
    assert frames_seen(oracle, w, 1) == [0, 1, 2, 14]
    assert frames_seen(oracle, w, 13) == [0, 12, 13, 14]
    # token granularity: every token of a frame shares the frame's answer
    for q in range(16 + 5 * 16, 16 + 6 * 16):
        for k in (16 + 3 * 16 + 15, 16 + 4 * 16, 16 + 6 * 16 + 15, 16 + 7 * 16):
            assert oracle.vdn_window_allows(*w, q, k) == (k // 16 - 1 in (4, 5, 6))


def test_global_rows_and_anchor_symmetry(oracle):
    w = (5, 4, 9, 2, 1)
    ve = 5 + 9 * 4
    m = oracle.vdn_window_dense_mask(*w, ve + 6, ve + 6)
    vis = m == 0
    assert set(np.unique(m)) <= {0.0, np.float32(-1e9)}
    assert vis[:5].all() and vis[ve:].all() and vis[:, :5].all() and vis[:, ve:].all()     # rows outside the video
    assert vis[5:9].all() and vis[ve - 4:ve].all() and vis[:, 5:9].all() and vis[:, ve - 4:ve].all()   # anchor frames
    inner = vis[9:ve - 4, 9:ve - 4]
    assert not inner.all()                              # something is masked
    # chunk 2, radius 1: frame f sees frames (f//2 - 1)*2 .. (f//2 + 2)*2 - 1
    for qf in range(1, 8):
        for kf in range(1, 8):
            want = (qf // 2 - 1) * 2 <= kf <= (qf // 2 + 2) * 2 - 1
            assert vis[5 + qf * 4, 5 + kf * 4 + 3] == want, (qf, kf)


def test_library_host_helper_equals_the_oracle(oracle):
    rng = np.random.Generator(np.random.PCG64(12))
    for _ in range(20):
        vs, t, frames = int(rng.integers(0, 9)), int(rng.integers(1, 7)), int(rng.integers(1, 12))
        chunk, radius = int(rng.integers(0, 4)), int(rng.integers(0, 3))
        s = vs + frames * t + int(rng.integers(0, 5))
        want = oracle.vdn_window_dense_mask(vs, t, frames, chunk, radius, s, s)
        got = fv_sdpa.VdnWindow(vs, t, frames, chunk, radius).dense_mask(s, s)
        assert np.array_equal(got, want)
