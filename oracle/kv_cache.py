"""CPU restatement (test infrastructure only) of the causal-Wan KV cache of the reference:
`KvSpec::plan` (crates/fastvideo-cudarc/src/wan/causal.rs:289-336) and `CausalKvCache::update`
in its tensor-per-write form (causal.rs:540-625: narrow / cat on the valid prefix), with the sink
guard (causal.rs:410-418). numpy arrays [b, h, tokens, d]; integer arithmetic and copies only.

Pinned by the reference's own known answers (causal.rs:872-910: appends / overwrites / refusal of a
22nd frame; the rolling cache that keeps its sink) in tests/test_oracle_kv_cache.py, by hand-built
roll sequences, and by the invariant the reference asserts at causal.rs:916-1000 (block by block
through the cache == the whole clip under the block-causal mask).
"""
import numpy as np

__all__ = ["KvSpecO", "KvError", "CausalKvCacheO", "rope_bhsd_f32"]


class KvError(ValueError):
    pass


def rope_bhsd_f32(x, cos, sin):
    """causal.rs:250-262 over `apply_rotary_bshd` (C/rt/ops.rs:1903-1935): pair (2i, 2i+1) of row r of
    every [b, h] plane turns by the angle whose cos / sin sit in the EVEN slot 2i of the [s, d] tables.
    f32 arithmetic, each product rounded before the sum."""
    x = np.asarray(x, dtype=np.float32)
    c = np.asarray(cos, dtype=np.float32)[None, None, :, 0::2]
    s = np.asarray(sin, dtype=np.float32)[None, None, :, 0::2]
    x1, x2 = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x)
    out[..., 0::2] = (x1 * c).astype(np.float32) - (x2 * s).astype(np.float32)
    out[..., 1::2] = (x1 * s).astype(np.float32) + (x2 * c).astype(np.float32)
    return out


class KvSpecO:
    def __init__(self, frame_tokens, capacity, sink, max_attention, rolling, rebase_sink=False):
        self.frame_tokens, self.capacity, self.sink = frame_tokens, capacity, sink
        self.max_attention, self.rolling = max_attention, rolling
        self.rebase_sink = rebase_sink and sink > 0

    def window_frames(self):
        return self.max_attention // max(self.frame_tokens, 1)

    def sink_target(self, end_frame):
        """causal.rs:136-138."""
        return max(end_frame - self.window_frames(), 0)

    def plan(self, global_end, local_end_prev, current_start, n):
        """causal.rs:289-336 -> (evicted, local_start, local_end, window_start)."""
        current_end = current_start + n
        if not self.rolling and current_end > self.max_attention:
            raise KvError("causal Wan local_attn_size=-1 keeps a %d-frame KV window; got current_end=%d"
                          % (self.max_attention // max(self.frame_tokens, 1), current_end))
        if current_end < global_end and current_end + local_end_prev < global_end:
            raise KvError("causal kv: block before the cache start")
        advance = max(current_end - global_end, 0)
        evicted = 0
        if self.rolling and current_end > global_end and n + local_end_prev > self.capacity:
            evicted = n + local_end_prev - self.capacity
        local_end = local_end_prev + advance - max(global_end - current_end, 0)
        if local_end < 0 or local_end - evicted < 0:
            raise KvError("causal kv: pointer underflow")
        local_end -= evicted
        local_start = local_end - n
        if local_start < 0:
            raise KvError("causal kv: block longer than the cache")
        if local_end > max(self.capacity, n):
            raise KvError("causal kv: write end %d past the cache" % local_end)
        return evicted, local_start, local_end, max(local_end - self.max_attention, 0)


class _Layer:
    def __init__(self):
        self.k = self.v = self.raw_sink = None
        self.global_end = self.local_end = self.sink_at = 0


class CausalKvCacheO:
    """causal.rs:540-625, the non-static path: the cache is the valid prefix, rebuilt per write."""

    def __init__(self, spec, num_layers):
        self.spec, self.layers, self.sink_guard = spec, [_Layer() for _ in range(num_layers)], False

    def reset(self):
        self.layers = [_Layer() for _ in self.layers]

    def rebase_sink(self, target, orig, new, quantize=None):
        """causal.rs:733-808 (tensor-per-write path): re-rope every layer's sink keys to start at frame
        `target`; orig / new = (cos, sin) [sink_tokens, d] of the sink's own frames / the target's.
        quantize: the rounding of a bf16 cache (None for f32)."""
        sink = self.spec.sink
        if sink == 0:
            return
        for slot in self.layers:
            if slot.sink_at == target or slot.k is None or slot.k.shape[2] < sink:
                continue
            if slot.raw_sink is None:
                slot.raw_sink = rope_bhsd_f32(slot.k[:, :, :sink], orig[0], -np.asarray(orig[1], dtype=np.float32))
            head = rope_bhsd_f32(slot.raw_sink, new[0], new[1])
            if quantize is not None:
                head = quantize(head)
            slot.k = np.concatenate([head, slot.k[:, :, sink:]], axis=2)
            slot.sink_at = target

    def update(self, layer, k, v, current_start):
        slot, spec = self.layers[layer], self.spec
        n = k.shape[2]
        evicted, local_start, local_end, window_start = spec.plan(slot.global_end, slot.local_end, current_start, n)
        skip = 0
        if self.sink_guard and current_start > 0 and current_start + n <= slot.global_end:
            skip = min(max(spec.sink - local_start, 0), n)

        def keep(t):
            if t is None:
                return None
            if evicted > 0:
                length = t.shape[2]
                sink = min(spec.sink, length)
                tail_start = min(sink + evicted, length)
                t = np.concatenate([t[:, :, :sink], t[:, :, tail_start:]], axis=2)
            at = local_start + skip
            if at == 0:
                return None
            if at > t.shape[2]:
                raise KvError("causal kv: write at %d leaves a gap after %d cached tokens" % (at, t.shape[2]))
            return t[:, :, :at]

        k_keep, v_keep = keep(slot.k), keep(slot.v)
        if local_start + skip > 0 and k_keep is None:
            raise KvError("causal kv: write past an empty cache")

        def join(prefix, new):
            new = new[:, :, skip:]
            return new.copy() if prefix is None else np.concatenate([prefix, new], axis=2)

        slot.k, slot.v = join(k_keep, k), join(v_keep, v)
        slot.global_end, slot.local_end = current_start + n, local_end
        return slot.k[:, :, window_start:local_end], slot.v[:, :, window_start:local_end]
