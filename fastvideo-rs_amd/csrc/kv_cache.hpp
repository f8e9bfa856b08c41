// The per-layer KV cache of causal (Self-Forcing) Wan generation and the arithmetic of its
// pointers, mirroring crates/fastvideo-cudarc/src/wan/causal.rs:38-57 (`KvSpec`), 276-336
// (`KvMove`, `KvSpec::plan`) and 341-723 (`CausalKvCache`, static mode): one persistent
// [batch, heads, capacity, d] buffer pair per layer, written in place; the window the queries read
// comes back as a row window of those buffers (no copy): the fused attention kernel reads a
// (batch, head) plane at any plane stride.
//
// RoPE policies (wan/causal.rs:59-76): absolute (keys arrive roped); relativistic (the caller caches
// un-roped keys and ropes the window itself at every forward: nothing for the cache to do but carry
// the flag); rebased sink (absolute keys, the sink re-roped in place by `rebase_sink` from an f32
// un-roped copy taken once).
#pragma once
#include <mutex>
#include <utility>

#include "rt_sdpa.hpp"

namespace fv::rt {

// wan/causal.rs:38-57 (token geometry of one cache)
struct KvSpec {
    size_t frame_tokens = 0;    // tokens per latent frame
    size_t capacity = 0;        // physical cache length in tokens
    size_t sink = 0;            // tokens kept at the head when the cache rolls
    size_t max_attention = 0;   // keys each query block reads, back from the end of the block
    bool rolling = false;       // a full cache drops its oldest tokens after the sink instead of refusing
    bool relativistic = false;  // raw (normed, un-roped) keys cached; the window is roped by the caller
    bool rebase_sink = false;   // absolute keys, the sink re-roped each block (`rebase_sink`)
    // wan/causal.rs:136-145: the frame the sink keys should sit at once the write ending at frame
    // end_frame is done, and the frames the queries can read
    size_t window_frames() const { return max_attention / (frame_tokens ? frame_tokens : 1); }
    size_t sink_target(size_t end_frame) const { return end_frame > window_frames() ? end_frame - window_frames() : 0; }
};

// wan/causal.rs:276-287
struct KvMove {
    size_t evicted = 0;                     // tokens dropped after the sink before writing
    size_t local_start = 0, local_end = 0;  // where the block's K/V are written
    size_t window_start = 0;                // the queries read [window_start, local_end)
};

// wan/causal.rs:289-336 `KvSpec::plan`: the pointer arithmetic for n new tokens at current_start
// from the cache state (global_end, local_end_prev).
Result<KvMove> kv_plan(const KvSpec& spec, size_t global_end, size_t local_end_prev, size_t current_start,
                       size_t n);

// wan/causal.rs:199-248 on device buffers [bh, rows, d] of f32 or bf16 elements:
// dst[:, dst_off .. dst_off + len] = src[:, src_off .. src_off + len] ...
int kv_copy_tokens(void* dst, size_t dst_rows, size_t dst_off, const void* src, size_t src_rows, size_t src_off,
                   size_t len, size_t bh, size_t d, DType dtype, hipStream_t st);
// ... and tokens [from, from + len) of t moved down to [to, to + len), to < from, in chunks no longer
// than the shift so that no launch reads what it writes.
int kv_shift_tokens_down(void* t, size_t rows, size_t from, size_t to, size_t len, size_t bh, size_t d,
                         DType dtype, hipStream_t st);

// wan/causal.rs:250-262 `rope_bhsd_f32` / 264-274 `rope_bhsd`: interleaved RoPE (even-slot tables
// [s, d]) of rows [0, s) of every plane of x into out; planes may be row windows (x_rows / out_rows
// rows per plane); the result is f32 or rounded once to bf16.
int kv_rope_bhsd(const void* x, DType x_dtype, size_t x_rows, const float* cos_t, const float* sin_t,
                 bool negate_sin, void* out, DType out_dtype, size_t out_rows, size_t bh, size_t s, size_t d,
                 hipStream_t st);

// wan/causal.rs:353-360
struct KvPointers {
    size_t global_end = 0, local_end = 0, sink_at = 0;
    bool raw_valid = false;
};

// wan/causal.rs:341-723. static_mode (`new_static`): persistent buffers written in place, the same
// addresses at every block forward (what a HIP-graph replay needs). Otherwise (`new`): every write
// builds the layer's K / V anew, exactly local_end tokens long (kept prefix + the block), in freshly
// allocated stream-ordered buffers, and releases the previous ones; the windows hold the same values.
class CausalKvCache {
  public:
    CausalKvCache(KvSpec spec, size_t num_layers, bool static_mode = true);
    bool is_static() const { return static_mode_; }
    ~CausalKvCache();
    CausalKvCache(const CausalKvCache&) = delete;
    CausalKvCache& operator=(const CausalKvCache&) = delete;

    // Writes one block's k / v ([b, h, n, d], contiguous, same dtype, RoPE applied) for `layer` at
    // token `current_start`; returns the K / V windows its queries attend to: borrowed row windows
    // [b, h, len, d] of the layer's buffers (plane_rows = capacity), valid until the next write.
    Result<std::pair<Tensor, Tensor>> update(size_t layer, const Tensor& k, const Tensor& v, size_t current_start,
                                             hipStream_t st);
    // wan/causal.rs:733-806 `rebase_sink`: re-rope every layer's sink keys to start at frame `target`.
    // orig_* are the tables of the sink's own frames [0, sink) (used once, to take the un-roped f32
    // copy), new_* those of frames [target, target + sink): f32 [sink_tokens, d] each, even-slot.
    // Returns whether any layer moved; a no-op where the sink is already there or not yet filled.
    Result<bool> rebase_sink(size_t target, const float* orig_cos, const float* orig_sin, const float* new_cos,
                             const float* new_sin, hipStream_t st);
    void reset();                         // a new rollout: pointers to zero, buffers (addresses) kept
    void set_sink_guard(bool on) { sink_guard_ = on; }
    bool sink_guard() const { return sink_guard_; }
    std::vector<KvPointers> pointers() const;
    // wan/causal.rs:457-476 `set_pointers`: put pointers back (a graph replay moves no host state, a
    // failed capture must leave none behind); one entry per layer.
    Result<bool> set_pointers(const std::vector<KvPointers>& p);
    // wan/causal.rs:503-536 `advance`: the host bookkeeping of one block forward of n tokens at
    // current_start (sink target frame `sink_target`, 0: none) without its device work: what a graph
    // replay of that forward leaves behind.
    Result<bool> advance(size_t current_start, size_t n, size_t sink_target);
    // wan/causal.rs:477-502 `block_key`: what a forward of n tokens at current_start (sink target frame
    // `sink_target`, 0: none) does to the cache, from layer 0's pointers (every layer moves in step).
    // Forwards with equal keys launch the same device work, so a captured graph of one serves the others.
    struct BlockKey {
        size_t local_end;
        bool appends;       // the block extends the cache (false: an in-place re-run of cached frames)
        size_t evicted;
        bool rebase;        // the rebased-sink policy re-ropes the sink before this block
        bool take_raw;      // ... and first takes the un-roped copy
    };
    Result<BlockKey> block_key(size_t current_start, size_t n, size_t sink_target) const;
    size_t bytes() const;
    const KvSpec spec;

  private:
    struct Layer {
        void* k = nullptr;
        void* v = nullptr;
        void* raw_sink = nullptr;   // f32 [b, h, sink, d], the un-roped sink keys
        size_t sink_at = 0;
        bool raw_valid = false;
        size_t b = 0, h = 0, cap = 0, d = 0, dv = 0;
        DType kd = DType::F32, vd = DType::F32;
        size_t global_end = 0, local_end = 0;
    };
    Result<std::pair<Tensor, Tensor>> update_dynamic(Layer& L, const KvMove& mv, size_t skip, const Tensor& k,
                                                     const Tensor& v, size_t current_start, hipStream_t st);
    mutable std::mutex mu_;
    std::vector<Layer> layers_;
    bool sink_guard_ = false;
    const bool static_mode_;
};

}  // namespace fv::rt
