// Host-side mirror of the reference's one dense-attention entry,
// `rt::sdpa::sdpa(q, k, v, &Plan)` (crates/fastvideo-cudarc/src/rt/sdpa.rs:29-342),
// over the gfx950 kernels. Same names, argument meaning and error strings; the
// chooser (`rt/sdpa_rule.rs`) collapses to ONE fused HIP kernel per plan with the
// device composed path behind it — no cuDNN / cuBLAS / FP8 / Sage steps, no
// sequence-parallel shards (the whole sequence stays on one GPU), and never a
// host computation behind the caller's back.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <optional>
#include <string>
#include <variant>
#include <vector>

namespace fv::rt {

// rt/tensor.rs:28-32 `TensorDType`
enum class DType : int { F32 = 0, Bf16 = 1 };

// rt/tensor.rs:92-98 `TensorError::Message`
struct TensorError {
    std::string message;
    int hip_code = 0;   // the hipError_t behind the message (allocation, launch); 0 = a refused argument
};

template <class T>
using Result = std::variant<T, TensorError>;
template <class T>
bool is_ok(const Result<T>& r) { return r.index() == 0; }

// A device tensor (rt/tensor.rs:196-210 `CudaTensor`, device side only):
// contiguous row-major storage of f32 or bf16 bits, owned (freed stream-ordered
// on `stream`) or borrowed from the caller.
class Tensor {
  public:
    Tensor() = default;
    Tensor(const Tensor&) = delete;
    Tensor& operator=(const Tensor&) = delete;
    Tensor(Tensor&& o) noexcept;
    Tensor& operator=(Tensor&& o) noexcept;
    ~Tensor();

    static Tensor borrowed(void* data, std::vector<size_t> shape, DType dtype);
    // A borrowed rank-4 row window: [b, h, s, d] whose (batch, head) planes sit plane_rows * d
    // elements apart in the underlying buffer (plane_rows >= s; 0 = contiguous). What `narrow(2, ..)`
    // of a longer BHSD tensor is without the copy (rt/tensor.rs:825-870 copies).
    static Tensor window(void* data, std::vector<size_t> shape, DType dtype, size_t plane_rows);
    static Result<Tensor> alloc(std::vector<size_t> shape, DType dtype, hipStream_t stream);

    size_t rank() const { return shape.size(); }
    bool strided() const { return plane_rows != 0 && shape.size() == 4 && plane_rows != shape[2]; }
    size_t numel() const;
    // Gives up ownership of the buffer (the caller frees it with hipFree).
    void* release();

    std::vector<size_t> shape;
    DType dtype = DType::F32;
    void* data = nullptr;
    size_t plane_rows = 0;   // rows per (batch, head) plane of the storage; 0 = shape[2]

  private:
    bool owned_ = false;
    hipStream_t stream_ = nullptr;
};

// rt/attn.rs:441-467
struct BlockCausal {
    size_t block_tokens = 0, window = 0, sink = 0;
    bool allows(size_t q, size_t k) const;
    std::vector<float> dense_mask(size_t sq, size_t sk) const;
};

// rt/attn.rs:469-524 — VDN-H3's window mask.
struct VdnWindow {
    size_t video_start = 0, frame_tokens = 0, frames = 0, chunk = 0, radius = 0;
    size_t video_end() const { return video_start + frames * frame_tokens; }
    bool allows(size_t q, size_t k) const;
    std::vector<float> dense_mask(size_t sq, size_t sk) const;
};

// rt/sdpa.rs:29-137
class Plan {
  public:
    static Plan dense(std::optional<float> scale);
    static Plan masked(std::optional<float> scale, const Tensor* mask);
    Plan fp8_first() const;
    static Plan composed(std::optional<float> scale, const Tensor* mask);
    static Plan block_causal(std::optional<float> scale, BlockCausal mask);
    static Plan vdn_window(std::optional<float> scale, VdnWindow mask);
    static Plan kv_window();
    static Plan kv_window_with(bool flash);

    enum class Kind { Dense, Composed, BlockCausalK, VdnWindowK, KvWindow };
    Kind kind = Kind::Dense;
    std::optional<float> scale;
    const Tensor* mask = nullptr;
    bool fp8_first_flag = false;
    BlockCausal causal;
    VdnWindow window;
    std::optional<bool> kv_flash;
};

// rt/tensor.rs:61-76 `bf16_activations` / `with_bf16_act`: FASTVIDEO_BF16_ACT
// (unset = on: a device is always live here), overridable per thread.
bool bf16_activations();
void set_bf16_activations_override(std::optional<bool> v);
// rt/sdpa_rule.rs `causal_flash_enabled`: FASTVIDEO_WAN_CAUSAL_FLASH, default on.
bool causal_flash_enabled();
// Whether the bf16 copy the library makes of an f32 q carries scale * log2(e) (one rounding of the product; the
// fused kernel then runs at scale = ln 2): FASTVIDEO_SDPA_FOLD_SCALE, default on, overridable per thread.
bool fold_scale();
void set_fold_scale_override(std::optional<bool> v);

// rt/sdpa_rule.rs:178-219 `Backend` / `parse_backend` / `backend`: FASTVIDEO_SDPA (lower-cased,
// read once), overridable per thread. Anything but the four names below is the dense default.
enum class Backend : int { Dense = 0, Cublas = 1, Flash = 2, Host = 3, Sparse = 4 };
Backend parse_backend(const std::string& v);
Backend backend();
void set_backend_override(std::optional<Backend> v);

// rt/sdpa_rule.rs:350-390 `Dims` / `Shape::of`: the lengths a dense call is chosen on, and the
// five dims when k and v are both [b, h, sk, d] of q's [b, h, sq, d].
struct Dims {
    size_t b, h, sq, sk, d;
};
struct Shape {
    size_t sq = 0, sk = 0;
    std::optional<Dims> dims;
    static Shape of(const std::vector<size_t>& q, const std::vector<size_t>& k, const std::vector<size_t>& v);
};

// rt/sdpa_rule.rs:392-437 `Step` / `dense_route`, with the NVIDIA alternates gone: an unmasked call
// tries the fused gfx950 kernel and then the composed f32 kernel; FASTVIDEO_SDPA=cublas|flash (the
// reference's f32-score kernels) go straight to the composed f32 kernel; host|sparse are retired and
// refuse the call; a masked call is composed.
enum class Step : int { Retired = 0, Fused = 1, Composed = 2 };
std::vector<Step> dense_route(const Shape& shape, bool masked, Backend backend);

// rt/sdpa.rs:141-164. Work is enqueued on `stream`; the result owns its buffer.
Result<Tensor> sdpa(const Tensor& q, const Tensor& k, const Tensor& v, const Plan& plan,
                    hipStream_t stream);

// rt/sdpa.rs:328-342 on the device: softmax(scale q k^T + mask) v in f32 from the
// operands as given (bf16 operands are widened exactly).
Result<Tensor> sdpa_composed(const Tensor& q, const Tensor& k, const Tensor& v,
                             std::optional<float> scale, const Tensor* mask, hipStream_t stream);

// Launch counters (rt/stats.rs:27-72 keeps h2d/d2h/launch/fallback counts).
struct Stats {
    uint64_t fused_launches = 0, causal_launches = 0, composed_launches = 0, cast_launches = 0,
             masks_materialised = 0;
};
Stats stats_snapshot();

}  // namespace fv::rt
