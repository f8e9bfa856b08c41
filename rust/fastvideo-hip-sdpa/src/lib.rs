//! `fastvideo-hip-sdpa`: the attention hot path of fastvideo-rs on AMD MI355X (gfx950).
//!
//! A thin binding of `libfv_sdpa_hip.so` (C ABI in `include/fv_sdpa_hip.h`, raw declarations in
//! [`ffi`]) plus drop-in shims with the signatures fastvideo-rs calls today:
//!
//! | fastvideo-cudarc (`crates/fastvideo-cudarc/src/rt`)            | here                         |
//! |----------------------------------------------------------------|------------------------------|
//! | `sdpa::sdpa(q, k, v, &Plan)` (`sdpa.rs:141`)                   | [`sdpa`]                     |
//! | `attn::device_mma_sdpa` (`attn.rs:225`)                        | [`device_mma_sdpa`]          |
//! | `attn::device_mma_sdpa_causal` (`attn.rs:652`)                 | [`device_mma_sdpa_causal`]   |
//! | `attn::device_mma_sdpa_window` (`attn.rs:526`)                 | [`device_mma_sdpa_window`]   |
//! | `vsa::vsa_attention_device` (`vsa.rs:358`)                     | [`vsa_attention_device`]     |
//!
//! The tensor type of the shims is [`CudaTensor`], an alias of [`HipTensor`]: a device buffer with
//! a shape and a dtype, what the device half of fastvideo-rs's `CudaTensor` (`rt/tensor.rs:196-210`)
//! becomes once `cudarc` is gone. Nothing here computes on the host and nothing falls back to
//! another backend: a call the fused kernel declines comes back as `Ok(None)` exactly where the
//! reference's launcher returns `Ok(None)`, and [`sdpa`] then takes the composed f32 kernel of the
//! same library.
//!
//! This crate is written against the header and is **not compiled in the environment that built
//! the library** (no Rust toolchain there); `tests/test_rust_ffi.py` of the repository checks every
//! `extern "C"` declaration in [`ffi`] against the header mechanically.
#![allow(clippy::too_many_arguments)]

pub mod ffi;
pub mod hip;

use std::ffi::{c_int, c_void, CStr};
use std::marker::PhantomData;
use std::ptr;

use ffi::{FvPlan, FvTensor, FV_DECLINED, FV_OK};
use hip::HipStream;

/// `rt/tensor.rs:92-98`. `Display` prints the message as it is, which is what the reference's
/// `#[error("{0}")]` derives; written out by hand so that the crate has no dependency to fetch.
#[derive(Debug)]
pub enum TensorError {
    Message(String),
}

impl std::fmt::Display for TensorError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        match self {
            TensorError::Message(m) => f.write_str(m),
        }
    }
}

impl std::error::Error for TensorError {}

pub type Result<T> = std::result::Result<T, TensorError>;

fn msg(s: impl Into<String>) -> TensorError {
    TensorError::Message(s.into())
}

/// The library's per-thread message for the last non-zero return.
pub fn last_error() -> String {
    // SAFETY: fv_sdpa_last_error returns a NUL-terminated string owned by the library (thread local).
    unsafe { CStr::from_ptr(ffi::fv_sdpa_last_error()) }.to_string_lossy().into_owned()
}

fn hip_check(code: c_int, what: &str) -> Result<()> {
    if code == 0 {
        Ok(())
    } else {
        Err(msg(format!("{what}: {} (hipError {code})", hip::error_string(code))))
    }
}

/// `rt/tensor.rs:28-32`.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub enum TensorDType {
    F32,
    Bf16,
}

impl TensorDType {
    pub fn size(self) -> usize {
        match self {
            TensorDType::F32 => 4,
            TensorDType::Bf16 => 2,
        }
    }
    fn code(self) -> c_int {
        match self {
            TensorDType::F32 => 0,
            TensorDType::Bf16 => 1,
        }
    }
}

// The stream every shim enqueues on. fastvideo-rs keeps one stream per device (`rt/device.rs`); a port
// sets it once per thread with `set_stream`. Null is HIP's default stream.
thread_local! {
    static STREAM: std::cell::Cell<HipStream> = const { std::cell::Cell::new(ptr::null_mut()) };
}

pub fn set_stream(stream: HipStream) {
    STREAM.with(|s| s.set(stream));
}

pub fn stream() -> HipStream {
    STREAM.with(|s| s.get())
}

/// A typed device allocation (what `cudarc::driver::CudaSlice<T>` is to the reference). Freed
/// stream-ordered on the stream it was allocated on.
pub struct HipSlice<T> {
    ptr: *mut c_void,
    len: usize,
    stream: HipStream,
    owned: bool,
    _elem: PhantomData<T>,
}

impl<T> HipSlice<T> {
    pub fn alloc(len: usize) -> Result<Self> {
        let mut p: *mut c_void = ptr::null_mut();
        let st = stream();
        // SAFETY: plain FFI call; `p` receives a device pointer or stays null on error.
        hip_check(unsafe { hip::hipMallocAsync(&mut p, len.max(1) * std::mem::size_of::<T>(), st) }, "hipMallocAsync")?;
        Ok(Self { ptr: p, len, stream: st, owned: true, _elem: PhantomData })
    }

    /// Wraps device memory owned elsewhere (the runtime's own allocator, a KV cache window).
    ///
    /// # Safety
    /// `data` must address at least `len` elements of `T` on the current device for the lifetime of the value.
    pub unsafe fn borrowed(data: *mut c_void, len: usize) -> Self {
        Self { ptr: data, len, stream: ptr::null_mut(), owned: false, _elem: PhantomData }
    }

    pub fn from_host(host: &[T]) -> Result<Self> {
        let s = Self::alloc(host.len())?;
        // SAFETY: `s.ptr` holds host.len() elements; the copy is ordered on the slice's stream.
        hip_check(
            unsafe {
                hip::hipMemcpyAsync(s.ptr, host.as_ptr().cast(), std::mem::size_of_val(host), hip::HIP_MEMCPY_HOST_TO_DEVICE, s.stream)
            },
            "hipMemcpyAsync",
        )?;
        // the source is pageable host memory: wait, so the caller may drop it
        // SAFETY: plain FFI call.
        hip_check(unsafe { hip::hipStreamSynchronize(s.stream) }, "hipStreamSynchronize")?;
        Ok(s)
    }

    pub fn len(&self) -> usize {
        self.len
    }
    pub fn is_empty(&self) -> bool {
        self.len == 0
    }
    pub fn as_ptr(&self) -> *const T {
        self.ptr.cast_const().cast()
    }
    pub fn as_mut_ptr(&mut self) -> *mut T {
        self.ptr.cast()
    }
}

impl<T> Drop for HipSlice<T> {
    fn drop(&mut self) {
        if self.owned && !self.ptr.is_null() {
            // SAFETY: the pointer came from hipMallocAsync on `self.stream` and is freed once.
            unsafe { hip::hipFreeAsync(self.ptr, self.stream) };
        }
    }
}

/// A device tensor: contiguous row-major f32 or bf16 storage with a shape. `plane_rows != 0` marks a
/// rank-4 row window of a longer BHSD buffer (`narrow(2, ..)` without the copy, `rt/tensor.rs:825`).
pub struct HipTensor {
    pub shape: Vec<usize>,
    pub dtype: TensorDType,
    pub plane_rows: usize,
    data: *mut c_void,
    owner: Owner,
}

enum Owner {
    /// memory of the caller
    Borrowed,
    /// a buffer `fv_rt_sdpa` allocated: released with `fv_rt_free` on the stream it was produced on
    Library(HipStream),
    /// a buffer this crate allocated with `hipMallocAsync`
    Hip(HipStream),
}

/// The name the rest of fastvideo-rs uses for its tensor.
pub type CudaTensor = HipTensor;

impl HipTensor {
    /// # Safety
    /// `data` must address `shape.iter().product()` elements of `dtype` (or, with `plane_rows`, the
    /// planes of the longer buffer) on the current device while the tensor lives.
    pub unsafe fn from_device(data: *mut c_void, shape: Vec<usize>, dtype: TensorDType) -> Self {
        Self { shape, dtype, plane_rows: 0, data, owner: Owner::Borrowed }
    }

    /// A rank-4 row window: the (batch, head) planes of `data` sit `plane_rows * d` elements apart.
    ///
    /// # Safety
    /// As [`HipTensor::from_device`], for the planes of the longer buffer.
    pub unsafe fn window(data: *mut c_void, shape: Vec<usize>, dtype: TensorDType, plane_rows: usize) -> Self {
        let rows = if shape.len() == 4 && plane_rows != shape[2] { plane_rows } else { 0 };
        Self { shape, dtype, plane_rows: rows, data, owner: Owner::Borrowed }
    }

    pub fn alloc(shape: Vec<usize>, dtype: TensorDType) -> Result<Self> {
        let n: usize = shape.iter().product();
        let mut p: *mut c_void = ptr::null_mut();
        let st = stream();
        // SAFETY: plain FFI call.
        hip_check(unsafe { hip::hipMallocAsync(&mut p, n.max(1) * dtype.size(), st) }, "hipMallocAsync")?;
        Ok(Self { shape, dtype, plane_rows: 0, data: p, owner: Owner::Hip(st) })
    }

    pub fn rank(&self) -> usize {
        self.shape.len()
    }
    pub fn numel(&self) -> usize {
        self.shape.iter().product()
    }
    pub fn device_ptr(&self) -> *mut c_void {
        self.data
    }

    fn desc(&self) -> Result<FvTensor> {
        if self.rank() > 8 {
            return Err(msg("tensor rank above 8"));
        }
        let mut shape = [0usize; 8];
        shape[..self.rank()].copy_from_slice(&self.shape);
        Ok(FvTensor { data: self.data, dtype: self.dtype.code(), rank: self.rank() as c_int, shape, plane_rows: self.plane_rows })
    }

    fn from_library(t: FvTensor, st: HipStream) -> Self {
        Self {
            shape: t.shape[..t.rank as usize].to_vec(),
            dtype: if t.dtype == 0 { TensorDType::F32 } else { TensorDType::Bf16 },
            plane_rows: 0,
            data: t.data,
            owner: Owner::Library(st),
        }
    }
}

impl Drop for HipTensor {
    fn drop(&mut self) {
        if self.data.is_null() {
            return;
        }
        match self.owner {
            Owner::Borrowed => {}
            // SAFETY: the buffer came from fv_rt_sdpa / hipMallocAsync and is released exactly once.
            Owner::Library(st) => unsafe {
                ffi::fv_rt_free(self.data, st);
            },
            Owner::Hip(st) => unsafe {
                hip::hipFreeAsync(self.data, st);
            },
        }
    }
}

/// `rt/attn.rs:441-467`. The predicate and the dense mask are the library's host helpers.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct BlockCausal {
    pub block_tokens: usize,
    pub window: usize,
    pub sink: usize,
}

impl BlockCausal {
    pub fn allows(&self, q: usize, k: usize) -> bool {
        // SAFETY: host arithmetic only.
        unsafe { ffi::fv_block_causal_allows(self.block_tokens, self.window, self.sink, q, k) != 0 }
    }

    /// The additive `[sq, sk]` mask (0 visible, `-1e9` masked).
    pub fn dense_mask(&self, sq: usize, sk: usize) -> Vec<f32> {
        let mut m = vec![0.0f32; sq * sk];
        // SAFETY: `m` holds sq * sk floats, which is what the helper writes.
        unsafe { ffi::fv_block_causal_dense_mask(self.block_tokens, self.window, self.sink, sq, sk, m.as_mut_ptr()) };
        m
    }
}

/// `rt/attn.rs:630-645`.
pub fn block_causal_for(num_frames_per_block: usize, local_attn_size: i64, frame_tokens: usize) -> Option<BlockCausal> {
    let mut out = [0usize; 3];
    // SAFETY: `out` holds the three values the helper writes.
    let ok = unsafe { ffi::fv_block_causal_for(num_frames_per_block, local_attn_size, frame_tokens, out.as_mut_ptr()) };
    (ok != 0).then_some(BlockCausal { block_tokens: out[0], window: out[1], sink: out[2] })
}

/// `rt/attn.rs:469-524`.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct VdnWindow {
    pub video_start: usize,
    pub frame_tokens: usize,
    pub frames: usize,
    pub chunk: usize,
    pub radius: usize,
}

impl VdnWindow {
    pub fn video_end(&self) -> usize {
        self.video_start + self.frames * self.frame_tokens
    }

    pub fn allows(&self, q: usize, k: usize) -> bool {
        // SAFETY: host arithmetic only.
        unsafe { ffi::fv_vdn_window_allows(self.video_start, self.frame_tokens, self.frames, self.chunk, self.radius, q, k) != 0 }
    }

    pub fn dense_mask(&self, sq: usize, sk: usize) -> Vec<f32> {
        let mut m = vec![0.0f32; sq * sk];
        // SAFETY: `m` holds sq * sk floats.
        unsafe {
            ffi::fv_vdn_window_dense_mask(self.video_start, self.frame_tokens, self.frames, self.chunk, self.radius, sq, sk, m.as_mut_ptr())
        };
        m
    }
}

/// What one attention call computes (`rt/sdpa.rs:29-137`): same constructors, the decision logic
/// (route, bf16-activation rounding, fallbacks) lives in the library's host layer behind `fv_rt_sdpa`.
#[derive(Clone, Copy)]
pub struct Plan<'a> {
    kind: c_int,
    scale: Option<f32>,
    mask: Option<&'a CudaTensor>,
    fp8_first: bool,
    causal: Option<BlockCausal>,
    window: Option<VdnWindow>,
    kv_flash: Option<bool>,
}

impl<'a> Plan<'a> {
    fn of(kind: c_int, scale: Option<f32>) -> Self {
        Self { kind, scale, mask: None, fp8_first: false, causal: None, window: None, kv_flash: None }
    }

    pub fn dense(scale: Option<f32>) -> Self {
        Self::masked(scale, None)
    }

    pub fn masked(scale: Option<f32>, mask: Option<&'a CudaTensor>) -> Self {
        Self { mask, ..Self::of(ffi::FV_PLAN_DENSE, scale) }
    }

    /// Accepted for source compatibility: this library is bf16 only, the flag changes nothing.
    pub fn fp8_first(self) -> Self {
        if self.kind == ffi::FV_PLAN_DENSE && self.mask.is_none() {
            Self { fp8_first: true, ..self }
        } else {
            self
        }
    }

    pub fn composed(scale: Option<f32>, mask: Option<&'a CudaTensor>) -> Self {
        Self { mask, ..Self::of(ffi::FV_PLAN_COMPOSED, scale) }
    }

    pub fn block_causal(scale: Option<f32>, mask: BlockCausal) -> Self {
        Self { causal: Some(mask), ..Self::of(ffi::FV_PLAN_BLOCK_CAUSAL, scale) }
    }

    pub fn vdn_window(scale: Option<f32>, mask: VdnWindow) -> Self {
        Self { window: Some(mask), ..Self::of(ffi::FV_PLAN_VDN_WINDOW, scale) }
    }

    pub fn kv_window() -> Self {
        Self::of(ffi::FV_PLAN_KV_WINDOW, None)
    }

    pub fn kv_window_with(flash: bool) -> Self {
        Self { kv_flash: Some(flash), ..Self::of(ffi::FV_PLAN_KV_WINDOW, None) }
    }
}

/// Scaled dot-product attention over BHSD `q [b, h, sq, d]`, `k` / `v` `[b, h, sk, d]`, as `plan`
/// says (`rt/sdpa.rs:141`). The result is a new device tensor: bf16 under bf16 activations, else f32.
pub fn sdpa(q: &CudaTensor, k: &CudaTensor, v: &CudaTensor, plan: &Plan<'_>) -> Result<CudaTensor> {
    let (dq, dk, dv) = (q.desc()?, k.desc()?, v.desc()?);
    let dm = plan.mask.map(|m| m.desc()).transpose()?;
    let c = plan.causal.unwrap_or(BlockCausal { block_tokens: 0, window: 0, sink: 0 });
    let w = plan.window.unwrap_or(VdnWindow { video_start: 0, frame_tokens: 0, frames: 0, chunk: 0, radius: 0 });
    let fp = FvPlan {
        kind: plan.kind,
        has_scale: plan.scale.is_some() as c_int,
        scale: plan.scale.unwrap_or(0.0),
        mask: dm.as_ref().map_or(ptr::null(), |m| m as *const FvTensor),
        fp8_first: plan.fp8_first as c_int,
        block_tokens: c.block_tokens,
        window: c.window,
        sink: c.sink,
        video_start: w.video_start,
        frame_tokens: w.frame_tokens,
        frames: w.frames,
        chunk: w.chunk,
        radius: w.radius,
        kv_flash: plan.kv_flash.map_or(-1, |f| f as c_int),
    };
    let mut out = FvTensor { data: ptr::null_mut(), dtype: 0, rank: 0, shape: [0; 8], plane_rows: 0 };
    let st = stream();
    // SAFETY: the descriptors point at live device tensors; `out` receives a buffer this call owns.
    let rc = unsafe { ffi::fv_rt_sdpa(&dq, &dk, &dv, &fp, &mut out, st) };
    if rc != FV_OK {
        return Err(msg(last_error()));
    }
    Ok(HipTensor::from_library(out, st))
}

/// `rt/attn.rs:44-54`: the five dims when k and v are both `[b, h, sk, d]` of q's `[b, h, sq, d]`.
fn bhsd(q: &CudaTensor, k: &CudaTensor, v: &CudaTensor) -> Option<(usize, usize, usize, usize, usize)> {
    if q.rank() != 4 || k.rank() != 4 || v.rank() != 4 {
        return None;
    }
    let (b, h, sq, d, sk) = (q.shape[0], q.shape[1], q.shape[2], q.shape[3], k.shape[2]);
    let want = [b, h, sk, d];
    (k.shape == want && v.shape == want).then_some((b, h, sq, sk, d))
}

/// `rt/attn.rs:112-128`.
pub fn mma_sdpa_supported(b: usize, h: usize, sq: usize, sk: usize, d: usize) -> bool {
    // SAFETY: host arithmetic only.
    unsafe { ffi::fv_sdpa_supported(b, h, sq, sk, d) != 0 }
}

enum Mask {
    None,
    Causal(BlockCausal),
    Window(VdnWindow),
}

/// One fused launch on bf16 operands; `Ok(None)` = the kernel declines (shape, dtype, parameters).
fn fused(q: &CudaTensor, k: &CudaTensor, v: &CudaTensor, scale: Option<f32>, out_bf16: bool, mask: Mask) -> Result<Option<CudaTensor>> {
    let Some((b, h, sq, sk, d)) = bhsd(q, k, v) else {
        return Ok(None);
    };
    if !mma_sdpa_supported(b, h, sq, sk, d) {
        return Ok(None);
    }
    // the fused kernels read bf16; f32 operands are rounded once (RNE), as the reference does. With the fold
    // switch on (fv_rt_fold_scale: FASTVIDEO_SDPA_FOLD_SCALE=1, off by default) an f32 q is rounded as
    // q * (scale * log2(e)) and the kernel then runs at ln 2, its form without the per-score multiply.
    let mut scale = scale.unwrap_or(1.0 / (d as f32).sqrt());
    let mut q_mul = 1.0f32;
    // SAFETY: reads a per-thread flag / host arithmetic only.
    if q.dtype == TensorDType::F32 && unsafe { ffi::fv_rt_fold_scale() != 0 && ffi::fv_sdpa_is_log2_domain_scale(scale) == 0 } {
        let c = scale * std::f32::consts::LOG2_E;
        if c > 0.0 && c < 3.0e38 {
            q_mul = c;
            scale = ffi::FV_SDPA_SCALE_LOG2_DOMAIN;
        }
    }
    let (tq, tk, tv);
    let as_bf16 = |t: &CudaTensor, mul: f32| -> Result<Option<CudaTensor>> {
        if t.dtype == TensorDType::Bf16 {
            return Ok(None);
        }
        let c = HipTensor::alloc(t.shape.clone(), TensorDType::Bf16)?;
        // SAFETY: both buffers hold numel() elements on the current device.
        let rc = unsafe { ffi::fv_cast_f32_bf16_scaled(t.device_ptr().cast_const().cast(), c.device_ptr().cast(), t.numel(), mul, stream()) };
        if rc != FV_OK {
            return Err(msg(last_error()));
        }
        Ok(Some(c))
    };
    if q.plane_rows != 0 || k.plane_rows != 0 || v.plane_rows != 0 {
        if !matches!(mask, Mask::None) {
            return Ok(None); // only the dense entry reads row windows in place
        }
        if q.dtype != TensorDType::Bf16 || k.dtype != TensorDType::Bf16 || v.dtype != TensorDType::Bf16 {
            return Ok(None);
        }
    }
    tq = as_bf16(q, q_mul)?;
    tk = as_bf16(k, 1.0)?;
    tv = as_bf16(v, 1.0)?;
    let (pq, pk, pv) = (
        tq.as_ref().unwrap_or(q).device_ptr().cast_const().cast::<u16>(),
        tk.as_ref().unwrap_or(k).device_ptr().cast_const().cast::<u16>(),
        tv.as_ref().unwrap_or(v).device_ptr().cast_const().cast::<u16>(),
    );
    let out = HipTensor::alloc(vec![b, h, sq, d], if out_bf16 { TensorDType::Bf16 } else { TensorDType::F32 })?;
    let st = stream();
    // SAFETY: operand pointers address [b*h, s, d] bf16 planes, `out` the [b*h, sq, d] result.
    let rc = unsafe {
        match mask {
            Mask::None => ffi::fv_sdpa_dense_bf16_strided(
                pq, pk, pv, out.device_ptr(), out_bf16 as c_int, b * h, sq, sk, d, scale, q.plane_rows, k.plane_rows, v.plane_rows, st,
            ),
            Mask::Causal(m) => ffi::fv_sdpa_block_causal_bf16(
                pq, pk, pv, out.device_ptr(), out_bf16 as c_int, b * h, sq, sk, d, scale, m.block_tokens, m.window, m.sink, st,
            ),
            Mask::Window(m) => ffi::fv_sdpa_vdn_window_bf16(
                pq, pk, pv, out.device_ptr(), out_bf16 as c_int, b * h, sq, sk, d, scale, m.video_start, m.frame_tokens, m.frames, m.chunk,
                m.radius, st,
            ),
        }
    };
    match rc {
        FV_OK => Ok(Some(out)),
        FV_DECLINED => Ok(None),
        _ => Err(msg(last_error())),
    }
}

/// Fused dense SDPA on the matrix cores (`rt/attn.rs:225`): bf16 Q/K/V, f32 online softmax, bf16 P, f32
/// accumulation, one launch, no score buffer. `None` when the kernel does not take the call.
pub fn device_mma_sdpa(q: &CudaTensor, k: &CudaTensor, v: &CudaTensor, scale: Option<f32>, out_bf16: bool) -> Result<Option<CudaTensor>> {
    fused(q, k, v, scale, out_bf16, Mask::None)
}

/// The same under a block-causal mask (`rt/attn.rs:652`).
pub fn device_mma_sdpa_causal(
    q: &CudaTensor,
    k: &CudaTensor,
    v: &CudaTensor,
    scale: Option<f32>,
    out_bf16: bool,
    mask: BlockCausal,
) -> Result<Option<CudaTensor>> {
    fused(q, k, v, scale, out_bf16, Mask::Causal(mask))
}

/// The same under VDN-H3's window mask (`rt/attn.rs:526`).
pub fn device_mma_sdpa_window(
    q: &CudaTensor,
    k: &CudaTensor,
    v: &CudaTensor,
    scale: Option<f32>,
    out_bf16: bool,
    mask: VdnWindow,
) -> Result<Option<CudaTensor>> {
    fused(q, k, v, scale, out_bf16, Mask::Window(mask))
}

/// `rt/vsa.rs:29-109` `TilePlan` + `rt/ops.rs:817-822` `VsaPlanDev`: the tile geometry of a latent grid,
/// host copy and device copy.
pub struct VsaPlanDev {
    pub slot_src: HipSlice<i32>,
    pub block_sizes: HipSlice<i32>,
    pub num_tiles: usize,
    pub tile_elems: usize,
    pub seq: usize,
    pub padded: usize,
}

/// Builds and uploads the plan of grid `(t, h, w)`.
pub fn vsa_plan_upload(t: usize, h: usize, w: usize) -> Result<VsaPlanDev> {
    let mut dims = [0usize; 5];
    // SAFETY: a sizing call: null arrays, `dims` receives {tiles_t, tiles_h, tiles_w, seq, padded}.
    let rc = unsafe { ffi::fv_vsa_tile_plan(t, h, w, dims.as_mut_ptr(), ptr::null_mut(), ptr::null_mut(), ptr::null_mut()) };
    if rc != FV_OK {
        return Err(msg(last_error()));
    }
    let (num_tiles, seq, padded) = (dims[0] * dims[1] * dims[2], dims[3], dims[4]);
    let mut slot_src = vec![0i32; padded];
    let mut token_slot = vec![0u32; seq];
    let mut block_sizes = vec![0i32; num_tiles];
    // SAFETY: the arrays have the sizes the sizing call reported.
    let rc = unsafe { ffi::fv_vsa_tile_plan(t, h, w, dims.as_mut_ptr(), slot_src.as_mut_ptr(), token_slot.as_mut_ptr(), block_sizes.as_mut_ptr()) };
    if rc != FV_OK {
        return Err(msg(last_error()));
    }
    Ok(VsaPlanDev {
        slot_src: HipSlice::from_host(&slot_src)?,
        block_sizes: HipSlice::from_host(&block_sizes)?,
        num_tiles,
        tile_elems: 64,
        seq,
        padded,
    })
}

/// `rt/vsa.rs:480-530` `topk_for`.
pub fn topk_for(sparsity: f64, num_tiles: usize) -> usize {
    // SAFETY: host arithmetic only.
    unsafe { ffi::fv_vsa_topk_for(sparsity, num_tiles) }
}

/// Video Sparse Attention on the device (`rt/vsa.rs:358`): q / k / v / gate `[bh, seq, dim]` f32,
/// result `[bh, seq, dim]` f32. `group` (the reference's bound on its gathered K/V buffer) has no
/// meaning here: the fine stage reads the selected tiles in place.
pub fn vsa_attention_device(
    q: &HipSlice<f32>,
    k: &HipSlice<f32>,
    v: &HipSlice<f32>,
    gate: Option<&HipSlice<f32>>,
    plan: &VsaPlanDev,
    topk: usize,
    bh: usize,
    seq: usize,
    dim: usize,
    scale: f32,
    group: usize,
) -> Result<HipSlice<f32>> {
    let _ = group;
    let nb = plan.num_tiles;
    let topk = topk.clamp(1, nb);
    let want = bh * seq * dim;
    if q.len() != want || k.len() != want || v.len() != want || gate.is_some_and(|g| g.len() != want) {
        return Err(msg("vsa: operand length differs from bh * seq * dim"));
    }
    // SAFETY: host arithmetic only.
    let ws_bytes = unsafe { ffi::fv_vsa_workspace_bytes(bh, nb, topk, dim) };
    let mut ws = HipSlice::<u8>::alloc(ws_bytes + 256)?;
    let ws_ptr = ((ws.as_mut_ptr() as usize + 255) & !255usize) as *mut c_void;
    let mut out = HipSlice::<f32>::alloc(want)?;
    // SAFETY: every pointer addresses a live device buffer of the size the header states.
    let rc = unsafe {
        ffi::fv_vsa_attention(
            q.as_ptr().cast(),
            k.as_ptr().cast(),
            v.as_ptr().cast(),
            0,
            gate.map_or(ptr::null(), |g| g.as_ptr().cast()),
            0,
            plan.slot_src.as_ptr(),
            plan.block_sizes.as_ptr(),
            out.as_mut_ptr(),
            ws_ptr,
            ws_bytes,
            ptr::null_mut(),
            bh,
            seq,
            nb,
            topk,
            dim,
            scale,
            stream(),
        )
    };
    match rc {
        FV_OK => Ok(out),
        FV_DECLINED => Err(msg(format!("vsa: the device path declined: {}", last_error()))),
        _ => Err(msg(last_error())),
    }
}

/// `rt/tensor.rs:61-76` `bf16_activations` / `with_bf16_act`.
pub fn bf16_activations() -> bool {
    // SAFETY: reads a per-thread flag of the library.
    unsafe { ffi::fv_rt_bf16_activations() != 0 }
}

pub fn with_bf16_act<R>(on: bool, f: impl FnOnce() -> R) -> R {
    let prev = bf16_activations();
    // SAFETY: sets / restores a per-thread flag of the library.
    unsafe { ffi::fv_rt_set_bf16_activations(on as c_int) };
    let out = f();
    unsafe { ffi::fv_rt_set_bf16_activations(prev as c_int) };
    out
}
