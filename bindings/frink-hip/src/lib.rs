//! FFI over `libfrink_hip` (include/frink_hip.h) and the safe wrappers Frink's backend seam calls.
//!
//! Each wrapper names the function of the reference it stands in for.  The crate mirrors
//! `frink-cuda`'s public surface for the quantized-matmul path: capability queries, the host-slice
//! launches `BackendDispatch` needs, and resident handles + device-pointer calls for a decode or
//! prefill stack that keeps activations on the GPU.
//!
//! Never compiled in the library's own repository (no Rust toolchain there); the same C ABI is
//! driven from C++ and Python by its tests.
#![cfg(feature = "hip")]
#![allow(clippy::too_many_arguments)]

use std::ffi::{c_char, c_int, c_void, CStr};

#[repr(C)]
pub struct FrkWeights {
    _p: [u8; 0],
}
#[repr(C)]
pub struct FrkBatchActs {
    _p: [u8; 0],
}

#[repr(C)]
pub struct FrkDeviceInfo {
    pub device_count: i32,
    pub compute_units: i32,
    pub name: [c_char; 128],
    pub gcn_arch: [c_char; 64],
    pub total_vram_bytes: u64,
    pub free_vram_bytes: u64,
}

/// `frink_cuda::matvec_launch::MatvecLaunch` as the C side takes it.
#[repr(C)]
pub struct FrkMatvecLaunch {
    pub kind: c_int,
    pub weights: *const u8,
    pub weights_len: usize,
    pub rows: usize,
    pub row_bytes: usize,
}

pub const ACT_F32: c_int = 0;
pub const ACT_INT8: c_int = 1;
/// K-quants on dequantized weights and the f32 activation (the reference's default x86 decode numerics).
pub const ACT_F32_DOT: c_int = 2;

pub const ERR_NO_DEVICE: c_int = -1;
pub const ERR_UNSUPPORTED: c_int = -2;

extern "C" {
    fn frk_hip_probe(out: *mut FrkDeviceInfo) -> c_int;
    fn frk_hip_dense_enabled() -> c_int;
    fn frk_hip_last_error() -> *const c_char;
    fn frk_hip_matvec_kernel(kind: c_int) -> *const c_char;
    fn frk_hip_gemm_supported(kind: c_int) -> c_int;
    fn frk_hip_has_launch(kind: c_int) -> c_int;
    fn frk_hip_block_bytes(kind: c_int) -> c_int;
    fn frk_hip_block_elems(kind: c_int) -> c_int;
    fn frk_hip_worth_a_gemm(batch: usize) -> c_int;

    // host slices in, host slices out (the BackendDispatch seam)
    fn frk_hip_launch_matvec(kind: c_int, weights: *const u8, weights_len: usize, x: *const f32, x_len: usize,
                             rows: usize, row_bytes: usize, out: *mut f32) -> c_int;
    fn frk_hip_launch_mul_mm(kind: c_int, weights: *const u8, weights_len: usize, x: *const f32, x_len: usize,
                             n_rows: usize, n_cols: usize, batch: usize, row_bytes: usize, out: *mut f32) -> c_int;
    fn frk_hip_launch_matvec_multi(x: *const f32, x_len: usize, launches: *const FrkMatvecLaunch, n: usize,
                                   outs: *const *mut f32) -> c_int;
    fn frk_hip_launch_dense_ffn_swiglu(gate: *const FrkMatvecLaunch, up: *const FrkMatvecLaunch,
                                       down: *const FrkMatvecLaunch, x: *const f32, x_len: usize, out: *mut f32) -> c_int;
    fn frk_hip_get_rows(w: *const FrkWeights, ids: *const i32, n_ids: usize, out: *mut f32) -> c_int;

    // resident weights
    fn frk_hip_weights_register(kind: c_int, bytes: *const c_void, len: usize, rows: usize, cols: usize,
                                out: *mut *mut FrkWeights) -> c_int;
    fn frk_hip_weights_from_device(kind: c_int, dev_bytes: *const c_void, len: usize, rows: usize, cols: usize,
                                   stream: *mut c_void, out: *mut *mut FrkWeights) -> c_int;
    fn frk_hip_weights_release(w: *mut FrkWeights) -> c_int;
    fn frk_hip_weights_keep_decoded(w: *mut FrkWeights, stream: *mut c_void) -> c_int;
    fn frk_hip_weights_rows(w: *const FrkWeights) -> usize;
    fn frk_hip_weights_cols(w: *const FrkWeights) -> usize;
    fn frk_hip_weights_kind(w: *const FrkWeights) -> c_int;

    // device pointers, asynchronous on a hipStream_t (or null)
    fn frk_hip_gemv_dev(w: *const FrkWeights, x: *const f32, y: *mut f32, act_mode: c_int, stream: *mut c_void) -> c_int;
    fn frk_hip_gemv_q8k_dev(w: *const FrkWeights, q: *const i8, d: *const f32, bsums: *const i16, y: *mut f32,
                            stream: *mut c_void) -> c_int;
    fn frk_hip_gemv_multi_dev(ws: *const *const FrkWeights, n: usize, x: *const f32, ys: *const *mut f32,
                              stream: *mut c_void) -> c_int;
    fn frk_hip_ffn_swiglu_dev(gate: *const FrkWeights, up: *const FrkWeights, down: *const FrkWeights, x: *const f32,
                              y: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_gemm_dev(w: *const FrkWeights, x: *const f32, batch: usize, y: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_gemm_q8k_dev(w: *const FrkWeights, q: *const i8, d: *const f32, bsums: *const i16, batch: usize,
                            y: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_gemm_pair_dev(w0: *const FrkWeights, w1: *const FrkWeights, x: *const f32, batch: usize, y0: *mut f32,
                             y1: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_gemm_noalloc_dev(w: *const FrkWeights, x: *const f32, batch: usize, y: *mut f32,
                                stream: *mut c_void) -> c_int;
    fn frk_hip_batch_acts_create(max_batch: usize, cols: usize, out: *mut *mut FrkBatchActs) -> c_int;
    fn frk_hip_batch_acts_release(acts: *mut FrkBatchActs) -> c_int;
    fn frk_hip_quantize_batch_acts_dev(acts: *mut FrkBatchActs, x: *const f32, batch: usize, stream: *mut c_void) -> c_int;
    fn frk_hip_gemm_acts_dev(w: *const FrkWeights, acts: *const FrkBatchActs, y: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_gemm_grouped_dev(stacked: *const FrkWeights, n_groups: usize, group_off: *const i32, gather: *const i32,
                                x: *const f32, x_rows: usize, pairs: usize, y: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_route_top_k_softmax_dev(logits: *const f32, batch: usize, n_experts: usize, k: usize, norm: c_int,
                                       ids: *mut i32, weights: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_moe_ffn_dev(gate: *const FrkWeights, up: *const FrkWeights, down: *const FrkWeights, n_experts: usize,
                           x: *const f32, batch: usize, ids: *const i32, weights: *const f32, k: usize,
                           out: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_quantize_q8_k_dev(x: *const f32, n: usize, q: *mut i8, d: *mut f32, bsums: *mut i16,
                                 stream: *mut c_void) -> c_int;
    fn frk_hip_dequant_dev(w: *const FrkWeights, out: *mut f32, stream: *mut c_void) -> c_int;
    fn frk_hip_get_rows_dev(w: *const FrkWeights, ids: *const i32, n_ids: usize, out: *mut f32,
                            stream: *mut c_void) -> c_int;
}

#[derive(Debug, Clone)]
pub struct HipError {
    pub status: i32,
    pub message: String,
}
impl std::fmt::Display for HipError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        write!(f, "frink-hip: {} (status {})", self.message, self.status)
    }
}
impl std::error::Error for HipError {}

fn check(rc: c_int) -> Result<(), HipError> {
    if rc == 0 {
        return Ok(());
    }
    // thread-local on the C side: the message belongs to this thread's last failed call
    let message = unsafe { CStr::from_ptr(frk_hip_last_error()) }.to_string_lossy().into_owned();
    Err(HipError { status: rc, message })
}

/// ggml type id of the kinds this backend has kernels for, keyed by `QuantKind::name()`
/// (crates/frink-core/src/weight_matrix.rs:264-290), so the table cannot drift from the C side.
pub fn kind_id(name: &str) -> Option<c_int> {
    match name {
        "Q4_0" => Some(2),
        "Q5_0" => Some(6),
        "Q8_0" => Some(8),
        "Q4_K" => Some(12),
        "Q5_K" => Some(13),
        "Q6_K" => Some(14),
        "IQ4_XS" => Some(23),
        "MXFP4" => Some(39),
        _ => None,
    }
}

// ---- BackendCaps / BackendDispatch queries (gpu_backend.rs:110-195) ----
pub fn matvec_kernel(kind: c_int) -> Option<&'static str> {
    let p = unsafe { frk_hip_matvec_kernel(kind) };
    if p.is_null() {
        None
    } else {
        unsafe { CStr::from_ptr(p) }.to_str().ok()
    }
}
pub fn gemm_supported(kind: c_int) -> bool {
    unsafe { frk_hip_gemm_supported(kind) != 0 }
}
pub fn has_launch(kind: c_int) -> bool {
    unsafe { frk_hip_has_launch(kind) != 0 }
}
/// `FRINK_HIP=0|false|off|cpu` switches the backend off without opening a device (env_or_probe's grammar).
pub fn dense_enabled() -> bool {
    unsafe { frk_hip_dense_enabled() != 0 }
}
pub fn worth_a_gemm(batch: usize) -> bool {
    unsafe { frk_hip_worth_a_gemm(batch) != 0 }
}
pub fn block_geometry(kind: c_int) -> Option<(usize, usize)> {
    let (b, e) = unsafe { (frk_hip_block_bytes(kind), frk_hip_block_elems(kind)) };
    (b > 0 && e > 0).then_some((b as usize, e as usize))
}
/// `frink_cuda::gpu::probe` (crates/frink-cuda/src/gpu.rs:79-145).
pub fn probe() -> Result<FrkDeviceInfo, HipError> {
    let mut info = std::mem::MaybeUninit::<FrkDeviceInfo>::zeroed();
    check(unsafe { frk_hip_probe(info.as_mut_ptr()) })?;
    Ok(unsafe { info.assume_init() })
}

// ---- host slices (what impl BackendDispatch for Hip calls) ----

/// `frink_cuda::gpu::launch_q4_k_matvec` and siblings (gpu.rs:319-446).
pub fn launch_matvec(kind: c_int, weights: &[u8], x: &[f32], rows: usize, row_bytes: usize) -> Result<Vec<f32>, HipError> {
    let mut out = vec![0f32; rows];
    check(unsafe {
        frk_hip_launch_matvec(kind, weights.as_ptr(), weights.len(), x.as_ptr(), x.len(), rows, row_bytes, out.as_mut_ptr())
    })?;
    Ok(out)
}

/// `frink_cuda::mul_mm_launch::launch_mul_mm` (mul_mm_launch.rs:40-68): `out[token * n_rows + row]`.
pub fn launch_mul_mm(kind: c_int, weights: &[u8], x_batch: &[f32], n_rows: usize, n_cols: usize, batch: usize,
                     row_bytes: usize) -> Result<Vec<f32>, HipError> {
    let mut out = vec![0f32; n_rows * batch];
    check(unsafe {
        frk_hip_launch_mul_mm(kind, weights.as_ptr(), weights.len(), x_batch.as_ptr(), x_batch.len(), n_rows, n_cols,
                              batch, row_bytes, out.as_mut_ptr())
    })?;
    Ok(out)
}

/// One matvec of a group that shares an activation (`MatvecLaunch`, matvec_launch.rs:485-493).
pub struct MatvecLaunch<'a> {
    pub kind: c_int,
    pub weights: &'a [u8],
    pub rows: usize,
    pub row_bytes: usize,
}
impl MatvecLaunch<'_> {
    fn raw(&self) -> FrkMatvecLaunch {
        FrkMatvecLaunch { kind: self.kind, weights: self.weights.as_ptr(), weights_len: self.weights.len(), rows: self.rows,
                          row_bytes: self.row_bytes }
    }
}

/// `frink_cuda::matvec_launch::launch_matvec_multi` (matvec_launch.rs:500-534): one upload of `x`,
/// n matvecs on resident weights (the K-quant matrices share one Q8_K quantization), n downloads.
pub fn launch_matvec_multi(x: &[f32], launches: &[MatvecLaunch<'_>]) -> Result<Vec<Vec<f32>>, HipError> {
    let raw: Vec<FrkMatvecLaunch> = launches.iter().map(MatvecLaunch::raw).collect();
    let mut outs: Vec<Vec<f32>> = launches.iter().map(|l| vec![0f32; l.rows]).collect();
    let ptrs: Vec<*mut f32> = outs.iter_mut().map(|o| o.as_mut_ptr()).collect();
    check(unsafe { frk_hip_launch_matvec_multi(x.as_ptr(), x.len(), raw.as_ptr(), raw.len(), ptrs.as_ptr()) })?;
    Ok(outs)
}

/// `frink_cuda::matvec_launch::launch_dense_ffn_swiglu` (matvec_launch.rs:551-570):
/// `down(silu(gate x) * up x)` with one upload and one download.
pub fn launch_dense_ffn_swiglu(gate: &MatvecLaunch<'_>, up: &MatvecLaunch<'_>, down: &MatvecLaunch<'_>, x: &[f32])
    -> Result<Vec<f32>, HipError> {
    let mut out = vec![0f32; down.rows];
    let (g, u, d) = (gate.raw(), up.raw(), down.raw());
    check(unsafe { frk_hip_launch_dense_ffn_swiglu(&g, &u, &d, x.as_ptr(), x.len(), out.as_mut_ptr()) })?;
    Ok(out)
}

// ---- resident weights and device pointers ----

/// One weight matrix resident in HBM (`frink_cuda::resident`, crates/frink-cuda/src/resident.rs).
pub struct Weights(*mut FrkWeights);
unsafe impl Send for Weights {}
unsafe impl Sync for Weights {}
impl Weights {
    /// Host GGUF bytes; cached by (pointer, length, 192 sampled bytes) like the reference's cache.
    pub fn register(kind: c_int, bytes: &[u8], rows: usize, cols: usize) -> Result<Self, HipError> {
        let mut w = std::ptr::null_mut();
        check(unsafe { frk_hip_weights_register(kind, bytes.as_ptr() as *const c_void, bytes.len(), rows, cols, &mut w) })?;
        Ok(Weights(w))
    }
    /// GGUF bytes already on the device (`len` bytes at `dev_bytes`), copied into the resident layout on `stream`.
    ///
    /// # Safety
    /// `dev_bytes` must be a device pointer to `len` readable bytes.
    pub unsafe fn from_device(kind: c_int, dev_bytes: *const c_void, len: usize, rows: usize, cols: usize,
                              stream: *mut c_void) -> Result<Self, HipError> {
        let mut w = std::ptr::null_mut();
        check(frk_hip_weights_from_device(kind, dev_bytes, len, rows, cols, stream, &mut w))?;
        Ok(Weights(w))
    }
    pub fn rows(&self) -> usize { unsafe { frk_hip_weights_rows(self.0) } }
    pub fn cols(&self) -> usize { unsafe { frk_hip_weights_cols(self.0) } }
    pub fn kind(&self) -> c_int { unsafe { frk_hip_weights_kind(self.0) } }
    pub fn raw(&self) -> *const FrkWeights { self.0 }
    /// Q5_0 / IQ4_XS / MXFP4: keep the rows decoded for the matrix cores beside the resident copy (decodes on
    /// `stream` and synchronizes it); batched calls then skip their per-call decoding.
    pub fn keep_decoded(&mut self, stream: *mut c_void) -> Result<(), HipError> {
        check(unsafe { frk_hip_weights_keep_decoded(self.0, stream) })
    }

    /// `WeightMatrix::dequant_row` / get_rows (crates/frink-cuda/src/get_rows.rs): host ids, host rows.
    pub fn get_rows(&self, ids: &[i32]) -> Result<Vec<f32>, HipError> {
        let mut out = vec![0f32; ids.len() * self.cols()];
        check(unsafe { frk_hip_get_rows(self.0, ids.as_ptr(), ids.len(), out.as_mut_ptr()) })?;
        Ok(out)
    }
}
impl Drop for Weights {
    fn drop(&mut self) {
        unsafe { frk_hip_weights_release(self.0) };
    }
}

/// The device-pointer family.  Every pointer is a device pointer; calls are asynchronous on `stream`
/// (a `hipStream_t` or null).  Scratch memory is per stream (one library-owned buffer a stream, held by the calling thread while it
/// enqueues a call's launches; see the comment in front of the device-pointer entry points in frink_hip.h).
pub mod dev {
    use super::*;

    /// # Safety
    /// `x` holds `w.cols()` floats and `y` room for `w.rows()`, both on the device.
    pub unsafe fn gemv(w: &Weights, x: *const f32, y: *mut f32, act_mode: c_int, stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_gemv_dev(w.0, x, y, act_mode, stream))
    }
    /// One Q8_K quantization shared by several projections (matvec_launch.rs:500-534).
    /// # Safety
    /// `q`, `d`, `bsums` are what `quantize_q8_k` wrote for `w.cols()` values.
    pub unsafe fn gemv_q8k(w: &Weights, q: *const i8, d: *const f32, bsums: *const i16, y: *mut f32, stream: *mut c_void)
        -> Result<(), HipError> {
        check(frk_hip_gemv_q8k_dev(w.0, q, d, bsums, y, stream))
    }
    /// `WeightMatrix::apply_gpu_multi` (weight_matrix.rs:3504-3667) on device pointers.
    /// # Safety
    /// `ys[i]` has room for `ws[i].rows()` floats.
    pub unsafe fn gemv_multi(ws: &[&Weights], x: *const f32, ys: &[*mut f32], stream: *mut c_void) -> Result<(), HipError> {
        assert_eq!(ws.len(), ys.len());
        let raw: Vec<*const FrkWeights> = ws.iter().map(|w| w.0 as *const FrkWeights).collect();
        check(frk_hip_gemv_multi_dev(raw.as_ptr(), raw.len(), x, ys.as_ptr(), stream))
    }
    /// `WeightMatrix::apply_gpu_dense_ffn_swiglu` (weight_matrix.rs:3676-3760) on device pointers.
    /// # Safety
    /// `x` holds `gate.cols()` floats, `y` room for `down.rows()`.
    pub unsafe fn ffn_swiglu(gate: &Weights, up: &Weights, down: &Weights, x: *const f32, y: *mut f32, stream: *mut c_void)
        -> Result<(), HipError> {
        check(frk_hip_ffn_swiglu_dev(gate.0, up.0, down.0, x, y, stream))
    }
    /// `WeightMatrix::apply_batch_with_acts` (weight_matrix.rs:2481): `y[batch][rows]`.
    /// # Safety
    /// `x` holds `batch * w.cols()` floats, `y` room for `batch * w.rows()`.
    pub unsafe fn gemm(w: &Weights, x: *const f32, batch: usize, y: *mut f32, stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_gemm_dev(w.0, x, batch, y, stream))
    }
    /// `apply_batch_with_acts` with `BatchActs::Q8K` (weight_matrix.rs:2481-2487, 757-768) for a thin batch: the
    /// activations are Q8_K already (`q [batch][cols]`, `d [batch][cols/256]`, `bsums [batch][cols/16]`).
    /// `Unsupported` beyond the rows the thin kernels take for the matrix.
    /// # Safety
    /// device pointers of those sizes; `y` has room for `batch * w.rows()` floats.
    pub unsafe fn gemm_q8k(w: &Weights, q: *const i8, d: *const f32, bsums: *const i16, batch: usize, y: *mut f32,
                           stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_gemm_q8k_dev(w.0, q, d, bsums, batch, y, stream))
    }
    /// `WeightMatrix::apply_batch_pair_with_acts` (weight_matrix.rs:2447-2479): gate and up of a prefill
    /// FFN over one quantization of the batch.
    /// # Safety
    /// as `gemm`, for both outputs.
    pub unsafe fn gemm_pair(w0: &Weights, w1: &Weights, x: *const f32, batch: usize, y0: *mut f32, y1: *mut f32,
                            stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_gemm_pair_dev(w0.0, w1.0, x, batch, y0, y1, stream))
    }
    /// `gemm` for callers that cannot allocate (graph capture, serving loops): a fixed 16 MiB scratch in
    /// the library's device image; larger shapes are refused; calls that overlap on one GPU race.
    /// # Safety
    /// as `gemm`.
    pub unsafe fn gemm_noalloc(w: &Weights, x: *const f32, batch: usize, y: *mut f32, stream: *mut c_void)
        -> Result<(), HipError> {
        check(frk_hip_gemm_noalloc_dev(w.0, x, batch, y, stream))
    }
    /// `BatchActs::Q8K` (weight_matrix.rs:757-768) on the device: a batch quantized once for any number of
    /// matrices of `cols` columns, at any batch size up to `max_batch`.
    pub struct BatchActs(pub(crate) *mut FrkBatchActs);
    impl BatchActs {
        pub fn new(max_batch: usize, cols: usize) -> Result<Self, HipError> {
            let mut p = std::ptr::null_mut();
            check(unsafe { frk_hip_batch_acts_create(max_batch, cols, &mut p) })?;
            Ok(BatchActs(p))
        }
        /// `quantize_batch_acts` (weight_matrix.rs:2348-2426).
        /// # Safety
        /// `x` holds `batch * cols` floats on the device.
        pub unsafe fn quantize(&mut self, x: *const f32, batch: usize, stream: *mut c_void) -> Result<(), HipError> {
            check(frk_hip_quantize_batch_acts_dev(self.0, x, batch, stream))
        }
    }
    impl Drop for BatchActs {
        fn drop(&mut self) {
            unsafe { frk_hip_batch_acts_release(self.0) };
        }
    }
    /// `apply_batch_with_acts` (weight_matrix.rs:2481-2487) over a `BatchActs`: `y[batch][rows]`, bit for bit `gemm`.
    /// # Safety
    /// `y` has room for the quantized batch times `w.rows()` floats.
    pub unsafe fn gemm_acts(w: &Weights, acts: &BatchActs, y: *mut f32, stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_gemm_acts_dev(w.0, acts.0, y, stream))
    }
    /// The grouped GEMM (`enqueue_mul_mm_grouped_dev`, crates/frink-cuda/src/mul_mm_launch.rs:391-470): group `g` is
    /// rows `[g*R, (g+1)*R)` of `stacked`; pair `p` of group `g` reads row `gather[p]` of `x` (row `p` when `gather`
    /// is null) and writes `y[p][R]`.
    /// # Safety
    /// `group_off[n_groups + 1]`, `gather[pairs]` (or null), `x[x_rows][cols]`, `y[pairs][R]` on the device.
    pub unsafe fn gemm_grouped(stacked: &Weights, n_groups: usize, group_off: *const i32, gather: *const i32, x: *const f32,
                               x_rows: usize, pairs: usize, y: *mut f32, stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_gemm_grouped_dev(stacked.0, n_groups, group_off, gather, x, x_rows, pairs, y, stream))
    }
    /// `frink_moe::route_top_k_softmax` (crates/frink-moe/src/lib.rs:567-589) for a batch of tokens.
    /// # Safety
    /// `logits[batch][n_experts]`, `ids[batch][k]`, `weights[batch][k]` on the device.
    pub unsafe fn route_top_k_softmax(logits: *const f32, batch: usize, n_experts: usize, k: usize, norm: bool,
                                      ids: *mut i32, weights: *mut f32, stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_route_top_k_softmax_dev(logits, batch, n_experts, k, norm as c_int, ids, weights, stream))
    }
    /// `Decoder::moe_ffn_batch` (crates/frink-models/src/decoder/ffn_batch.rs:343-434) in one call.
    /// # Safety
    /// `x[batch][hidden]`, `ids`/`weights[batch][k]`, `out[batch][hidden]` on the device.
    pub unsafe fn moe_ffn(gate: &Weights, up: &Weights, down: &Weights, n_experts: usize, x: *const f32, batch: usize,
                          ids: *const i32, weights: *const f32, k: usize, out: *mut f32, stream: *mut c_void)
        -> Result<(), HipError> {
        check(frk_hip_moe_ffn_dev(gate.0, up.0, down.0, n_experts, x, batch, ids, weights, k, out, stream))
    }
    /// `quantize_activations_q8_k` (crates/frink-quant/src/act_quant.rs:69-104) on the device.
    /// # Safety
    /// `x[n]`, `q[n]`, `d[n/256]`, `bsums[n/16]` on the device, `n` a multiple of 256.
    pub unsafe fn quantize_q8_k(x: *const f32, n: usize, q: *mut i8, d: *mut f32, bsums: *mut i16, stream: *mut c_void)
        -> Result<(), HipError> {
        check(frk_hip_quantize_q8_k_dev(x, n, q, d, bsums, stream))
    }
    /// # Safety
    /// `out` has room for `rows * cols` floats.
    pub unsafe fn dequant(w: &Weights, out: *mut f32, stream: *mut c_void) -> Result<(), HipError> {
        check(frk_hip_dequant_dev(w.0, out, stream))
    }
    /// # Safety
    /// `ids[n_ids]` and `out[n_ids][cols]` on the device.
    pub unsafe fn get_rows(w: &Weights, ids: *const i32, n_ids: usize, out: *mut f32, stream: *mut c_void)
        -> Result<(), HipError> {
        check(frk_hip_get_rows_dev(w.0, ids, n_ids, out, stream))
    }
}
