//! Safe wrappers over `libferric_hip.so` with the signatures and failure modes of the reference's quantized linear
//! path (`crates/ferric-tensor/src/dtype.rs`): `Err(String)` where the reference returns `Err`, a panic where it asserts.
//! Not compiled in the library's own build image (no Rust toolchain there); the C ABI underneath is what its tests drive.
pub mod ffi;

use std::ffi::{c_void, CStr};
use std::ptr;

fn last_error() -> String {
    unsafe { CStr::from_ptr(ffi::fhip_last_error()).to_string_lossy().into_owned() }
}

/// Maps a return code the way the reference behaves at the same spot.
fn check(rc: i32) -> Result<(), String> {
    match rc {
        ffi::FHIP_OK => Ok(()),
        ffi::FHIP_ERR_SHAPE => panic!("{}", last_error()), // the reference's assert!/assert_eq!
        _ => Err(last_error()),
    }
}

/// Selects the GPU (`fhip_init`); call once before anything else.
pub fn init(device: i32) -> Result<(), String> {
    check(unsafe { ffi::fhip_init(device) })
}

/// `ferric_gguf::type_size` (crates/ferric-gguf/src/lib.rs:460): bytes of `n` elements, 0 for an unknown type.
pub fn type_size(ggml_type: u32, n: usize) -> usize {
    unsafe { ffi::fhip_type_size(ggml_type, n) }
}

/// `ferric_gguf::deq_raw` (crates/ferric-gguf/src/lib.rs:497) on the GPU, host slices on both sides.
pub fn deq_raw(raw: &[u8], n: usize, ggml_type: u32) -> Result<Vec<f32>, String> {
    let mut out = vec![0f32; n];
    let mut written = 0usize;
    check(unsafe { ffi::fhip_deq_raw(raw.as_ptr(), raw.len(), n, ggml_type, out.as_mut_ptr(), &mut written) })?;
    out.truncate(written);
    Ok(out)
}

/// A device buffer of f32 (activations, outputs, workspaces).
pub struct DeviceF32 {
    ptr: *mut f32,
    len: usize,
}
impl DeviceF32 {
    pub fn zeros(len: usize) -> Result<Self, String> {
        let mut p: *mut c_void = ptr::null_mut();
        check(unsafe { ffi::fhip_malloc(&mut p, len.max(1) * 4) })?;
        check(unsafe { ffi::fhip_memset(p, 0, len * 4, ptr::null_mut()) })?;
        Ok(Self { ptr: p as *mut f32, len })
    }
    pub fn from_slice(v: &[f32]) -> Result<Self, String> {
        let mut p: *mut c_void = ptr::null_mut();
        check(unsafe { ffi::fhip_malloc(&mut p, v.len().max(1) * 4) })?;
        check(unsafe { ffi::fhip_memcpy_h2d(p, v.as_ptr() as *const c_void, v.len() * 4, ptr::null_mut()) })?;
        Ok(Self { ptr: p as *mut f32, len: v.len() })
    }
    pub fn to_vec(&self) -> Result<Vec<f32>, String> {
        let mut v = vec![0f32; self.len];
        check(unsafe { ffi::fhip_memcpy_d2h(v.as_mut_ptr() as *mut c_void, self.ptr as *const c_void, self.len * 4, ptr::null_mut()) })?;
        Ok(v)
    }
    pub fn len(&self) -> usize { self.len }
    pub fn is_empty(&self) -> bool { self.len == 0 }
    pub fn as_ptr(&self) -> *const f32 { self.ptr }
    pub fn as_mut_ptr(&mut self) -> *mut f32 { self.ptr }
}
impl Drop for DeviceF32 {
    fn drop(&mut self) { unsafe { ffi::fhip_free(self.ptr as *mut c_void); } }
}

/// `QMatrix` (crates/ferric-tensor/src/dtype.rs:859-1010) on one GPU: the raw GGUF block bytes resident in HBM, one shard.
pub struct HipQMatrix {
    h: *mut ffi::FhipWeight,
    rows: usize,
    cols: usize,
}
// The handle may move between threads. It is not `Sync`: every method enqueues on the default stream, and the batched paths
// of one stream share that stream's library workspace across the several launches of a call, so two threads enqueueing
// through one handle (or on one stream) at once could interleave those launches. One thread drives one stream, as in the
// reference (its pipeline cache and batch recorder are thread-local, crates/ferric-tensor/src/lib.rs:1515-1532).
unsafe impl Send for HipQMatrix {}

impl HipQMatrix {
    /// `QMatrix::from_bytes` (dtype.rs:893): `Err` for a type without a native matmul, panic on `cols % block` or a wrong
    /// byte length, as `Q4_KWeights::from_bytes` asserts (dtype.rs:1389-1390).
    pub fn from_bytes(bytes: &[u8], ggml_type: u32, rows: usize, cols: usize) -> Result<Self, String> {
        let mut h = ptr::null_mut();
        check(unsafe { ffi::fhip_weight_create(ggml_type, bytes.as_ptr(), bytes.len(), rows, cols, &mut h) })?;
        Ok(Self { h, rows, cols })
    }
    pub fn rows(&self) -> usize { self.rows }
    pub fn cols(&self) -> usize { self.cols }
    pub fn n_shards(&self) -> usize { 1 }
    pub fn nbytes(&self) -> usize { unsafe { ffi::fhip_weight_nbytes(self.h) } }
    /// Activation bits of this weight's streaming mat-vec: 24 as created (the f32 significand; the reference examples' 1e-5
    /// bar), 16 for the faster opt-in. Returns the setting before the call.
    pub fn set_matvec_precision(&mut self, bits: i32) -> Result<i32, String> {
        let rc = unsafe { ffi::fhip_weight_matvec_precision(self.h, bits) };
        if rc < 0 { Err(last_error()) } else { Ok(rc) }
    }
    /// Which kernels batches of three rows and more take (`ffi::FHIP_BATCH_*`; `FHIP_BATCH_ORDERED` as created).
    pub fn set_batch_policy(&mut self, policy: i32) -> i32 { unsafe { ffi::fhip_weight_batch_policy(self.h, policy) } }

    /// `Tensor::matmul_q` (dtype.rs:935): y [rows_x, rows] = x [rows_x, cols] * W^T.
    pub fn matmul_q(&self, x: &DeviceF32, rows_x: usize) -> Result<DeviceF32, String> {
        assert_eq!(x.len(), rows_x * self.cols, "matmul_q: inner dim");
        let mut y = DeviceF32::zeros(rows_x * self.rows)?;
        check(unsafe { ffi::fhip_matmul_q(self.h, x.as_ptr(), rows_x, y.as_mut_ptr(), ptr::null_mut()) })?;
        Ok(y)
    }

    /// `Tensor::try_matmul_swiglu` (dtype.rs:949): `None` where the reference has no fused kernel (Q8_0).
    pub fn try_matmul_swiglu(&self, x: &DeviceF32, rows_x: usize) -> Option<DeviceF32> {
        assert_eq!(x.len(), rows_x * self.cols, "matmul_swiglu: inner dim");
        let mut y = DeviceF32::zeros(rows_x * self.rows / 2).ok()?;
        match unsafe { ffi::fhip_matmul_q_swiglu(self.h, x.as_ptr(), rows_x, y.as_mut_ptr(), ptr::null_mut()) } {
            ffi::FHIP_OK => Some(y),
            ffi::FHIP_ERR_UNSUPPORTED_TYPE => None,
            ffi::FHIP_ERR_SHAPE => panic!("{}", last_error()),
            _ => None,
        }
    }

    /// The FFN block of crates/ferric-llama/src/qwen3.rs:944-964: down(swiglu(gate_up(x))).
    pub fn ffn(gate_up: &HipQMatrix, down: &HipQMatrix, x: &DeviceF32, rows_x: usize) -> Result<DeviceF32, String> {
        assert_eq!(x.len(), rows_x * gate_up.cols, "ffn: inner dim");
        let mut ws = DeviceF32::zeros(rows_x * gate_up.rows / 2)?;
        let mut y = DeviceF32::zeros(rows_x * down.rows)?;
        check(unsafe { ffi::fhip_ffn(gate_up.h, down.h, x.as_ptr(), rows_x, y.as_mut_ptr(), ws.as_mut_ptr(), ptr::null_mut()) })?;
        Ok(y)
    }

    /// Rows `[row0, row0 + nrows)` dequantized (the embedding lookup of crates/ferric-llama/src/qwen3.rs:733-750).
    pub fn dequant_rows(&self, row0: usize, nrows: usize) -> Result<DeviceF32, String> {
        let mut out = DeviceF32::zeros(nrows * self.cols)?;
        check(unsafe { ffi::fhip_dequant_rows(self.h, row0, nrows, out.as_mut_ptr(), ptr::null_mut()) })?;
        Ok(out)
    }
}
impl Drop for HipQMatrix {
    fn drop(&mut self) { unsafe { ffi::fhip_weight_destroy(self.h) } }
}

/// `cpu_simd::matvec_q8_0` (crates/ferric-tensor/src/cpu_simd.rs:79) with the weight streamed by the GPU.
pub fn matvec_q8_0(x: &[f32], w: &[u8], rows: usize, cols: usize) -> Vec<f32> {
    let mut y = vec![0f32; rows];
    assert_eq!(x.len(), cols, "x length");
    if let Err(e) = check(unsafe { ffi::fhip_matvec_q8_0_host(x.as_ptr(), w.as_ptr(), w.len(), rows, cols, y.as_mut_ptr()) }) {
        panic!("{e}");
    }
    y
}
