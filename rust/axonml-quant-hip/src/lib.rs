//! Safe layer over `libaxq.so` with the public names of `axonml-quant`
//! (`crates/axonml-quant/src/lib.rs:35-39`: `QuantError`, `QuantResult`, `quantize_tensor`, `quantize_model`,
//! `dequantize_tensor`, `dequantize_block`, `QuantType`, `QuantizedTensor`), plus what that crate lacks: a device
//! context, a device-resident weight and the quantized matmul.
//!
//! NOT COMPILED in this repository's build or tests: the image this library is built in has no Rust toolchain.
//! The same boundary is exercised by the Python `ctypes` binding and by the C++ host mirror, which are compiled
//! and tested.  Tensors cross this layer as slices plus shapes so that the crate stands without `axonml-tensor`;
//! inside the reference workspace `Tensor<f32>::to_vec()` / `Tensor::from_vec` sit on either side.
//!
//! Differences from the reference crate, all forced by the device library:
//!  * a `QuantizedTensor` holds one flat byte buffer (the blocks' `to_bytes` images in block order) instead of a
//!    `Vec<QuantizedBlock>`;
//!  * `QuantType` has `Q4_K`, `Q6_K` and `Q5_K` (GGUF superblocks) behind `F32`, and `Q5_0` / `Q5_1` have codecs of their own
//!    (`quantize.rs:47-50` sends them to Q4_0);
//!  * every function takes the device context first.
use axonml_quant_hip_sys as sys;
use std::ffi::CStr;
use std::fmt;
use std::os::raw::c_void;

// ---------------------------------------------------------------------------------------------------------------------
// QuantType (types.rs:17-120); discriminants equal `axq_type`
// ---------------------------------------------------------------------------------------------------------------------
#[allow(non_camel_case_types)]
#[derive(Clone, Copy, Debug, PartialEq, Eq, Hash)]
#[repr(i32)]
pub enum QuantType { Q8_0 = 0, Q4_0 = 1, Q4_1 = 2, Q5_0 = 3, Q5_1 = 4, F16 = 5, F32 = 6, Q4_K = 7, Q6_K = 8, Q5_K = 9 }

impl QuantType {
    /// types.rs:45-52
    pub fn block_size(self) -> usize {
        match self { QuantType::F16 | QuantType::F32 => 1, QuantType::Q4_K | QuantType::Q6_K | QuantType::Q5_K => 256, _ => 32 }
    }
    /// types.rs:55-66
    pub fn bytes_per_block(self) -> usize {
        match self {
            QuantType::Q8_0 => 34, QuantType::Q4_0 => 18, QuantType::Q4_1 => 20, QuantType::Q5_0 => 22,
            QuantType::Q5_1 => 24, QuantType::F16 => 2, QuantType::F32 => 4, QuantType::Q4_K => 144, QuantType::Q6_K => 210, QuantType::Q5_K => 176,
        }
    }
    /// types.rs:69-78
    pub fn bits_per_value(self) -> usize {
        match self {
            QuantType::Q8_0 => 8, QuantType::Q4_0 | QuantType::Q4_1 | QuantType::Q4_K => 4,
            QuantType::Q5_0 | QuantType::Q5_1 | QuantType::Q5_K => 5, QuantType::Q6_K => 6, QuantType::F16 => 16, QuantType::F32 => 32,
        }
    }
    /// types.rs:81-83
    pub fn compression_ratio(self) -> f32 { 32.0 / self.bits_per_value() as f32 }
    /// types.rs:86-91
    pub fn is_block_quantized(self) -> bool { !matches!(self, QuantType::F16 | QuantType::F32) }
    /// types.rs:94-105, with the two GGUF names added
    pub fn from_str(s: &str) -> Option<Self> {
        Some(match s.to_uppercase().as_str() {
            "Q8_0" | "Q8" | "INT8" => QuantType::Q8_0,
            "Q4_0" | "Q4" | "INT4" => QuantType::Q4_0,
            "Q4_1" => QuantType::Q4_1,
            "Q5_0" | "Q5" => QuantType::Q5_0,
            "Q5_1" => QuantType::Q5_1,
            "F16" | "FLOAT16" | "HALF" => QuantType::F16,
            "F32" | "FLOAT32" | "FLOAT" => QuantType::F32,
            "Q4_K" | "Q4K" => QuantType::Q4_K,
            "Q6_K" | "Q6K" => QuantType::Q6_K,
            "Q5_K" | "Q5K" => QuantType::Q5_K,
            _ => return None,
        })
    }
}

impl fmt::Display for QuantType {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result { write!(f, "{:?}", self) } // types.rs:108-120
}

// ---------------------------------------------------------------------------------------------------------------------
// QuantError / QuantResult (error.rs:14-60), with the device errors of CudaError (backends/cuda.rs:272-289) behind them
// ---------------------------------------------------------------------------------------------------------------------
#[derive(Debug)]
pub enum QuantError {
    InvalidBlockSize(String),
    InvalidQuantType(String),
    ShapeMismatch(String),
    DataLengthMismatch(String),
    CalibrationError(String),
    Overflow,
    InvalidData(String),
    TensorConversion(String),
    /// status -20 .. -30 of `axq_status`: no device, out of memory, launch or copy failure
    Device { status: i32, message: String },
}
pub type QuantResult<T> = Result<T, QuantError>;

impl fmt::Display for QuantError {
    fn fmt(&self, f: &mut fmt::Formatter<'_>) -> fmt::Result {
        match self {
            QuantError::InvalidBlockSize(m) | QuantError::InvalidQuantType(m) | QuantError::ShapeMismatch(m)
            | QuantError::DataLengthMismatch(m) | QuantError::CalibrationError(m) | QuantError::InvalidData(m)
            | QuantError::TensorConversion(m) => f.write_str(m), // the library words its messages as error.rs does
            QuantError::Overflow => f.write_str("Numerical overflow during quantization"),
            QuantError::Device { status, message } => write!(f, "{message} (status {status})"),
        }
    }
}
impl std::error::Error for QuantError {}

fn check(ctx: *mut sys::axq_ctx, rc: i32) -> QuantResult<()> {
    if rc == 0 { return Ok(()); }
    let msg = unsafe { CStr::from_ptr(sys::axq_last_error(ctx)) }.to_string_lossy().into_owned();
    Err(match rc {
        -1 => QuantError::InvalidBlockSize(msg), -2 => QuantError::InvalidQuantType(msg),
        -3 => QuantError::ShapeMismatch(msg),    -4 => QuantError::DataLengthMismatch(msg),
        -5 => QuantError::CalibrationError(msg), -6 => QuantError::Overflow,
        -7 => QuantError::InvalidData(msg),      -8 => QuantError::TensorConversion(msg),
        s  => QuantError::Device { status: s, message: msg },
    })
}

// ---------------------------------------------------------------------------------------------------------------------
// QuantizedTensor (types.rs:296-352)
// ---------------------------------------------------------------------------------------------------------------------
#[derive(Clone, Debug)]
pub struct QuantizedTensor {
    pub shape: Vec<usize>,
    pub quant_type: QuantType,
    /// the blocks' `to_bytes` images, concatenated in block order
    pub data: Vec<u8>,
}

impl QuantizedTensor {
    pub fn new(shape: Vec<usize>, quant_type: QuantType, data: Vec<u8>) -> Self { Self { shape, quant_type, data } }
    pub fn numel(&self) -> usize { self.shape.iter().product() }                              // types.rs:318-320
    pub fn num_blocks(&self) -> usize { self.data.len() / self.quant_type.bytes_per_block() } // types.rs:335-337
    pub fn size_bytes(&self) -> usize { self.data.len() }                                     // types.rs:323-326
    pub fn compression_ratio(&self) -> f32 { (self.numel() * 4) as f32 / self.size_bytes() as f32 } // types.rs:329-332
}

// ---------------------------------------------------------------------------------------------------------------------
// Device context: one GPU, one stream (the shape of CudaBackend::new, backends/cuda.rs:69-81)
// ---------------------------------------------------------------------------------------------------------------------
pub struct HipQuant { ctx: *mut sys::axq_ctx }
// One stream: calls through one context must not overlap, so the context moves between threads but is not shared.
unsafe impl Send for HipQuant {}

impl HipQuant {
    /// `None` when the device is not an MI355X (gfx950) or the library cannot initialise.
    pub fn new(device: i32) -> Option<Self> {
        let mut ctx = std::ptr::null_mut();
        (unsafe { sys::axq_init(device, &mut ctx) } == 0).then(|| Self { ctx })
    }

    /// quantize_tensor (quantize.rs:36-54): flat row-major f32 of `shape` -> QuantizedTensor, blocks along the buffer.
    pub fn quantize_tensor(&self, data: &[f32], shape: &[usize], ty: QuantType) -> QuantResult<QuantizedTensor> {
        let numel: usize = shape.iter().product();
        if numel != data.len() {
            return Err(QuantError::DataLengthMismatch(format!("Data length mismatch: expected {numel}, got {}", data.len())));
        }
        let mut out = vec![0u8; unsafe { sys::axq_packed_bytes(ty as i32, numel) }];
        check(self.ctx, unsafe {
            sys::axq_quantize(self.ctx, ty as i32, data.as_ptr(), numel, out.as_mut_ptr() as *mut c_void, sys::AXQ_MEM_HOST)
        })?;
        Ok(QuantizedTensor::new(shape.to_vec(), ty, out))
    }

    /// quantize_model (quantize.rs:64-75): names and order kept, the first error ends the call.
    pub fn quantize_model(&self, tensors: &[(&str, &[f32], &[usize])], ty: QuantType) -> QuantResult<Vec<(String, QuantizedTensor)>> {
        tensors.iter().map(|(name, data, shape)| Ok((name.to_string(), self.quantize_tensor(data, shape, ty)?))).collect()
    }

    /// dequantize_tensor (dequantize.rs:34-54): back to f32, truncated to the tensor's element count.
    pub fn dequantize_tensor(&self, q: &QuantizedTensor) -> QuantResult<Vec<f32>> {
        let mut out = vec![0f32; q.numel()];
        check(self.ctx, unsafe {
            sys::axq_dequantize(self.ctx, q.quant_type as i32, q.data.as_ptr() as *const c_void, out.len(), out.as_mut_ptr(),
                                sys::AXQ_MEM_HOST)
        })?;
        Ok(out)
    }

    /// dequantize_block (dequantize.rs:57-65): one block image -> its `block_size` values.
    pub fn dequantize_block(&self, block: &[u8], ty: QuantType) -> QuantResult<Vec<f32>> {
        if block.len() != ty.bytes_per_block() {
            return Err(QuantError::InvalidData(format!("Invalid quantized data: a {ty} block has {} bytes, got {}", ty.bytes_per_block(), block.len())));
        }
        let mut out = vec![0f32; ty.block_size()];
        check(self.ctx, unsafe {
            sys::axq_dequantize(self.ctx, ty as i32, block.as_ptr() as *const c_void, out.len(), out.as_mut_ptr(), sys::AXQ_MEM_HOST)
        })?;
        Ok(out)
    }

    /// A Linear weight `[out, in]` (linear.rs:41-42) made resident on the device, planar.
    pub fn upload(&self, w: &QuantizedTensor) -> QuantResult<DeviceWeight<'_>> {
        if w.shape.len() != 2 {
            return Err(QuantError::ShapeMismatch(format!("Shape mismatch: expected a matrix [out, in], got {:?}", w.shape)));
        }
        let (n, k) = (w.shape[0], w.shape[1]);
        let mut h = std::ptr::null_mut();
        check(self.ctx, unsafe {
            sys::axq_weight_upload(self.ctx, w.quant_type as i32, n as i64, k as i64, w.data.as_ptr() as *const c_void,
                                   w.data.len(), sys::AXQ_MEM_HOST, &mut h)
        })?;
        Ok(DeviceWeight { q: self, h, n, k })
    }

    /// The same from f32: quantised on the device, the packed image never visits the host.
    pub fn upload_f32(&self, w: &[f32], n: usize, k: usize, ty: QuantType) -> QuantResult<DeviceWeight<'_>> {
        if w.len() != n * k {
            return Err(QuantError::DataLengthMismatch(format!("Data length mismatch: expected {}, got {}", n * k, w.len())));
        }
        let mut h = std::ptr::null_mut();
        check(self.ctx, unsafe {
            sys::axq_weight_quantize(self.ctx, ty as i32, n as i64, k as i64, w.as_ptr(), sys::AXQ_MEM_HOST, &mut h)
        })?;
        Ok(DeviceWeight { q: self, h, n, k })
    }
}
impl Drop for HipQuant { fn drop(&mut self) { unsafe { sys::axq_destroy(self.ctx) } } }

pub struct DeviceWeight<'a> { q: &'a HipQuant, h: *mut sys::axq_weight, n: usize, k: usize }
impl DeviceWeight<'_> {
    pub fn out_features(&self) -> usize { self.n }
    pub fn in_features(&self) -> usize { self.k }
}
impl Drop for DeviceWeight<'_> { fn drop(&mut self) { unsafe { sys::axq_weight_free(self.q.ctx, self.h) } } }

/// `y = x · Wᵀ (+ bias)` straight from the packed blocks: replaces `x.matmul(&dequantize_tensor(w)?.t()?)` and the
/// broadcast add of `Linear::forward` (linear.rs:104-140).  `x` is `[rows, in]` row-major; returns `[rows, out]`.
pub fn quantized_matmul(x: &[f32], rows: usize, w: &DeviceWeight<'_>, bias: Option<&[f32]>) -> QuantResult<Vec<f32>> {
    if x.len() != rows * w.k {
        return Err(QuantError::ShapeMismatch(format!("Shape mismatch: expected [{rows}, {}], got {} values", w.k, x.len())));
    }
    if let Some(b) = bias {
        if b.len() != w.n {
            return Err(QuantError::ShapeMismatch(format!("Shape mismatch: expected bias [{}], got [{}]", w.n, b.len())));
        }
    }
    let mut y = vec![0f32; rows * w.n];
    check(w.q.ctx, unsafe {
        sys::axq_gemv_f32(w.q.ctx, w.h, x.as_ptr(), rows as i32, bias.map_or(std::ptr::null(), |b| b.as_ptr()), y.as_mut_ptr(),
                          sys::AXQ_MEM_HOST)
    })?;
    Ok(y)
}

/// `Linear::from_weights` (linear.rs:80-90) over a device weight.
pub struct QuantizedLinear<'a> { pub weight: DeviceWeight<'a>, pub bias: Option<Vec<f32>> }
impl QuantizedLinear<'_> {
    pub fn forward(&self, x: &[f32], rows: usize) -> QuantResult<Vec<f32>> {
        quantized_matmul(x, rows, &self.weight, self.bias.as_deref())
    }
}
