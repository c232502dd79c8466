//! Executor and resident matrices over the C ABI (`include/native_hip.h`), with the method set of
//! `native-cuda/src/gpu.rs:125-418`.
use crate::Shape;
use crate::ffi;
use std::ffi::{CStr, c_char, c_int};

fn text(p: *const c_char) -> String {
    if p.is_null() {
        return String::new();
    }
    // SAFETY: the library returns NUL-terminated strings that stay valid until the next call on
    // the same executor / thread; the text is copied before any such call.
    unsafe { CStr::from_ptr(p) }.to_string_lossy().into_owned()
}

/// Device bytes a packed `rows x cols` matrix holds once it has met products of up to `tokens` tokens
/// (the single-token layout, plus the multi-token layout when such a product reads it): what a residency
/// cache charges before the upload.  `None` for a dtype or shape the packed kernels do not take.
pub fn resident_bytes(ggml_type: u32, rows: usize, cols: usize, tokens: usize) -> Option<usize> {
    // SAFETY: a pure function of its arguments.
    match unsafe { ffi::lnh_resident_bytes(ggml_type, rows, cols, tokens) } {
        0 => None,
        n => Some(n),
    }
}

/// Immutable matrix uploaded once and retained on the GPU (stands in for `CudaMatrix`).  Packed
/// uploads keep the GGUF bytes packed; `shape` is the logical rows x cols either way.
pub struct HipMatrix {
    raw: *mut ffi::LnhMatrix,
    shape: Shape,
}

impl HipMatrix {
    /// Logical dimensions.
    pub fn shape(&self) -> Shape {
        self.shape
    }

    /// Bytes this matrix holds in device memory now (it grows once, when the multi-token layout is made).
    pub fn device_bytes(&self) -> usize {
        let mut bytes = 0usize;
        // SAFETY: `raw` is a live matrix handle; the three unused outputs may be null.
        unsafe { ffi::lnh_matrix_info(self.raw, std::ptr::null_mut(), std::ptr::null_mut(), std::ptr::null_mut(), &mut bytes) };
        bytes
    }
}

impl Drop for HipMatrix {
    fn drop(&mut self) {
        // SAFETY: the handle came from an upload and is freed exactly once; the library allows a
        // matrix to outlive its executor.
        unsafe { ffi::lnh_matrix_free(self.raw) }
    }
}

/// MI355X executor (stands in for `CudaGemv`). Errors propagate without CPU fallback.
pub struct HipGemv {
    raw: *mut ffi::LnhExec,
}

impl Drop for HipGemv {
    fn drop(&mut self) {
        // SAFETY: created by lnh_create, destroyed once.
        unsafe { ffi::lnh_destroy(self.raw) }
    }
}

impl HipGemv {
    fn check(&self, code: c_int) -> Result<(), String> {
        if code == 0 {
            Ok(())
        } else {
            // SAFETY: `raw` is live; the message belongs to the call that just failed.
            Err(text(unsafe { ffi::lnh_last_error(self.raw) }))
        }
    }

    /// Initialize the selected device, its stream and the kernels (`gpu.rs:148-161`).
    pub fn new(device_ordinal: usize) -> Result<Self, String> {
        let ordinal = c_int::try_from(device_ordinal).map_err(|_| "HIP device ordinal out of range".to_string())?;
        let mut raw = std::ptr::null_mut();
        // SAFETY: `raw` is a valid output location.
        if unsafe { ffi::lnh_create(ordinal, &mut raw) } != 0 {
            return Err(text(unsafe { ffi::lnh_thread_error() }));
        }
        Ok(Self { raw })
    }

    /// Return `(free, total)` device-memory bytes (`gpu.rs:164-175`).
    pub fn memory_info(&self) -> Result<(usize, usize), String> {
        let (mut free, mut total) = (0usize, 0usize);
        // SAFETY: both outputs are valid for the duration of the call.
        self.check(unsafe { ffi::lnh_memory_info(self.raw, &mut free, &mut total) })?;
        Ok((free, total))
    }

    /// Upload an immutable F32 matrix (`gpu.rs:264-277`).
    pub fn upload(&mut self, rows: usize, cols: usize, weights: &[f32]) -> Result<HipMatrix, String> {
        let shape = Shape::checked(rows, cols, weights.len(), cols)?;
        let mut raw = std::ptr::null_mut();
        // SAFETY: `weights` is valid for `weights.len()` elements during the synchronous call.
        self.check(unsafe { ffi::lnh_upload_f32(self.raw, rows, cols, weights.as_ptr(), weights.len(), &mut raw) })?;
        Ok(HipMatrix { raw, shape })
    }

    /// Upload the GGUF bytes of a rows x cols tensor and keep them packed on the device.  Replaces
    /// `expand()` + `upload` in `langtax/src/native_gpu.rs:190-194`.
    pub fn upload_packed(&mut self, ggml_type: u32, rows: usize, cols: usize, packed: &[u8]) -> Result<HipMatrix, String> {
        // the shape first: nothing can fail between the upload and the handle's owner
        let shape = Shape {
            rows: u32::try_from(rows).map_err(|_| "GEMV rows exceed u32")?,
            cols: u32::try_from(cols).map_err(|_| "GEMV columns exceed u32")?,
        };
        let mut raw = std::ptr::null_mut();
        // SAFETY: `packed` is valid for `packed.len()` bytes during the synchronous call.
        self.check(unsafe { ffi::lnh_upload_packed(self.raw, ggml_type, rows, cols, packed.as_ptr(), packed.len(), &mut raw) })?;
        Ok(HipMatrix { raw, shape })
    }

    /// Multiply a resident matrix by a host vector and synchronize the output (`gpu.rs:280-335`).
    pub fn gemv_resident(&mut self, matrix: &HipMatrix, input: &[f32], output: &mut [f32]) -> Result<(), String> {
        // SAFETY: slices are valid for their lengths; the library validates before touching `output`.
        self.check(unsafe { ffi::lnh_gemv(self.raw, matrix.raw, input.as_ptr(), input.len(), output.as_mut_ptr(), output.len()) })
    }

    /// Upload a one-shot matrix and run one GEMV (`gpu.rs:339-347`).
    pub fn gemv(&mut self, weights: &[f32], input: &[f32], output: &mut [f32]) -> Result<(), String> {
        let matrix = self.upload(output.len(), input.len(), weights)?;
        self.gemv_resident(&matrix, input, output)
    }

    /// Multiply a resident matrix by `tokens` token-major rows (`gpu.rs:351-417`).
    pub fn gemm_resident(&mut self, matrix: &HipMatrix, tokens: usize, input: &[f32], output: &mut [f32]) -> Result<(), String> {
        // SAFETY: as for gemv_resident.
        self.check(unsafe { ffi::lnh_gemm(self.raw, matrix.raw, tokens, input.as_ptr(), input.len(), output.as_mut_ptr(), output.len()) })
    }

    /// Makes now what products of up to `max_tokens` tokens by `matrix` need beyond the upload (the multi-token
    /// layout of a quantized matrix is otherwise made by the first such product). For callers that run products
    /// where nothing may be allocated, e.g. while a stream is being captured.
    pub fn prepare(&mut self, matrix: &HipMatrix, max_tokens: usize) -> Result<(), String> {
        // SAFETY: both handles are live and belong together (checked by the library).
        self.check(unsafe { ffi::lnh_matrix_prepare(self.raw, matrix.raw, max_tokens) })
    }

    /// The per-expert products of one MoE projection in one call: group `g` multiplies `tokens[g]`
    /// packed rows of `input` by `matrices[g]` (`langtax/src/decode.rs:10035-10058`).
    pub fn gemm_grouped(&mut self, matrices: &[&HipMatrix], tokens: &[usize], input: &[f32], output: &mut [f32]) -> Result<(), String> {
        if matrices.len() != tokens.len() {
            return Err("HIP GEMM buffer lengths do not match shape".into());
        }
        let raws: Vec<*const ffi::LnhMatrix> = matrices.iter().map(|m| m.raw.cast_const()).collect();
        // SAFETY: `raws` and `tokens` hold `raws.len()` entries each; slices are valid for their lengths.
        self.check(unsafe {
            ffi::lnh_gemm_grouped(self.raw, raws.len(), raws.as_ptr(), tokens.as_ptr(), input.as_ptr(), input.len(), output.as_mut_ptr(), output.len())
        })
    }
}
