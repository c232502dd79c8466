//! AMD MI355X (gfx950) matrix execution and shape/result validation for llama-rust.
//!
//! Drop-in for `llama-native-cuda` (`native-cuda/src/lib.rs:3-53`, `native-cuda/src/gpu.rs:125-418`):
//! the same `Shape`, `validate`, executor and resident-matrix types with the same methods, error
//! strings and ownership rules, over the C ABI of `include/native_hip.h`.  Beyond that interface:
//! `upload_packed` keeps the GGUF bytes packed in device memory (no host-side expansion to F32) and
//! `gemm_grouped` issues the per-expert products of one MoE projection as one call.
//!
//! This crate is written against the C header and checked against it by
//! `tests/test_rust_binding.py` (every `extern "C"` declaration against the header's, textually); the
//! image it was written in has no Rust toolchain, so it has been neither compiled nor run: nothing
//! beyond that signature check pins its behaviour.

#[cfg(feature = "hip")]
mod ffi {
    use std::ffi::{c_char, c_int, c_void};

    #[repr(C)]
    pub struct LnhExec {
        _private: [u8; 0],
    }
    #[repr(C)]
    pub struct LnhMatrix {
        _private: [u8; 0],
    }
    #[repr(C)]
    pub struct LnhAct {
        _private: [u8; 0],
    }

    // One declaration per entry point of include/native_hip.h that a Rust caller uses, in the
    // header's order.  `usize` is `size_t`, `u32` is `uint32_t`, `c_int` is `int`.
    unsafe extern "C" {
        pub fn lnh_create(device_ordinal: c_int, out: *mut *mut LnhExec) -> c_int;
        pub fn lnh_destroy(exec: *mut LnhExec);
        pub fn lnh_memory_info(exec: *mut LnhExec, free_bytes: *mut usize, total_bytes: *mut usize) -> c_int;
        pub fn lnh_last_error(exec: *const LnhExec) -> *const c_char;
        pub fn lnh_thread_error() -> *const c_char;
        pub fn lnh_upload_f32(exec: *mut LnhExec, rows: usize, cols: usize, weights: *const f32, weights_len: usize, out: *mut *mut LnhMatrix) -> c_int;
        pub fn lnh_upload_packed(exec: *mut LnhExec, ggml_type: u32, rows: usize, cols: usize, bytes: *const u8, nbytes: usize, out: *mut *mut LnhMatrix) -> c_int;
        pub fn lnh_upload_packed_device(exec: *mut LnhExec, ggml_type: u32, rows: usize, cols: usize, device_bytes: *const c_void, nbytes: usize, out: *mut *mut LnhMatrix) -> c_int;
        pub fn lnh_matrix_free(matrix: *mut LnhMatrix);
        pub fn lnh_matrix_info(matrix: *const LnhMatrix, ggml_type: *mut u32, rows: *mut usize, cols: *mut usize, device_bytes: *mut usize) -> c_int;
        pub fn lnh_matrix_prepare(exec: *mut LnhExec, matrix: *const LnhMatrix, max_tokens: usize) -> c_int;
        pub fn lnh_gemv(exec: *mut LnhExec, matrix: *const LnhMatrix, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnh_gemm(exec: *mut LnhExec, matrix: *const LnhMatrix, tokens: usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnh_gemv_once(exec: *mut LnhExec, weights: *const f32, weights_len: usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnh_gemm_grouped(exec: *mut LnhExec, n_groups: usize, mats: *const *const LnhMatrix, tokens: *const usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnh_gemm_shared(exec: *mut LnhExec, n_mats: usize, mats: *const *const LnhMatrix, tokens: usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnh_gemm_device(exec: *mut LnhExec, matrix: *const LnhMatrix, tokens: usize, device_x: *const f32, device_y: *mut f32, stream: *mut c_void) -> c_int;
        pub fn lnh_gemm_grouped_device(exec: *mut LnhExec, n_groups: usize, mats: *const *const LnhMatrix, tokens: *const usize, device_x: *const f32, device_y: *mut f32, stream: *mut c_void) -> c_int;
        pub fn lnh_gemm_device_noalloc(exec: *mut LnhExec, matrix: *const LnhMatrix, tokens: usize, device_x: *const f32, device_y: *mut f32, stream: *mut c_void) -> c_int;
        pub fn lnh_gemm_batch_device(exec: *mut LnhExec, n: usize, mats: *const *const LnhMatrix, tokens: *const usize, device_x: *const *const f32, device_y: *const *mut f32, stream: *mut c_void) -> c_int;
        pub fn lnh_gemv_shared_device(exec: *mut LnhExec, n_mats: usize, mats: *const *const LnhMatrix, device_x: *const f32, device_ys: *const *mut f32, accumulate: c_int, stream: *mut c_void) -> c_int;
        pub fn lnh_gemv_fused_device(exec: *mut LnhExec, n_mats: usize, mats: *const *const LnhMatrix, device_x: *const f32, device_ys: *const *mut f32, accumulate: c_int, prologue: c_int, device_x2: *const f32, eps: f32, stream: *mut c_void) -> c_int;
        pub fn lnh_gemv_swiglu_device(exec: *mut LnhExec, gate: *const LnhMatrix, up: *const LnhMatrix, device_x: *const f32, device_h: *mut f32, prologue: c_int, device_x2: *const f32, eps: f32, stream: *mut c_void) -> c_int;
        pub fn lnh_act_create(exec: *mut LnhExec, ggml_type: u32, cols: usize, max_tokens: usize, out: *mut *mut LnhAct) -> c_int;
        pub fn lnh_act_free(act: *mut LnhAct);
        pub fn lnh_act_split_device(exec: *mut LnhExec, act: *mut LnhAct, tokens: usize, device_x: *const f32, stream: *mut c_void) -> c_int;
        pub fn lnh_gemm_act_device(exec: *mut LnhExec, n_mats: usize, mats: *const *const LnhMatrix, x: *const LnhAct, tokens: usize, device_ys: *const *mut f32, epilogue: c_int, device_residual: *mut f32, device_norm_w: *const f32, eps: f32, device_xn: *mut f32, next: *mut LnhAct, stream: *mut c_void) -> c_int;
        pub fn lnh_gemm_plain_act_device(exec: *mut LnhExec, n_mats: usize, mats: *const *const LnhMatrix, device_x: *const f32, tokens: usize, device_ys: *const *mut f32, epilogue: c_int, device_residual: *mut f32, device_norm_w: *const f32, eps: f32, device_xn: *mut f32, next: *mut LnhAct, stream: *mut c_void) -> c_int;
        pub fn lnh_synchronize(exec: *mut LnhExec) -> c_int;
        pub fn lnh_shape_checked(rows: usize, cols: usize, weights_len: usize, input_len: usize, rows_out: *mut u32, cols_out: *mut u32) -> c_int;
        pub fn lnh_validate(actual: *const f32, actual_len: usize, expected: *const f64, expected_len: usize) -> c_int;
        pub fn lnh_row_bytes(ggml_type: u32, cols: usize) -> usize;
        pub fn lnh_resident_bytes(ggml_type: u32, rows: usize, cols: usize, tokens: usize) -> usize;
        pub fn lnq_gemv(ggml_type: u32, n_cols: usize, w: *const u8, w_len: usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnq_gemm(ggml_type: u32, n_cols: usize, n_tokens: usize, w: *const u8, w_len: usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnq_gemm_grouped(ggml_type: u32, n_cols: usize, n_rows: usize, n_groups: usize, parts: *const *const u8, part_len: usize, tokens: *const usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize) -> c_int;
        pub fn lnq_last_error() -> *const c_char;
    }
}

#[cfg(feature = "hip")]
mod gpu;
#[cfg(feature = "hip")]
pub use gpu::{HipGemv, HipMatrix, resident_bytes};

/// ggml type ids of the eight dtypes the kernels handle (`langtax/src/gguf.rs:245-258`,
/// `include/native_hip.h`).
pub mod ggml_type {
    pub const F32: u32 = 0;
    pub const F16: u32 = 1;
    pub const Q4_0: u32 = 2;
    pub const Q5_0: u32 = 6;
    pub const Q5_1: u32 = 7;
    pub const Q8_0: u32 = 8;
    pub const Q4_K: u32 = 12;
    pub const Q6_K: u32 = 14;
}

/// ggml type id for `GemmKind as u8` (`langtax/src/quant.rs:6646-6676`), `None` for the kinds the
/// packed kernels do not cover (those keep the expand-to-F32 path through `upload`).
pub fn ggml_type_of_gemm_kind(kind: u8) -> Option<u32> {
    match kind {
        0 => Some(ggml_type::F16),   // GemmKind::F16
        2 => Some(ggml_type::F32),   // GemmKind::F32
        6 => Some(ggml_type::Q5_0),  // GemmKind::Q50
        7 => Some(ggml_type::Q5_1),  // GemmKind::Q51
        12 => Some(ggml_type::Q4_0), // GemmKind::Q40
        13 => Some(ggml_type::Q8_0), // GemmKind::Q80
        17 => Some(ggml_type::Q4_K), // GemmKind::Q4K
        19 => Some(ggml_type::Q6_K), // GemmKind::Q6K
        _ => None,
    }
}

/// Checked row-major GEMV dimensions. Dimensions must fit the kernels' u32 ABI.
#[derive(Clone, Copy, Debug, PartialEq, Eq)]
pub struct Shape {
    /// Number of output rows.
    pub rows: u32,
    /// Number of input columns.
    pub cols: u32,
}

impl Shape {
    /// Validate dimensions and exact backing-buffer lengths before any GPU work
    /// (`native-cuda/src/lib.rs:19-34`, same order, same messages; `lnh_shape_checked` is the
    /// C twin used by non-Rust callers).
    pub fn checked(rows: usize, cols: usize, weights: usize, input: usize) -> Result<Self, String> {
        if rows == 0 || cols == 0 {
            return Err("GEMV dimensions must be positive".into());
        }
        let elements = rows.checked_mul(cols).ok_or("GEMV shape overflow")?;
        let _ = u32::try_from(elements).map_err(|_| "GEMV matrix exceeds u32 indexing")?;
        if weights != elements || input != cols {
            return Err("GEMV buffer lengths do not match shape".into());
        }
        Ok(Self {
            rows: u32::try_from(rows).map_err(|_| "GEMV rows exceed u32")?,
            cols: u32::try_from(cols).map_err(|_| "GEMV columns exceed u32")?,
        })
    }
}

/// Compare GPU output against a scalar f64 oracle, rejecting NaN and infinity
/// (`native-cuda/src/lib.rs:37-53`: `|a - e| <= 1e-4 + 1e-4 |e|`).
pub fn validate(actual: &[f32], expected: &[f64]) -> Result<(), String> {
    if actual.len() != expected.len() {
        return Err("GEMV output length mismatch".into());
    }
    for (row, (&actual, &expected)) in actual.iter().zip(expected).enumerate() {
        let tolerance = 1e-4 + 1e-4 * expected.abs();
        if !actual.is_finite() || !expected.is_finite() || (f64::from(actual) - expected).abs() > tolerance {
            return Err(format!("GEMV mismatch at row {row}: expected {expected}, got {actual}"));
        }
    }
    Ok(())
}

#[cfg(test)]
mod tests {
    use super::*;

    // native-cuda/src/lib.rs:59-75: the same cases, host only.
    #[test]
    fn rejects_shapes_that_would_make_device_access_unsafe() {
        assert!(Shape::checked(0, 2, 0, 2).is_err());
        assert!(Shape::checked(2, 3, 5, 3).is_err());
        assert!(Shape::checked(2, 3, 6, 2).is_err());
        assert!(Shape::checked(usize::MAX, 2, 0, 2).is_err());
        assert!(Shape::checked(17, 33, 561, 33).is_ok());
    }

    #[test]
    fn oracle_comparison_catches_nonfinite_and_wrong_results() {
        assert!(validate(&[f32::NAN], &[0.0]).is_err());
        assert!(validate(&[f32::INFINITY], &[f64::INFINITY]).is_err());
        assert!(validate(&[1.0], &[2.0]).is_err());
        assert!(validate(&[], &[0.0]).is_err());
        assert!(validate(&[1.00001, -2.0], &[1.0, -2.0]).is_ok());
    }

    #[test]
    fn gemm_kinds_map_to_the_ggml_ids_of_the_header() {
        let covered: Vec<(u8, u32)> = (0u8..29).filter_map(|k| ggml_type_of_gemm_kind(k).map(|t| (k, t))).collect();
        assert_eq!(covered, [(0, 1), (2, 0), (6, 6), (7, 7), (12, 2), (13, 8), (17, 12), (19, 14)]);
    }
}
