// Foreign declarations of libag_hip.so for the crate (to sit next to src/tensor_ops/blas_ffi.rs,
// the reference's only other FFI: cblas_sgemm / cblas_dgemm through cblas-sys, blas_ffi.rs:1-15).
// GENERATED from include/ag_hip.h by rust/gen_hip_ffi.py -- one `pub fn` per C function, same order.
// UNCOMPILED in this repository: the image it was written in has no Rust toolchain.
#![allow(clippy::too_many_arguments, non_snake_case)]
use std::os::raw::{c_char, c_int, c_longlong, c_void};

pub type AgStatus = c_int; // ag_status_t: 0 ok, 1..5 = op::OpError variants in order, 100 + n = hipError_t n
pub type AgStream = *mut c_void; // hipStream_t

#[link(name = "ag_hip")]
extern "C" {
    pub fn ag_last_error() -> *const c_char;
    pub fn ag_version() -> *const c_char;
    pub fn ag_conv_out_size(x: c_int, k: c_int, pad: c_int, stride: c_int, dilation: c_int) -> c_int;
    pub fn ag_conv_transpose_out_size(y: c_int, k: c_int, pad: c_int, stride: c_int, dilation: c_int) -> c_int;
    pub fn ag_pool_out_size(x: c_int, size: c_int, pad: c_int, stride: c_int) -> c_int;
    pub fn ag_pool_grad_in_size(y: c_int, size: c_int, pad: c_int, stride: c_int) -> c_int;
    pub fn ag_im2col_f32(stream: AgStream, x: *const f32, cols: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, kh: c_int, kw: c_int, ph: c_int, pw: c_int, sh: c_int, sw: c_int, dh: c_int, dw: c_int) -> AgStatus;
    pub fn ag_col2im_f32(stream: AgStream, cols: *const f32, gx: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, kh: c_int, kw: c_int, ph: c_int, pw: c_int, sh: c_int, sw: c_int, dh: c_int, dw: c_int, OH: c_int, OW: c_int) -> AgStatus;
    pub fn ag_gemm_f32(stream: AgStream, transA: c_int, transB: c_int, M: c_int, N: c_int, K: c_int, alpha: f32, A: *const f32, lda: c_int, strideA: c_longlong, B: *const f32, ldb: c_int, strideB: c_longlong, beta: f32, C: *mut f32, ldc: c_int, strideC: c_longlong, batch: c_int) -> AgStatus;
    pub fn ag_gemm_batchsum_f32_workspace(M: c_int, N: c_int, K: c_int, batch: c_int) -> usize;
    pub fn ag_gemm_batchsum_f32(stream: AgStream, transA: c_int, transB: c_int, M: c_int, N: c_int, K: c_int, alpha: f32, A: *const f32, lda: c_int, strideA: c_longlong, B: *const f32, ldb: c_int, strideB: c_longlong, beta: f32, C: *mut f32, ldc: c_int, batch: c_int, ws: *mut c_void, ws_bytes: usize) -> AgStatus;
    pub fn ag_matmul_f32_workspace(M: c_int, N: c_int, K: c_int) -> usize;
    pub fn ag_matmul_f32(stream: AgStream, transA: c_int, transB: c_int, M: c_int, N: c_int, K: c_int, A: *const f32, lda: c_int, B: *const f32, ldb: c_int, C: *mut f32, ldc: c_int, ws: *mut c_void, ws_bytes: usize) -> AgStatus;
    pub fn ag_conv2d_fwd_f32(stream: AgStream, x: *const f32, w: *const f32, y: *mut f32, cols: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int) -> AgStatus;
    pub fn ag_conv2d_with_cols_f32(stream: AgStream, cols: *const f32, w: *const f32, y: *mut f32, B: c_int, CK: c_int, P: c_int, K: c_int) -> AgStatus;
    pub fn ag_conv2d_filter_grad_f32_workspace(B: c_int, CK: c_int, P: c_int, K: c_int) -> usize;
    pub fn ag_conv2d_filter_grad_f32(stream: AgStream, cols: *const f32, gy: *const f32, gw: *mut f32, B: c_int, CK: c_int, P: c_int, K: c_int, ws: *mut c_void, ws_bytes: usize) -> AgStatus;
    pub fn ag_conv2d_transpose_f32(stream: AgStream, gy: *const f32, w: *const f32, gx: *mut f32, gcols: *mut f32, B: c_int, ych: c_int, yh: c_int, yw: c_int, xch: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int, xh: c_int, xw: c_int) -> AgStatus;
    pub fn ag_conv_input_grad_scratch_floats(B: c_int, ych: c_int, yh: c_int, yw: c_int, xch: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int, xh: c_int, xw: c_int) -> usize;
    pub fn ag_conv_input_grad_prepare_f32(stream: AgStream, gy: *const f32, w: *const f32, scratch: *mut f32, B: c_int, ych: c_int, yh: c_int, yw: c_int, xch: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int, xh: c_int, xw: c_int) -> AgStatus;
    pub fn ag_conv_input_grad_gemm_f32(stream: AgStream, scratch: *mut f32, gx: *mut f32, B: c_int, ych: c_int, yh: c_int, yw: c_int, xch: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int, xh: c_int, xw: c_int) -> AgStatus;
    pub fn ag_conv2d_nocols_scratch_floats(B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int) -> usize;
    pub fn ag_conv2d_fwd_nocols_f32(stream: AgStream, x: *const f32, w: *const f32, y: *mut f32, xpad: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int) -> AgStatus;
    pub fn ag_conv2d_nocols_prepare_f32(stream: AgStream, x: *const f32, w: *const f32, xpad: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int) -> AgStatus;
    pub fn ag_conv2d_nocols_gemm_f32(stream: AgStream, xpad: *mut f32, y: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int) -> AgStatus;
    pub fn ag_conv2d_nocols_with_filter_f32(stream: AgStream, xpad: *const f32, w: *const f32, wf: *mut f32, y: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int) -> AgStatus;
    pub fn ag_conv2d_filter_grad_nocols_f32_workspace(B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int) -> usize;
    pub fn ag_conv2d_filter_grad_nocols_f32(stream: AgStream, xpad: *const f32, gypad: *const f32, gw: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, K: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int, ws: *mut c_void, ws_bytes: usize) -> AgStatus;
    pub fn ag_conv2d_transpose_filter_grad_f32(stream: AgStream, x: *const f32, gy: *const f32, gw: *mut f32, gycols: *mut f32, B: c_int, ych: c_int, yh: c_int, yw: c_int, xch: c_int, H: c_int, W: c_int, kh: c_int, kw: c_int, pad: c_int, stride: c_int, dilation: c_int, ws: *mut c_void, ws_bytes: usize) -> AgStatus;
    pub fn ag_maxpool2d_fwd_f32(stream: AgStream, x: *const f32, y: *mut f32, argmax: *mut f32, taps: *mut u8, B: c_int, C: c_int, H: c_int, W: c_int, size: c_int, pad: c_int, stride: c_int) -> AgStatus;
    pub fn ag_relu_maxpool2d_2x2_f32(stream: AgStream, a: *const f32, b: *const f32, bshape: *const c_int, r: *mut f32, y: *mut f32, argmax: *mut f32, taps: *mut u8, B: c_int, C: c_int, H: c_int, W: c_int) -> AgStatus;
    pub fn ag_maxpool2d_bwd_f32(stream: AgStream, gy: *const f32, argmax: *const f32, taps: *const u8, gx: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, size: c_int, pad: c_int, stride: c_int) -> AgStatus;
    pub fn ag_maxpool2d_bwd_relu_f32(stream: AgStream, gy: *const f32, argmax: *const f32, taps: *const u8, relu_x: *const f32, gx: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, size: c_int, pad: c_int, stride: c_int) -> AgStatus;
    pub fn ag_maxpool2d_gradgrad_f32(stream: AgStream, ggx: *const f32, argmax: *const f32, taps: *const u8, ggy: *mut f32, B: c_int, C: c_int, H: c_int, W: c_int, size: c_int, pad: c_int, stride: c_int) -> AgStatus;
    pub fn ag_sum_all_f32_workspace(n: usize) -> usize;
    pub fn ag_sum_all_f32(stream: AgStream, x: *const f32, n: usize, out: *mut f32, ws: *mut c_void, ws_bytes: usize) -> AgStatus;
    pub fn ag_reduce_sum_f32_workspace(shape: *const c_int, rank: c_int, axes: *const c_int, n_axes: c_int) -> usize;
    pub fn ag_reduce_sum_f32(stream: AgStream, x: *const f32, out: *mut f32, shape: *const c_int, rank: c_int, axes: *const c_int, n_axes: c_int, mean: c_int, ws: *mut c_void, ws_bytes: usize) -> AgStatus;
    pub fn ag_broadcast_grad_f32(stream: AgStream, gy: *const f32, gx: *mut f32, shape: *const c_int, rank: c_int, axes: *const c_int, n_axes: c_int) -> AgStatus;
    pub fn ag_adam_update_f32(stream: AgStream, param: *mut f32, grad: *const f32, m: *mut f32, v: *mut f32, t: *mut f32, n: usize, alpha: f32, eps: f32, b1: f32, b2: f32) -> AgStatus;
    pub fn ag_adam_update_multi_max() -> c_int;
    pub fn ag_adam_update_multi_f32(stream: AgStream, count: c_int, params: *const *mut f32, grads: *const *const f32, ms: *const *mut f32, vs: *const *mut f32, ts: *const *mut f32, ns: *const usize, alpha: f32, eps: f32, b1: f32, b2: f32) -> AgStatus;
    pub fn ag_relu_f32(stream: AgStream, x: *const f32, y: *mut f32, n: usize) -> AgStatus;
    pub fn ag_relu_grad_f32(stream: AgStream, x: *const f32, gy: *const f32, gx: *mut f32, n: usize) -> AgStatus;
    pub fn ag_add_bias_f32(stream: AgStream, x: *const f32, bias: *const f32, y: *mut f32, rows: usize, cols: usize) -> AgStatus;
    pub fn ag_add_broadcast_f32(stream: AgStream, x: *const f32, b: *const f32, y: *mut f32, shape: *const c_int, bshape: *const c_int, rank: c_int) -> AgStatus;
    pub fn ag_add_broadcast_relu_f32(stream: AgStream, x: *const f32, b: *const f32, y: *mut f32, shape: *const c_int, bshape: *const c_int, rank: c_int) -> AgStatus;
    pub fn ag_bias_grad_f32(stream: AgStream, gy: *const f32, out: *mut f32, rows: usize, cols: usize) -> AgStatus;
    pub fn ag_add_n_f32(stream: AgStream, xs: *const *const f32, count: c_int, out: *mut f32, n: usize) -> AgStatus;
    pub fn ag_mul_f32(stream: AgStream, a: *const f32, b: *const f32, out: *mut f32, n: usize) -> AgStatus;
    pub fn ag_scale_f32(stream: AgStream, a: *const f32, s: f32, out: *mut f32, n: usize) -> AgStatus;
    pub fn ag_div_scalar_f32(stream: AgStream, a: *const f32, s: f32, out: *mut f32, n: usize) -> AgStatus;
    pub fn ag_fill_f32(stream: AgStream, out: *mut f32, value: f32, n: usize) -> AgStatus;
    pub fn ag_sparse_softmax_xent_f32(stream: AgStream, logits: *const f32, labels: *const f32, loss: *mut f32, log_softmax: *mut f32, rows: usize, classes: usize) -> AgStatus;
    pub fn ag_sparse_softmax_xent_grad_f32(stream: AgStream, log_softmax: *const f32, labels: *const f32, gy: *const f32, gx: *mut f32, rows: usize, classes: usize) -> AgStatus;
    pub fn ag_sparse_softmax_xent_grad_logits_f32(stream: AgStream, logits: *const f32, labels: *const f32, gy: *const f32, gy_const: f32, gx: *mut f32, rows: usize, classes: usize) -> AgStatus;
    pub fn ag_matmul_f32_static_scratch_bytes() -> usize;
    pub fn ag_matmul_f32_noalloc(stream: AgStream, transA: c_int, transB: c_int, M: c_int, N: c_int, K: c_int, A: *const f32, lda: c_int, B: *const f32, ldb: c_int, C: *mut f32, ldc: c_int) -> AgStatus;
}

/// ag_status_t -> the crate's OpError (src/op.rs:66-73); 1..5 are its variants in declaration order.
pub fn to_op_error(st: AgStatus) -> crate::op::OpError {
    let msg = unsafe { std::ffi::CStr::from_ptr(ag_last_error()) }.to_string_lossy().into_owned();
    match st {
        1 => crate::op::OpError::NdArrayError(msg, ndarray::ShapeError::from_kind(ndarray::ErrorKind::IncompatibleLayout)),
        2 => crate::op::OpError::IncompatibleShape(msg),
        3 => crate::op::OpError::TypeUnsupported(msg),
        5 => crate::op::OpError::OutOfBounds(msg),
        _ => crate::op::OpError::InvalidDims(msg), // 4, and 100 + hipError_t
    }
}

/// `Ok(())` for AG_OK, the mapped OpError otherwise.
pub fn check(st: AgStatus) -> Result<(), crate::op::OpError> {
    if st == 0 { Ok(()) } else { Err(to_op_error(st)) }
}
