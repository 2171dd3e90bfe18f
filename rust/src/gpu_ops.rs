// `op::Op<f32>` implementations whose `compute` runs on the GPU through libag_hip.so.
// UNCOMPILED in this repository (no Rust toolchain in the image it was written in); meant to live
// at src/tensor_ops/gpu_ops.rs next to hip_ffi.rs and device.rs, with `mod` lines in
// src/tensor_ops/mod.rs.
//
// Inputs and outputs go through `DeviceIo` (device.rs): with the crate's host-resident storage each
// op stages its arrays through the host; under the cargo feature `device_storage` (device_storage.rs)
// the same bodies pass device arrays from op to op.
//
// Each struct carries the hyper-parameters of the CPU op it stands in for (same field names), keeps
// that op's shape checks and output list, and replaces the numeric core by C-ABI calls.  `grad`
// builds the same gradient nodes as the CPU op -- out of the Gpu* ops -- so `grad()`, the evaluator
// and the optimizers (src/gradient.rs, src/evaluation.rs, src/optimizers/) run unchanged.
// The reference lines each piece follows are cited where it stands.
use super::device::{stream, DeviceBuf, DeviceIo};
use super::hip_ffi as ffi;
use crate::op::{ComputeContext, GradientContext, Op, OpError};
use crate::tensor::Tensor;
use crate::tensor_ops::{nth_tensor, shape, stop_gradient};
use std::os::raw::c_int;

type R = Result<(), OpError>;

fn bad_shape(msg: String) -> OpError {
    OpError::IncompatibleShape(msg)
}

/// A node with plain inputs (none mutable, no back-prop override).
fn node<'g, O: Op<f32> + 'static>(ctx: &GradientContext<'_, 'g, f32>, inputs: &[&Tensor<'g, f32>], op: O) -> Tensor<'g, f32> {
    let mut b = Tensor::builder(ctx.graph());
    for t in inputs {
        b = b.append_input(*t, false);
    }
    b.build(op)
}

// ------------------------------------------------------------------------------------------------
// convolution                                             conv_ops/conv2d.rs, conv2d_transpose.rs
// ------------------------------------------------------------------------------------------------
#[derive(Clone, Copy)]
pub struct ConvHyper {
    pub pad: usize,
    pub stride: usize,
    pub dilation: usize,
}
impl ConvHyper {
    fn ints(&self) -> (c_int, c_int, c_int) {
        (self.pad as c_int, self.stride as c_int, self.dilation as c_int)
    }
}

/// Conv2D (conv2d.rs:6-10, compute :531-554).  Outputs: y [B,K,OH,OW] and the im2col columns,
/// labelled [B,C,kw,kh,OH,OW] as conv2d.rs:482-485 does.
pub struct GpuConv2D(pub ConvHyper);
/// Conv2DWithCols (conv2d.rs:589-597): the GEMM half over existing columns.
pub struct GpuConv2DWithCols(pub ConvHyper);
/// Conv2DFilterGrad (conv2d.rs:736-744).
pub struct GpuConv2DFilterGrad(pub ConvHyper);
/// Conv2DTranspose (conv2d_transpose.rs:249-272).
pub struct GpuConv2DTranspose(pub ConvHyper);
/// Conv2DTransposeFilterGrad (conv2d_transpose.rs:433-451).
pub struct GpuConv2DTransposeFilterGrad(pub ConvHyper);

fn dims4(s: &[usize], what: &str) -> Result<[usize; 4], OpError> {
    if s.len() != 4 {
        return Err(bad_shape(format!("{what} must be 4D (got {s:?})")));
    }
    Ok([s[0], s[1], s[2], s[3]])
}

impl Op<f32> for GpuConv2D {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (x, w) = (ctx.dev_in(0), ctx.dev_in(1));
        // conv2d_extract_params, conv2d.rs:349-404
        let [b, c, h, wd] = dims4(x.shape(), "conv2d: lhs input")?;
        let [k, c2, kh, kw] = dims4(w.shape(), "conv2d: filter")?;
        if c != c2 {
            return Err(bad_shape(format!("conv2d: input channel dim ({c}) must match filter's second dim ({c2})")));
        }
        let (pad, stride, dil) = self.0.ints();
        let (oh, ow) = unsafe {
            (ffi::ag_conv_out_size(h as c_int, kh as c_int, pad, stride, dil) as usize,
             ffi::ag_conv_out_size(wd as c_int, kw as c_int, pad, stride, dil) as usize)
        };
        let dy = DeviceBuf::<f32>::alloc(b * k * oh * ow);
        let dcols = DeviceBuf::<f32>::alloc(b * c * kh * kw * oh * ow);
        ffi::check(unsafe {
            ffi::ag_conv2d_fwd_f32(stream(), x.ptr(), w.ptr(), dy.ptr_mut(), dcols.ptr_mut(), b as c_int, c as c_int,
                                   h as c_int, wd as c_int, k as c_int, kh as c_int, kw as c_int, pad, stride, dil)
        })?;
        ctx.dev_out(dy, &[b, k, oh, ow]);
        ctx.dev_out(dcols, &[b, c, kw, kh, oh, ow]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // conv2d.rs:556-586: gx = Conv2DTranspose(gy, w); gw = Conv2DFilterGrad(cols, gy, w) whose
        // back-prop inputs are (x, gy)
        let (gy, y, x, w) = (ctx.output_grad(), ctx.output(), ctx.input(0), ctx.input(1));
        let gx = node(ctx, &[&gy, &w], GpuConv2DTranspose(self.0));
        let cols = nth_tensor(y, 1);
        let gw = Tensor::builder(ctx.graph())
            .append_input(&cols, false)
            .append_input(&gy, false)
            .append_input(&w, false)
            .append_backprop_input(&x)
            .append_backprop_input(&gy)
            .build(GpuConv2DFilterGrad(self.0));
        ctx.append_input_grad(Some(gx));
        ctx.append_input_grad(Some(gw));
    }
}

impl Op<f32> for GpuConv2DWithCols {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (cols, w) = (ctx.dev_in(0), ctx.dev_in(1));
        let [k, c, kh, kw] = dims4(w.shape(), "conv2d_with_cols: filter")?;
        let cs = cols.shape(); // [B, C, kw, kh, OH, OW] (conv2d.rs:484)
        if cs.len() != 6 {
            return Err(bad_shape(format!("conv2d_with_cols: columns must be 6D (got {cs:?})")));
        }
        let (b, oh, ow) = (cs[0], cs[4], cs[5]);
        let dy = DeviceBuf::<f32>::alloc(b * k * oh * ow);
        ffi::check(unsafe {
            ffi::ag_conv2d_with_cols_f32(stream(), cols.ptr(), w.ptr(), dy.ptr_mut(), b as c_int, (c * kh * kw) as c_int,
                                         (oh * ow) as c_int, k as c_int)
        })?;
        ctx.dev_out(dy, &[b, k, oh, ow]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // conv2d.rs:599-628: as Conv2D::grad, the filter gradient's first back-prop input being the
        // one this node inherited
        let (cols, w, y, gy) = (ctx.input(0), ctx.input(1), ctx.output(), ctx.output_grad());
        let gx = node(ctx, &[&gy, &w], GpuConv2DTranspose(self.0));
        let gw = Tensor::builder(ctx.graph())
            .append_input(&cols, false)
            .append_input(&gy, false)
            .append_input(&w, false)
            .append_backprop_input(&y.get_backprop_input(0))
            .append_backprop_input(&gy)
            .build(GpuConv2DFilterGrad(self.0));
        ctx.append_input_grad(Some(gx));
        ctx.append_input_grad(Some(gw));
    }
}

impl Op<f32> for GpuConv2DFilterGrad {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (cols, gy, w) = (ctx.dev_in(0), ctx.dev_in(1), ctx.dev_in(2));
        let [b, k, oh, ow] = dims4(gy.shape(), "conv2d_filter_grad: gradient")?;
        let [k2, c, kh, kw] = dims4(w.shape(), "conv2d_filter_grad: filter")?;
        if k != k2 {
            return Err(bad_shape(format!("conv2d_filter_grad: {k} gradient channels for {k2} filters")));
        }
        let (ck, p) = (c * kh * kw, oh * ow);
        let dgw = DeviceBuf::<f32>::alloc(k * ck);
        let ws = DeviceBuf::<u8>::alloc(unsafe { ffi::ag_conv2d_filter_grad_f32_workspace(b as c_int, ck as c_int, p as c_int, k as c_int) });
        ffi::check(unsafe {
            ffi::ag_conv2d_filter_grad_f32(stream(), cols.ptr(), gy.ptr(), dgw.ptr_mut(), b as c_int, ck as c_int, p as c_int,
                                           k as c_int, ws.void(), ws.bytes())
        })?;
        ctx.dev_out(dgw, &[k, c, kh, kw]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // conv2d.rs:746-775: two gradients for the two back-prop inputs (x, gy)
        let (cols, gy, ggw, y) = (ctx.input(0), ctx.input(1), ctx.output_grad(), ctx.output());
        let gx = node(ctx, &[&gy, &ggw], GpuConv2DTranspose(self.0));
        let ggy = Tensor::builder(ctx.graph())
            .append_input(&cols, false)
            .append_input(&ggw, false)
            .append_backprop_input(&y.get_backprop_input(0))
            .append_backprop_input(&ggw)
            .build(GpuConv2DWithCols(self.0));
        ctx.append_input_grad(Some(gx));
        ctx.append_input_grad(Some(ggy));
    }
}

impl Op<f32> for GpuConv2DTranspose {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (gy, w) = (ctx.dev_in(0), ctx.dev_in(1));
        // conv2d_transpose_extract_params, conv2d_transpose.rs:29-87
        let [b, ych, yh, yw] = dims4(gy.shape(), "conv2d_transpose: Input")?;
        let [ych2, xch, kh, kw] = dims4(w.shape(), "conv2d_transpose: Filter")?;
        if ych != ych2 {
            return Err(bad_shape(format!("conv2d_transpose: Number of input channels ({ych}) must match second filter dim ({ych2})")));
        }
        let (pad, stride, dil) = self.0.ints();
        // the output extent the reference reconstructs (conv2d_transpose.rs:55-56)
        let (xh, xw) = unsafe {
            (ffi::ag_conv_transpose_out_size(yh as c_int, kh as c_int, pad, stride, dil) as usize,
             ffi::ag_conv_transpose_out_size(yw as c_int, kw as c_int, pad, stride, dil) as usize)
        };
        let dgx = DeviceBuf::<f32>::alloc(b * xch * xh * xw);
        let dgcols = DeviceBuf::<f32>::alloc(b * xch * kh * kw * yh * yw); // the reference's temporary, :148-151
        ffi::check(unsafe {
            ffi::ag_conv2d_transpose_f32(stream(), gy.ptr(), w.ptr(), dgx.ptr_mut(), dgcols.ptr_mut(), b as c_int, ych as c_int,
                                         yh as c_int, yw as c_int, xch as c_int, kh as c_int, kw as c_int, pad, stride, dil,
                                         xh as c_int, xw as c_int)
        })?;
        ctx.dev_out(dgx, &[b, xch, xh, xw]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // conv2d_transpose.rs:274-300: gx = Conv2D(gy, w); gw = Conv2DTransposeFilterGrad(gy, x, stop_gradient(w))
        let (x, w, gy) = (ctx.input(0), ctx.input(1), ctx.output_grad());
        let gx = node(ctx, &[&gy, &w], GpuConv2D(self.0));
        let gw = node(ctx, &[&gy, &x, &stop_gradient(w)], GpuConv2DTransposeFilterGrad(self.0));
        ctx.append_input_grad(Some(gx));
        ctx.append_input_grad(Some(gw));
    }
}

impl Op<f32> for GpuConv2DTransposeFilterGrad {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        // inputs (gy, x, w): conv2d_transpose.rs:435-438
        let (gy, x, w) = (ctx.dev_in(0), ctx.dev_in(1), ctx.dev_in(2));
        let [b, xch, h, wd] = dims4(gy.shape(), "conv2d_transpose_filter_grad: gradient")?;
        let [_, ych, yh, yw] = dims4(x.shape(), "conv2d_transpose_filter_grad: input")?;
        let [_, _, kh, kw] = dims4(w.shape(), "conv2d_transpose_filter_grad: filter")?;
        let (pad, stride, dil) = self.0.ints();
        let dgw = DeviceBuf::<f32>::alloc(ych * xch * kh * kw);
        let dcols = DeviceBuf::<f32>::alloc(b * xch * kh * kw * yh * yw);
        let ws = DeviceBuf::<u8>::alloc(unsafe {
            ffi::ag_conv2d_filter_grad_f32_workspace(b as c_int, (xch * kh * kw) as c_int, (yh * yw) as c_int, ych as c_int)
        });
        ffi::check(unsafe {
            ffi::ag_conv2d_transpose_filter_grad_f32(stream(), x.ptr(), gy.ptr(), dgw.ptr_mut(), dcols.ptr_mut(), b as c_int,
                                                     ych as c_int, yh as c_int, yw as c_int, xch as c_int, h as c_int, wd as c_int,
                                                     kh as c_int, kw as c_int, pad, stride, dil, ws.void(), ws.bytes())
        })?;
        ctx.dev_out(dgw, &[ych, xch, kh, kw]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // conv2d_transpose.rs:453-479
        let (gy, gw, x) = (ctx.input(0), ctx.output_grad(), ctx.input(1));
        let ggy = node(ctx, &[&x, &gw], GpuConv2DTranspose(self.0));
        let ggx = node(ctx, &[&gy, &gw], GpuConv2D(self.0));
        ctx.append_input_grad(Some(ggy));
        ctx.append_input_grad(Some(ggx));
        ctx.append_input_grad(None);
    }
}

// ------------------------------------------------------------------------------------------------
// max pooling                                                             conv_ops/max_pool2d.rs
// ------------------------------------------------------------------------------------------------
#[derive(Clone, Copy)]
pub struct PoolHyper {
    pub pad: usize,
    pub stride: usize,
    pub size: usize,
}
/// MaxPool2D (max_pool2d.rs:3-7, compute :166-227): outputs y and the f32-encoded argmax.
pub struct GpuMaxPool2D(pub PoolHyper);
/// MaxPool2DGrad (max_pool2d.rs:245-279).
pub struct GpuMaxPool2DGrad(pub PoolHyper);
/// MaxPool2DGradGrad (max_pool2d.rs:297-331).
pub struct GpuMaxPool2DGradGrad(pub PoolHyper);

impl Op<f32> for GpuMaxPool2D {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let x = ctx.dev_in(0);
        let [b, c, h, w] = dims4(x.shape(), "max_pool2d: input")?;
        let (size, pad, stride) = (self.0.size as c_int, self.0.pad as c_int, self.0.stride as c_int);
        let (oh, ow) = unsafe {
            (ffi::ag_pool_out_size(h as c_int, size, pad, stride) as usize, ffi::ag_pool_out_size(w as c_int, size, pad, stride) as usize)
        };
        let (dy, dam) = (DeviceBuf::<f32>::alloc(b * c * oh * ow), DeviceBuf::<f32>::alloc(b * c * oh * ow));
        // taps = NULL: this wrapper keeps to the reference's two outputs (exact while x has <= 2^24 elements)
        ffi::check(unsafe {
            ffi::ag_maxpool2d_fwd_f32(stream(), x.ptr(), dy.ptr_mut(), dam.ptr_mut(), std::ptr::null_mut(), b as c_int, c as c_int,
                                      h as c_int, w as c_int, size, pad, stride)
        })?;
        ctx.dev_out(dy, &[b, c, oh, ow]);
        ctx.dev_out(dam, &[b, c, oh, ow]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // max_pool2d.rs:229-242
        let (gy, y) = (ctx.output_grad(), ctx.output());
        let indices = nth_tensor(y, 1);
        ctx.append_input_grad(Some(node(ctx, &[&gy, &indices], GpuMaxPool2DGrad(self.0))));
    }
}

impl Op<f32> for GpuMaxPool2DGrad {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (gy, argmax) = (ctx.dev_in(0), ctx.dev_in(1));
        let [b, c, yh, yw] = dims4(gy.shape(), "max_pool2d_grad: gradient")?;
        let (size, pad, stride) = (self.0.size as c_int, self.0.pad as c_int, self.0.stride as c_int);
        // the input extent the reference reconstructs (max_pool2d.rs:263-264)
        let (xh, xw) = unsafe {
            (ffi::ag_pool_grad_in_size(yh as c_int, size, pad, stride) as usize, ffi::ag_pool_grad_in_size(yw as c_int, size, pad, stride) as usize)
        };
        let dgx = DeviceBuf::<f32>::alloc(b * c * xh * xw);
        ffi::check(unsafe {
            ffi::ag_maxpool2d_bwd_f32(stream(), gy.ptr(), argmax.ptr(), std::ptr::null(), dgx.ptr_mut(), b as c_int, c as c_int,
                                      xh as c_int, xw as c_int, size, pad, stride)
        })?;
        ctx.dev_out(dgx, &[b, c, xh, xw]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // max_pool2d.rs:281-294
        let (ggx, argmax) = (ctx.output_grad(), ctx.input(1));
        ctx.append_input_grad(Some(node(ctx, &[&ggx, &argmax], GpuMaxPool2DGradGrad(self.0))));
        ctx.append_input_grad(None);
    }
}

impl Op<f32> for GpuMaxPool2DGradGrad {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (ggx, argmax) = (ctx.dev_in(0), ctx.dev_in(1));
        let [b, c, h, w] = dims4(ggx.shape(), "max_pool2d_grad_grad: input")?;
        let out: Vec<usize> = argmax.shape().to_vec();
        let (size, pad, stride) = (self.0.size as c_int, self.0.pad as c_int, self.0.stride as c_int);
        let dggy = DeviceBuf::<f32>::alloc(out.iter().product());
        ffi::check(unsafe {
            ffi::ag_maxpool2d_gradgrad_f32(stream(), ggx.ptr(), argmax.ptr(), std::ptr::null(), dggy.ptr_mut(), b as c_int, c as c_int,
                                           h as c_int, w as c_int, size, pad, stride)
        })?;
        ctx.dev_out(dggy, &out);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // max_pool2d.rs:333-336: not differentiable further
        ctx.append_input_grad(None);
        ctx.append_input_grad(None);
    }
}

// ------------------------------------------------------------------------------------------------
// matrix products                                                                     dot_ops.rs
// ------------------------------------------------------------------------------------------------
/// MatMul (dot_ops.rs:554-557, compute :564-606).
pub struct GpuMatMul {
    pub transpose_a: bool,
    pub transpose_b: bool,
}
/// BatchMatMul (dot_ops.rs:559-562, compute :631-695).
pub struct GpuBatchMatMul {
    pub transpose_a: bool,
    pub transpose_b: bool,
}

impl Op<f32> for GpuMatMul {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (a, b) = (ctx.dev_in(0), ctx.dev_in(1));
        if a.ndim() != 2 {
            return Err(bad_shape("lhs input for MatMul must be 2D".into())); // dot_ops.rs:566-569
        }
        if b.ndim() != 2 {
            return Err(bad_shape("rhs input for MatMul must be 2D".into())); // dot_ops.rs:570-573
        }
        let (ar, ac, br, bc) = (a.shape()[0], a.shape()[1], b.shape()[0], b.shape()[1]);
        let (m, k) = if self.transpose_a { (ac, ar) } else { (ar, ac) };
        let (k2, n) = if self.transpose_b { (bc, br) } else { (br, bc) };
        if k != k2 {
            return Err(bad_shape(format!("ndarray: inputs {m} × {k} and {k2} × {n} are not compatible for matrix multiplication")));
        }
        let dc = DeviceBuf::<f32>::alloc(m * n);
        let ws = DeviceBuf::<u8>::alloc(unsafe { ffi::ag_matmul_f32_workspace(m as c_int, n as c_int, k as c_int) });
        ffi::check(unsafe {
            ffi::ag_matmul_f32(stream(), self.transpose_a as c_int, self.transpose_b as c_int, m as c_int, n as c_int, k as c_int,
                               a.ptr(), ac.max(1) as c_int, b.ptr(), bc.max(1) as c_int, dc.ptr_mut(), n.max(1) as c_int,
                               ws.void(), ws.bytes())
        })?;
        ctx.dev_out(dc, &[m, n]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // dot_ops.rs:608-628: ga = gy . b^T, gb = a^T . gy (this op's own flags are not consulted)
        let gy = ctx.output_grad();
        let ga = node(ctx, &[&gy, &ctx.input(1)], GpuMatMul { transpose_a: false, transpose_b: true });
        let gb = node(ctx, &[&ctx.input(0), &gy], GpuMatMul { transpose_a: true, transpose_b: false });
        ctx.append_input_grad(Some(ga));
        ctx.append_input_grad(Some(gb));
    }
}

impl Op<f32> for GpuBatchMatMul {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let (a, b) = (ctx.dev_in(0), ctx.dev_in(1));
        let (ra, rb) = (a.ndim(), b.ndim());
        if ra < 2 {
            return Err(bad_shape(format!("BatchMatMul: Left-hand-side input's ndim must be >= 2, actual: {ra}")));
        }
        if rb < 2 {
            return Err(bad_shape(format!("BatchMatMul: Right-hand-side input's ndim must be >= 2, actual: {rb}")));
        }
        let (mut sa, mut sb) = (a.shape().to_vec(), b.shape().to_vec());
        if self.transpose_a {
            sa.swap(ra - 2, ra - 1);
        }
        if self.transpose_b {
            sb.swap(rb - 2, rb - 1);
        }
        // dot_ops.rs:661-672: equal rank, equal leading extents, matching inner extent
        if ra != rb || sa[..ra - 2] != sb[..rb - 2] || sa[ra - 1] != sb[rb - 2] {
            return Err(bad_shape(format!("Input shapes mismatch: {sa:?} vs {sb:?}")));
        }
        let (m, k, n) = (sa[ra - 2], sa[ra - 1], sb[rb - 1]);
        let batch: usize = sa[..ra - 2].iter().product();
        let (lda, ldb) = (a.shape()[ra - 1].max(1), b.shape()[rb - 1].max(1));
        let dc = DeviceBuf::<f32>::alloc(batch * m * n);
        ffi::check(unsafe {
            ffi::ag_gemm_f32(stream(), self.transpose_a as c_int, self.transpose_b as c_int, m as c_int, n as c_int, k as c_int, 1.0,
                             a.ptr(), lda as c_int, (a.shape()[ra - 2] * a.shape()[ra - 1]) as i64, b.ptr(), ldb as c_int,
                             (b.shape()[rb - 2] * b.shape()[rb - 1]) as i64, 0.0, dc.ptr_mut(), n.max(1) as c_int, (m * n) as i64,
                             batch as c_int)
        })?;
        let mut out = sa[..ra - 2].to_vec();
        out.extend([m, n]);
        ctx.dev_out(dc, &out);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // dot_ops.rs:697-717
        let gy = ctx.output_grad();
        let ga = node(ctx, &[&gy, &ctx.input(1)], GpuBatchMatMul { transpose_a: false, transpose_b: true });
        let gb = node(ctx, &[&ctx.input(0), &gy], GpuBatchMatMul { transpose_a: true, transpose_b: false });
        ctx.append_input_grad(Some(ga));
        ctx.append_input_grad(Some(gb));
    }
}

// ------------------------------------------------------------------------------------------------
// reductions                                                                   reduction_ops.rs
// ------------------------------------------------------------------------------------------------
/// ReduceSumToScalar (reduction_ops.rs:123-137).
pub struct GpuReduceSumToScalar;
/// ReduceSum (reduction_ops.rs:29-32, compute :161-170).
pub struct GpuReduceSum {
    pub keep_dims: bool,
    pub sparse_axes: bool,
}
/// ReduceMean (reduction_ops.rs:34-37, compute :187-215).
pub struct GpuReduceMean {
    pub keep_dims: bool,
    pub sparse_axes: bool,
}

/// Axes tensor -> ascending, unique, non-negative axes (reduction_ops.rs:111-121).
fn axes_of(x_rank: usize, axes: &crate::ndarray_ext::NdArrayView<f32>, sparse: bool) -> Vec<c_int> {
    let mut v: Vec<usize> = if sparse {
        crate::ndarray_ext::sparse_to_dense(axes)
    } else {
        crate::ndarray_ext::normalize_negative_axes(axes, x_rank)
    };
    v.sort_unstable();
    v.dedup();
    v.into_iter().map(|a| a as c_int).collect()
}

fn reduce(ctx: &mut ComputeContext<f32>, keep_dims: bool, sparse: bool, mean: bool) -> R {
    let x = ctx.dev_in(0);
    let axes = axes_of(x.ndim(), &ctx.input(1), sparse); // a handful of indices: read on the host
    if x.ndim() == 0 || axes.is_empty() {
        ctx.dev_out_shared(x); // reduction_ops.rs:63-70, 192-195
        return Ok(());
    }
    let dims: Vec<c_int> = x.shape().iter().map(|&d| d as c_int).collect();
    let out_shape: Vec<usize> = x.shape().iter().enumerate()
        .filter_map(|(i, &d)| if axes.contains(&(i as c_int)) { if keep_dims { Some(1) } else { None } } else { Some(d) })
        .collect();
    let dout = DeviceBuf::<f32>::alloc(out_shape.iter().product());
    let ws = DeviceBuf::<u8>::alloc(unsafe {
        ffi::ag_reduce_sum_f32_workspace(dims.as_ptr(), dims.len() as c_int, axes.as_ptr(), axes.len() as c_int)
    });
    ffi::check(unsafe {
        ffi::ag_reduce_sum_f32(stream(), x.ptr(), dout.ptr_mut(), dims.as_ptr(), dims.len() as c_int, axes.as_ptr(),
                               axes.len() as c_int, mean as c_int, ws.void(), ws.bytes())
    })?;
    ctx.dev_out(dout, &out_shape);
    Ok(())
}

impl Op<f32> for GpuReduceSumToScalar {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let x = ctx.dev_in(0);
        let dout = DeviceBuf::<f32>::alloc(1);
        let ws = DeviceBuf::<u8>::alloc(unsafe { ffi::ag_sum_all_f32_workspace(x.len()) });
        ffi::check(unsafe { ffi::ag_sum_all_f32(stream(), x.ptr(), x.len(), dout.ptr_mut(), ws.void(), ws.bytes()) })?;
        ctx.dev_out(dout, &[]);
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // reduction_ops.rs:130-136: the CPU ReduceSumToScalarGrad (a fill) serves as it is
        let gx = Tensor::builder(ctx.graph())
            .append_input(&ctx.output_grad(), false)
            .append_input(&shape(ctx.input(0)), false)
            .build(crate::tensor_ops::reduction_ops::ReduceSumToScalarGrad);
        ctx.append_input_grad(Some(gx));
    }
}

impl Op<f32> for GpuReduceSum {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        reduce(ctx, self.keep_dims, self.sparse_axes, false)
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // reduction_ops.rs:172-184: ReduceGradCommon(gy, shape(x), axes) with should_make_broadcast_dims = !keep_dims
        let gx = Tensor::builder(ctx.graph())
            .append_input(&ctx.output_grad(), false)
            .append_input(&shape(&ctx.input(0)), false)
            .append_input(&ctx.input(1), false)
            .build(crate::tensor_ops::reduction_ops::ReduceGradCommon {
                should_make_broadcast_dims: !self.keep_dims,
                sparse_axes: self.sparse_axes,
            });
        ctx.append_input_grad(Some(gx));
        ctx.append_input_grad(None);
    }
}

impl Op<f32> for GpuReduceMean {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        reduce(ctx, self.keep_dims, self.sparse_axes, true)
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // reduction_ops.rs:217-238: broadcast gy, then divide by the product of the reduced extents
        let (x, axes) = (ctx.input(0), ctx.input(1));
        let broadcast = Tensor::builder(ctx.graph())
            .append_input(&ctx.output_grad(), false)
            .append_input(&shape(&x), false)
            .append_input(&axes, false)
            .build(crate::tensor_ops::reduction_ops::ReduceGradCommon {
                should_make_broadcast_dims: !self.keep_dims,
                sparse_axes: self.sparse_axes,
            });
        let reduced = crate::tensor_ops::gather_common(shape(&x), &axes, 0);
        let len = crate::tensor_ops::reduce_prod(reduced, &[0], false);
        ctx.append_input_grad(Some(broadcast / len));
        ctx.append_input_grad(None);
    }
}

// ------------------------------------------------------------------------------------------------
// Adam                                                         gradient_descent_ops/adam.rs
// ------------------------------------------------------------------------------------------------
/// AdamOp (adam.rs:3-8).  Inputs [param (mut), grad, m (mut), v (mut), t (mut)] in the order
/// optimizers/adam.rs:138-143 builds them; returns the empty 0-d array of adam.rs:56.
pub struct GpuAdamOp {
    pub alpha: f32,
    pub eps: f32,
    pub b1: f32,
    pub b2: f32,
}

impl Op<f32> for GpuAdamOp {
    fn compute(&self, ctx: &mut ComputeContext<f32>) -> R {
        let g = ctx.dev_in(1);
        let n = g.len();
        // one fused pass in place on param, m, v; t is read by the update and incremented after it
        let (p, m, v, t) = (ctx.dev_in_mut(0), ctx.dev_in_mut(2), ctx.dev_in_mut(3), ctx.dev_in_mut(4));
        if p.len() != n || m.len() != n || v.len() != n || t.len() != 1 {
            return Err(bad_shape(format!("adam: param {:?}, grad {:?}, m {:?}, v {:?}, t {:?}", p.shape(), g.shape(), m.shape(), v.shape(), t.shape())));
        }
        let status = unsafe {
            ffi::ag_adam_update_f32(stream(), p.ptr_mut(), g.ptr(), m.ptr_mut(), v.ptr_mut(), t.ptr_mut(), n, self.alpha, self.eps,
                                    self.b1, self.b2)
        };
        // hand every array back before reporting: with host storage this is where they are written back
        ctx.dev_commit(0, p);
        ctx.dev_commit(2, m);
        ctx.dev_commit(3, v);
        ctx.dev_commit(4, t);
        ffi::check(status)?;
        ctx.append_empty_output();
        Ok(())
    }
    fn grad(&self, ctx: &mut GradientContext<f32>) {
        // adam.rs:60-66: an update has no gradient, for any of its five inputs
        for _ in 0..5 {
            ctx.append_input_grad(None);
        }
    }
}
