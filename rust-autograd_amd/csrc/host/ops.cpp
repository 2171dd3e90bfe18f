// Operators of the conv / matmul / pool / reduce / Adam path as `Op` implementations whose
// `compute` calls the C ABI of libag_hip.so and whose `grad` builds the same gradient sub-graphs
// as the reference.  Citations are to the reference's src/tensor_ops/.
#include <algorithm>
#include <sstream>

#include "ag_hip.h"
#include "ag_host.hpp"

namespace ag {
namespace host {

namespace {

std::string shape_str(const Shape &s)
{
    std::ostringstream os;
    os << "[";
    for (size_t i = 0; i < s.size(); ++i) os << (i ? ", " : "") << s[i];
    os << "]";
    return os.str();
}

// Status of a C-ABI call -> OpError (1..5 are the OpError variants, src/op.rs:66-73).
OpError from_status(ag_status_t st)
{
    if (st == AG_OK) return OpError::none();
    const ErrorKind k = (st >= 1 && st <= 5) ? static_cast<ErrorKind>(st) : ErrorKind::Hip;
    return OpError::make(k, ag_last_error());
}

NdArray workspace(size_t bytes) { return NdArray::empty({(int64_t)((bytes + 3) / 4 + 4)}); }

Tensor build(Graph *g, std::initializer_list<Tensor> inputs, std::unique_ptr<Op> op)
{
    TensorBuilder b = g->builder();
    for (const Tensor &t : inputs) b.append_input(t, false);
    return b.build(std::move(op));
}

// ------------------------------------------------------------------------------------------
// Identity (selector for multi-output ops)                     activation_ops.rs:169-181
// ------------------------------------------------------------------------------------------
struct Identity : Op {
    const char *name() const override { return "Identity"; }
    OpError compute(ComputeContext &ctx) const override
    {
        ctx.append_output_view(ctx.input(0));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override { ctx.append_input_grad(ctx.output_grad()); }
};

struct StopGradient : Op {  // gradient_ops.rs
    const char *name() const override { return "StopGradient"; }
    OpError compute(ComputeContext &ctx) const override
    {
        ctx.append_output_view(ctx.input(0));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override { ctx.append_input_grad(std::nullopt); }
};

// The extents of its input as an array without elements: what an op is handed when all it needs of a tensor is its
// shape (the convolution's input, from which its gradients take their output extents).  No counterpart in the reference,
// whose gradient ops reconstruct those extents (conv2d_transpose.rs:55-56, max_pool2d.rs:263-264).  Unlike a
// StopGradient view it never copies: the view of a variable is copied before it is handed on (src/op.rs:273-287), which
// for a convolution over a variable would be a copy of the whole input for the sake of four numbers.
struct ExtentsOf : Op {
    const char *name() const override { return "ExtentsOf"; }
    OpError compute(ComputeContext &ctx) const override
    {
        ctx.append_output(NdArray::extents_only(ctx.input_shape(0)));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override { ctx.append_input_grad(std::nullopt); }
};

static Tensor extents_of(Tensor x)
{
    return x.graph->builder().append_input(x, false).set_differentiable(false).build(std::make_unique<ExtentsOf>());
}

struct ScalarOp : Op {  // const_gen_ops.rs Scalar
    float value;
    explicit ScalarOp(float v) : value(v) {}
    const char *name() const override { return "Scalar"; }
    OpError compute(ComputeContext &ctx) const override
    {
        ctx.append_output(NdArray::scalar(value));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override { (void)ctx; }
};

// zeros(shape(x)) with the shape read from x's array.
struct ZerosLike : Op {
    const char *name() const override { return "Zeros"; }
    OpError compute(ComputeContext &ctx) const override
    {
        ctx.append_output(NdArray::zeros(ctx.input(0).shape()));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override { ctx.append_input_grad(std::nullopt); }
};

// A constant spread over the extents of input 0: what broadcasting a constant gradient back through a
// reduction gives (ReduceSumToScalarGrad, ReduceGradCommon: reduction_ops.rs:139-159, 459-512) when that
// gradient is itself a constant -- the seed scalar(1) of a back-propagation and everything between it and the
// first tensor that depends on data.  One fill instead of a fill, a broadcast per reduction and a division per
// mean: the nodes it stands for are never evaluated.  `mean_axes[j]`: the value is divided by the product of
// those extents of input 1 + j, as f32, for the j-th mean reduction the constant passed back through -- the
// arithmetic of the nodes it replaces, in their order.
struct FilledLike : Op {
    float value;
    std::vector<std::vector<int>> mean_axes;
    FilledLike(float v, std::vector<std::vector<int>> m) : value(v), mean_axes(std::move(m)) {}
    const char *name() const override { return "FilledLike"; }
    // The constant after its divisions; division j reads the extents of input `first_ref + j`.
    OpError resolve(ComputeContext &ctx, size_t first_ref, float *out) const
    {
        float v = value;
        for (size_t j = 0; j < mean_axes.size(); ++j) {
            const NdArray x = ctx.input(first_ref + j);
            const int rank = x.ndim();
            float len = 1.f;
            for (int a : mean_axes[j]) {
                const int ax = a < 0 ? a + rank : a;
                if (ax < 0 || ax >= rank) return OpError::make(ErrorKind::OutOfBounds, "reduce: axis out of range");
                len *= (float)x.shape()[(size_t)ax];
            }
            v = v / len;
        }
        *out = v;
        return OpError::none();
    }
    OpError compute(ComputeContext &ctx) const override
    {
        float v;
        const OpError e = resolve(ctx, 1, &v);
        if (!e.ok()) return e;
        ctx.append_output(NdArray::filled(ctx.input(0).shape(), v));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        for (size_t i = 0; i < ctx.num_inputs(); ++i) ctx.append_input_grad(std::nullopt);
    }
};

// The broadcast of `gy` over the extents of `x` as a FilledLike node when gy is a constant (a Scalar or a
// FilledLike node); `mean_axes` != null: followed by the division by those extents of x.
std::optional<Tensor> constant_broadcast(Graph *g, Tensor gy, Tensor x, const std::vector<int> *mean_axes)
{
    const TensorInternal &n = g->node(gy.id);
    float value;
    std::vector<std::vector<int>> divisions;
    std::vector<Tensor> refs;
    if (const auto *s = dynamic_cast<const ScalarOp *>(n.op.get())) {
        value = s->value;
    } else if (const auto *f = dynamic_cast<const FilledLike *>(n.op.get())) {
        value = f->value;
        divisions = f->mean_axes;
        for (size_t i = 1; i < n.incoming_nodes.size(); ++i) refs.push_back(g->tensor(n.incoming_nodes[i].id));
    } else {
        return std::nullopt;
    }
    if (mean_axes) {
        divisions.push_back(*mean_axes);
        refs.push_back(x);
    }
    TensorBuilder b = g->builder();
    b.append_input(x, false);
    for (const Tensor &r : refs) b.append_input(r, false);
    return b.build(std::make_unique<FilledLike>(value, std::move(divisions)));
}

// ------------------------------------------------------------------------------------------
// convolution                                   conv_ops/conv2d.rs, conv_ops/conv2d_transpose.rs
// ------------------------------------------------------------------------------------------
struct Conv2D;
struct Conv2DTranspose;
struct Conv2DFilterGrad;
struct Conv2DWithCols;
struct Conv2DTransposeFilterGrad;

struct ConvHyper {
    int pad, stride, dilation;
};

struct Conv2DTransposeFilterGrad : Op, ConvHyper {  // conv2d_transpose.rs:433-480
    explicit Conv2DTransposeFilterGrad(ConvHyper h) : ConvHyper(h) {}
    const char *name() const override { return "Conv2DTransposeFilterGrad"; }
    OpError compute(ComputeContext &ctx) const override;
    void grad(GradientContext &ctx) const override;
};

// The scratch of the column-free gradients of one convolution -- the zero-bordered upstream gradient with the filter in
// tap order behind it (ag_conv_input_grad_prepare_f32) -- is the same for the filter gradient and the input gradient.
// Whichever of the two nodes runs first leaves it on gy (NdArray::set_derived), the other finds it there instead of
// copying gy again: 0.15 ms of a 3 ms backward at B = 256, 128 channels, 56 x 56.
static NdArray bordered_gradient(void *stream, const NdArray &gy, const NdArray &w, size_t floats, int B, int K, int OH, int OW,
                                 int C, int kh, int kw, int pad, int stride, int dilation, int H, int W, OpError *err)
{
    const std::vector<int64_t> key = {(int64_t)floats, (int64_t)(intptr_t)w.allocation(), w.version(), B, K, OH, OW, C, kh, kw,
                                      pad, stride, dilation, H, W};
    NdArray scratch = gy.derived(key);
    if (scratch.defined()) return scratch;
    scratch = NdArray::empty({(int64_t)floats});
    *err = from_status(ag_conv_input_grad_prepare_f32(stream, gy.ptr(), w.ptr(), scratch.ptr(), B, K, OH, OW, C, kh, kw, pad, stride,
                                                      dilation, H, W));
    if (err->ok()) gy.set_derived(key, scratch);
    return scratch;
}

// Column elements from which the host operators take the column-free routines (below, the step is bound by its
// launches and the column path has fewer).
constexpr int64_t kColumnFreeFrom = 8LL << 20;

struct Conv2DTranspose : Op, ConvHyper {  // conv2d_transpose.rs:249-301
    // Inputs (gy, w) as in the reference, which reconstructs the output extent from gy
    // (conv2d_transpose.rs:55-56).  An optional third input supplies the extent instead (only its
    // shape is read): Conv2D::grad passes the convolution's input there, so the input gradient
    // has the input's size even when (H + 2p - k_eff) is not a multiple of the stride.
    explicit Conv2DTranspose(ConvHyper h) : ConvHyper(h) {}
    const char *name() const override { return "Conv2DTranspose"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray gy = ctx.input(0), w = ctx.input(1);
        int out_h = -1, out_w = -1;
        if (ctx.num_inputs() > 2) {
            const NdArray like = ctx.input(2);
            if (like.ndim() == 4) {
                out_h = (int)like.shape()[2];
                out_w = (int)like.shape()[3];
            }
        }
        if (gy.ndim() != 4)
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "conv2d_transpose: Input must be 4D (got " + shape_str(gy.shape()) + ")");
        if (w.ndim() != 4)
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "conv2d_transpose: Filter must be 4D (got " + shape_str(w.shape()) + ")");
        const int B = (int)gy.shape()[0], ych = (int)gy.shape()[1], yh = (int)gy.shape()[2], yw = (int)gy.shape()[3];
        const int xch = (int)w.shape()[1], kh = (int)w.shape()[2], kw = (int)w.shape()[3];
        if (ych != w.shape()[0])
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "conv2d_transpose: Number of input channels (" + std::to_string(ych) +
                                     ") must match second filter dim (" + std::to_string(w.shape()[0]) + ")");
        const int xh = out_h >= 0 ? out_h : ag_conv_transpose_out_size(yh, kh, pad, stride, dilation);
        const int xw = out_w >= 0 ? out_w : ag_conv_transpose_out_size(yw, kw, pad, stride, dilation);
        if (xh < 0 || xw < 0)
            return OpError::make(ErrorKind::IncompatibleShape, "conv2d_transpose: negative output extent");
        NdArray gx = NdArray::empty({B, xch, xh, xw});
        // the staged column-free routines where a column-free Conv2D stands in front (same size gate), so that the
        // bordered gradient is shared with the filter gradient
        const int64_t col_elems = (int64_t)B * xch * kh * kw * yh * yw;
        const size_t staged = col_elems >= kColumnFreeFrom && B > 0
                                  ? ag_conv_input_grad_scratch_floats(B, ych, yh, yw, xch, kh, kw, pad, stride, dilation, xh, xw)
                                  : 0;
        if (staged > 0) {
            OpError e = OpError::none();
            NdArray scratch = bordered_gradient(ctx.stream(), gy, w, staged, B, ych, yh, yw, xch, kh, kw, pad, stride, dilation, xh,
                                                xw, &e);
            if (!e.ok()) return e;
            e = from_status(ag_conv_input_grad_gemm_f32(ctx.stream(), scratch.ptr(), gx.ptr(), B, ych, yh, yw, xch, kh, kw, pad, stride,
                                                        dilation, xh, xw));
            if (!e.ok()) return e;
            ctx.append_output(gx);
            return OpError::none();
        }
        NdArray gcols = NdArray::empty({B, (int64_t)xch * kh * kw, (int64_t)yh * yw});
        const OpError e = from_status(ag_conv2d_transpose_f32(ctx.stream(), gy.ptr(), w.ptr(), gx.ptr(), gcols.ptr(), B,
                                                              ych, yh, yw, xch, kh, kw, pad, stride, dilation, xh, xw));
        if (!e.ok()) return e;
        ctx.append_output(gx);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override;
};

struct Conv2DFilterGrad : Op, ConvHyper {  // conv2d.rs:736-776
    explicit Conv2DFilterGrad(ConvHyper h) : ConvHyper(h) {}
    const char *name() const override { return "Conv2DFilterGrad"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray cols = ctx.input(0), gy = ctx.input(1), w = ctx.input(2);
        if (gy.ndim() != 4)
            return OpError::make(ErrorKind::IncompatibleShape, "Conv2DFilterGrad: gradient must be 4D (got " + shape_str(gy.shape()) + ")");
        if (w.ndim() != 4)
            return OpError::make(ErrorKind::IncompatibleShape, "Conv2DFilterGrad: filter must be 4D (got " + shape_str(w.shape()) + ")");
        const int B = (int)gy.shape()[0], K = (int)gy.shape()[1], P = (int)(gy.shape()[2] * gy.shape()[3]);
        const int CK = (int)(w.shape()[1] * w.shape()[2] * w.shape()[3]);
        NdArray gw = NdArray::empty(w.shape());
        if (cols.ndim() == 1) {  // the rearranged input of a column-free Conv2D (stride 1, or stride 2 with dilation 1)
            const int C = (int)w.shape()[1], kh = (int)w.shape()[2], kw = (int)w.shape()[3];
            const int OH = (int)gy.shape()[2], OW = (int)gy.shape()[3];
            // extents of x: from the optional fourth input (only its shape is read), else what a unit
            // stride implies
            int H = OH + kh - 1 - 2 * pad, W = OW + kw - 1 - 2 * pad;
            bool have_extents = false;
            if (ctx.num_inputs() > 3) {
                const NdArray like = ctx.input(3);  // (an input may be taken once)
                if (like.ndim() == 4) {
                    H = (int)like.shape()[2];
                    W = (int)like.shape()[3];
                    have_extents = true;
                }
            }
            if (!have_extents && stride != 1)
                return OpError::make(ErrorKind::IncompatibleShape, "Conv2DFilterGrad: the input's extents are needed for stride 2");
            const size_t n_gyp = ag_conv_input_grad_scratch_floats(B, K, OH, OW, C, kh, kw, pad, stride, dilation, H, W);
            const size_t nb = ag_conv2d_filter_grad_nocols_f32_workspace(B, C, H, W, K, kh, kw, pad, stride, dilation);
            if (n_gyp == 0 || nb == 0 || cols.len() != ag_conv2d_nocols_scratch_floats(B, C, H, W, K, kh, kw, pad, stride, dilation))
                return OpError::make(ErrorKind::IncompatibleShape, "Conv2DFilterGrad: the rearranged input does not match gy and the filter");
            OpError e = OpError::none();
            NdArray gyp = bordered_gradient(ctx.stream(), gy, w, n_gyp, B, K, OH, OW, C, kh, kw, pad, stride, dilation, H, W, &e);
            if (!e.ok()) return e;
            NdArray ws = workspace(nb);
            e = from_status(ag_conv2d_filter_grad_nocols_f32(ctx.stream(), cols.ptr(), gyp.ptr(), gw.ptr(), B, C, H, W, K, kh, kw,
                                                             pad, stride, dilation, ws.ptr(), ws.len() * 4));
            if (!e.ok()) return e;
            ctx.append_output(gw);
            return OpError::none();
        }
        const size_t nb = ag_conv2d_filter_grad_f32_workspace(B, CK, P, K);
        NdArray ws = workspace(nb);
        const OpError e = from_status(
            ag_conv2d_filter_grad_f32(ctx.stream(), cols.ptr(), gy.ptr(), gw.ptr(), B, CK, P, K, ws.ptr(), ws.len() * 4));
        if (!e.ok()) return e;
        ctx.append_output(gw);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override;
};

struct Conv2DWithCols : Op, ConvHyper {  // conv2d.rs:589-629
    explicit Conv2DWithCols(ConvHyper h) : ConvHyper(h) {}
    const char *name() const override { return "Conv2DWithCols"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray cols = ctx.input(0), w = ctx.input(1);
        if (w.ndim() != 4)
            return OpError::make(ErrorKind::IncompatibleShape, "Conv2DWithCols: filter must be 4D (got " + shape_str(w.shape()) + ")");
        if (cols.ndim() != 1 && cols.ndim() < 3)
            return OpError::make(ErrorKind::IncompatibleShape, "Conv2DWithCols: columns must have at least 3 axes (got " + shape_str(cols.shape()) + ")");
        if (cols.ndim() == 1) {
            // the zero-bordered input of a column-free Conv2D; the third input (only its extents are
            // read) has the shape of the result
            if (ctx.num_inputs() < 3) return OpError::make(ErrorKind::IncompatibleShape, "Conv2DWithCols: columns expected");
            const NdArray like = ctx.input(2);
            if (like.ndim() != 4) return OpError::make(ErrorKind::IncompatibleShape, "Conv2DWithCols: 4D result extents expected");
            const int B = (int)like.shape()[0], OH = (int)like.shape()[2], OW = (int)like.shape()[3];
            const int K = (int)w.shape()[0], C = (int)w.shape()[1], kh = (int)w.shape()[2], kw = (int)w.shape()[3];
            int H = OH + kh - 1 - 2 * pad, W = OW + kw - 1 - 2 * pad;
            bool have_extents = false;
            if (ctx.num_inputs() > 3) {  // extents of x (needed for stride 2)
                const NdArray xl = ctx.input(3);  // (an input may be taken once)
                if (xl.ndim() == 4) {
                    H = (int)xl.shape()[2];
                    W = (int)xl.shape()[3];
                    have_extents = true;
                }
            }
            if (!have_extents && stride != 1)
                return OpError::make(ErrorKind::IncompatibleShape, "Conv2DWithCols: the input's extents are needed for stride 2");
            if (cols.len() != ag_conv2d_nocols_scratch_floats(B, C, H, W, K, kh, kw, pad, stride, dilation))
                return OpError::make(ErrorKind::IncompatibleShape, "Conv2DWithCols: the rearranged input does not match the filter");
            NdArray y = NdArray::empty({B, K, OH, OW});
            NdArray wf = NdArray::empty(w.shape());
            const OpError e = from_status(ag_conv2d_nocols_with_filter_f32(ctx.stream(), cols.ptr(), w.ptr(), wf.ptr(), y.ptr(), B, C,
                                                                           H, W, K, kh, kw, pad, stride, dilation));
            if (!e.ok()) return e;
            ctx.append_output(y);
            return OpError::none();
        }
        // cols carries [B, C*kh*kw, OH, OW] here (the reference labels it [B,C,kw,kh,OH,OW], conv2d.rs:484)
        const int B = (int)cols.shape()[0], K = (int)w.shape()[0];
        const int CK = (int)(w.shape()[1] * w.shape()[2] * w.shape()[3]);
        const int OH = (int)cols.shape()[cols.ndim() - 2], OW = (int)cols.shape()[cols.ndim() - 1];
        NdArray y = NdArray::empty({B, K, OH, OW});
        const OpError e = from_status(ag_conv2d_with_cols_f32(ctx.stream(), cols.ptr(), w.ptr(), y.ptr(), B, CK, OH * OW, K));
        if (!e.ok()) return e;
        ctx.append_output(y);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override;
};

struct Conv2D : Op, ConvHyper {  // conv2d.rs:531-587
    // true: always write the im2col columns as output 1, like the reference (no column-free path)
    bool materialise_columns;
    explicit Conv2D(ConvHyper h, bool columns = false) : ConvHyper(h), materialise_columns(columns) {}
    const char *name() const override { return "Conv2D"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0), w = ctx.input(1);
        // conv2d_extract_params, conv2d.rs:349-404
        if (x.ndim() != 4)
            return OpError::make(ErrorKind::IncompatibleShape, "conv2d: lhs input must be 4D (got " + shape_str(x.shape()) + ")");
        if (w.ndim() != 4)
            return OpError::make(ErrorKind::IncompatibleShape, "conv2d: filter must be 4D (got " + shape_str(w.shape()) + ")");
        if (x.shape()[1] != w.shape()[1])
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "conv2d: input channel dim (" + std::to_string(x.shape()[1]) +
                                     ") must match filter's second dim (" + std::to_string(w.shape()[1]) + ")");
        const int B = (int)x.shape()[0], C = (int)x.shape()[1], H = (int)x.shape()[2], W = (int)x.shape()[3];
        const int K = (int)w.shape()[0], kh = (int)w.shape()[2], kw = (int)w.shape()[3];
        const int OH = ag_conv_out_size(H, kh, pad, stride, dilation), OW = ag_conv_out_size(W, kw, pad, stride, dilation);
        if (OH <= 0 || OW <= 0)
            return OpError::make(ErrorKind::IncompatibleShape, "conv2d: filter extent exceeds the padded input");
        NdArray y = NdArray::empty({B, K, OH, OW});
        // Column-free path when all three contractions of this convolution support it: the second
        // output, which only Conv2DFilterGrad and Conv2DWithCols read, is then the zero-bordered
        // input (rank 1) instead of the columns.
        // (small problems are launch-bound and the column path has fewer launches: from 32 MB of columns on --
        // 128 images of 32 -> 64 channels at 14 x 14, 7.2 M column elements, cost the same either way; 32 images of
        // 256 -> 256 channels at 14 x 14 with dilation 2, 14.5 M, take 0.27 ms without columns and 0.31 ms with them)
        const bool large = (long long)B * C * kh * kw * OH * OW >= kColumnFreeFrom;
        const size_t n_xpad =
            (large && !materialise_columns) ? ag_conv2d_nocols_scratch_floats(B, C, H, W, K, kh, kw, pad, stride, dilation) : 0;
        if (n_xpad > 0 && ag_conv2d_filter_grad_nocols_f32_workspace(B, C, H, W, K, kh, kw, pad, stride, dilation) > 0 &&
            ag_conv_input_grad_scratch_floats(B, K, OH, OW, C, kh, kw, pad, stride, dilation, H, W) > 0) {
            NdArray xpad = NdArray::empty({(int64_t)n_xpad});
            const OpError e = from_status(ag_conv2d_fwd_nocols_f32(ctx.stream(), x.ptr(), w.ptr(), y.ptr(), xpad.ptr(), B, C, H, W, K,
                                                                   kh, kw, pad, stride, dilation));
            if (!e.ok()) return e;
            ctx.append_output(y);
            ctx.append_output(xpad);
            return OpError::none();
        }
        NdArray cols = NdArray::empty({B, (int64_t)C * kh * kw, OH, OW});
        const OpError e = from_status(ag_conv2d_fwd_f32(ctx.stream(), x.ptr(), w.ptr(), y.ptr(), cols.ptr(), B, C, H, W, K, kh,
                                                        kw, pad, stride, dilation));
        if (!e.ok()) return e;
        ctx.append_output(y);
        ctx.append_output(cols);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        Graph *g = ctx.graph();
        const Tensor gy = ctx.output_grad(), y = ctx.output(), x = ctx.input(0), w = ctx.input(1);
        const Tensor gx = build(g, {gy, w, extents_of(x)},
                                std::make_unique<Conv2DTranspose>(ConvHyper{pad, stride, dilation}));
        const Tensor cols = tensor_ops::nth_tensor(y, 1);
        const Tensor gw = g->builder()
                              .append_input(cols, false)
                              .append_input(gy, false)
                              .append_input(w, false)
                              .append_input(extents_of(x), false)  // extents of x only
                              .append_backprop_input(x)
                              .append_backprop_input(gy)
                              .build(std::make_unique<Conv2DFilterGrad>(ConvHyper{pad, stride, dilation}));
        ctx.append_input_grad(gx);
        ctx.append_input_grad(gw);
    }
};

void Conv2DWithCols::grad(GradientContext &ctx) const
{
    Graph *g = ctx.graph();
    const Tensor cols = ctx.input(0), w = ctx.input(1), y = ctx.output(), gy = ctx.output_grad();
    const Tensor gx = build(g, {gy, w}, std::make_unique<Conv2DTranspose>(ConvHyper{pad, stride, dilation}));
    const Tensor x0 = g->tensor(g->node(y.id).get_backprop_inputs()[0].id);
    const Tensor gw = g->builder()
                          .append_input(cols, false)
                          .append_input(gy, false)
                          .append_input(w, false)
                          .append_input(extents_of(x0), false)  // extents of x only
                          .append_backprop_input(x0)
                          .append_backprop_input(gy)
                          .build(std::make_unique<Conv2DFilterGrad>(ConvHyper{pad, stride, dilation}));
    ctx.append_input_grad(gx);
    ctx.append_input_grad(gw);
}

void Conv2DFilterGrad::grad(GradientContext &ctx) const
{
    // conv2d.rs:746-775: two gradients for the two back-prop inputs (x, gy)
    Graph *g = ctx.graph();
    const Tensor cols = ctx.input(0), gy = ctx.input(1), ggw = ctx.output_grad(), y = ctx.output();
    const Tensor gx = build(g, {gy, ggw}, std::make_unique<Conv2DTranspose>(ConvHyper{pad, stride, dilation}));
    const Tensor x0 = g->tensor(g->node(y.id).get_backprop_inputs()[0].id);
    const Tensor ggy = g->builder()
                           .append_input(cols, false)
                           .append_input(ggw, false)
                           .append_input(extents_of(gy), false)  // extents of the result
                           .append_input(extents_of(x0), false)  // extents of x
                           .append_backprop_input(x0)
                           .append_backprop_input(ggw)
                           .build(std::make_unique<Conv2DWithCols>(ConvHyper{pad, stride, dilation}));
    ctx.append_input_grad(gx);
    ctx.append_input_grad(ggy);
}

void Conv2DTranspose::grad(GradientContext &ctx) const
{
    // conv2d_transpose.rs:274-300
    Graph *g = ctx.graph();
    const Tensor x = ctx.input(0), w = ctx.input(1), gy = ctx.output_grad();
    const Tensor gx = build(g, {gy, w}, std::make_unique<Conv2D>(ConvHyper{pad, stride, dilation}));
    const Tensor gw = build(g, {gy, x, tensor_ops::stop_gradient(w)},
                            std::make_unique<Conv2DTransposeFilterGrad>(ConvHyper{pad, stride, dilation}));
    ctx.append_input_grad(gx);
    ctx.append_input_grad(gw);
    if (ctx.num_inputs() > 2) ctx.append_input_grad(std::nullopt);  // the extent-only input
}

OpError Conv2DTransposeFilterGrad::compute(ComputeContext &ctx) const
{
    const NdArray gy = ctx.input(0), x = ctx.input(1), w = ctx.input(2);
    if (gy.ndim() != 4 || x.ndim() != 4 || w.ndim() != 4)
        return OpError::make(ErrorKind::IncompatibleShape, "Conv2DTransposeFilterGrad: gradient, input and filter must be 4D (got " +
                                                               shape_str(gy.shape()) + ", " + shape_str(x.shape()) + ", " +
                                                               shape_str(w.shape()) + ")");
    const int B = (int)x.shape()[0], ych = (int)x.shape()[1], yh = (int)x.shape()[2], yw = (int)x.shape()[3];
    const int xch = (int)gy.shape()[1], H = (int)gy.shape()[2], W = (int)gy.shape()[3];
    const int kh = (int)w.shape()[2], kw = (int)w.shape()[3];
    NdArray gw = NdArray::empty(w.shape());
    NdArray gycols = NdArray::empty({B, (int64_t)xch * kh * kw, (int64_t)yh * yw});
    const size_t nb = ag_conv2d_filter_grad_f32_workspace(B, xch * kh * kw, yh * yw, ych);
    NdArray ws = workspace(nb);
    const OpError e = from_status(ag_conv2d_transpose_filter_grad_f32(ctx.stream(), x.ptr(), gy.ptr(), gw.ptr(), gycols.ptr(),
                                                                      B, ych, yh, yw, xch, H, W, kh, kw, pad, stride, dilation,
                                                                      ws.ptr(), ws.len() * 4));
    if (!e.ok()) return e;
    ctx.append_output(gw);
    return OpError::none();
}

void Conv2DTransposeFilterGrad::grad(GradientContext &ctx) const
{
    // conv2d_transpose.rs:453-479
    Graph *g = ctx.graph();
    const Tensor gy = ctx.input(0), gw = ctx.output_grad(), x = ctx.input(1);
    const Tensor ggy = build(g, {x, gw}, std::make_unique<Conv2DTranspose>(ConvHyper{pad, stride, dilation}));
    const Tensor ggx = build(g, {gy, gw}, std::make_unique<Conv2D>(ConvHyper{pad, stride, dilation}));
    ctx.append_input_grad(ggy);
    ctx.append_input_grad(ggx);
    ctx.append_input_grad(std::nullopt);
}

// ------------------------------------------------------------------------------------------
// max pooling                                                       conv_ops/max_pool2d.rs
// ------------------------------------------------------------------------------------------
struct PoolHyper {
    int pad, stride, size;
};

// Outputs of MaxPool2D: [0] y, [1] argmax as f32 (the reference's encoding), [2] one tap byte per
// output (the exact selection inside each window, packed four to an f32 of a rank-1 array; an
// addition of this implementation that the backward uses so it stays exact above 2^24 elements).
struct MaxPool2DGradGrad : Op, PoolHyper {  // max_pool2d.rs:297-337
    explicit MaxPool2DGradGrad(PoolHyper h) : PoolHyper(h) {}
    const char *name() const override { return "MaxPool2DGradGrad"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray ggx = ctx.input(0), argmax = ctx.input(1), idx = ctx.input(2);
        const int B = (int)ggx.shape()[0], C = (int)ggx.shape()[1], H = (int)ggx.shape()[2], W = (int)ggx.shape()[3];
        NdArray ggy = NdArray::empty(argmax.shape());
        const OpError e = from_status(ag_maxpool2d_gradgrad_f32(ctx.stream(), ggx.ptr(), argmax.ptr(),
                                                                reinterpret_cast<const uint8_t *>(idx.ptr()), ggy.ptr(), B, C,
                                                                H, W, size, pad, stride));
        if (!e.ok()) return e;
        ctx.append_output(ggy);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        ctx.append_input_grad(std::nullopt);
        ctx.append_input_grad(std::nullopt);
        ctx.append_input_grad(std::nullopt);
    }
};

struct MaxPool2DGrad : Op, PoolHyper {  // max_pool2d.rs:245-295
    // Inputs (gy, argmax, exact indices[, x]).  Without the optional last input the input extent
    // is reconstructed like the reference (max_pool2d.rs:263-264); MaxPool2D::grad passes x so
    // that the gradient has x's size (the reference's reconstruction is too small whenever
    // (H - size) is not a multiple of the stride, and it then writes out of bounds).
    // relu_masked: one more input at the end, the input (or output) x of a ReLU; the result is multiplied by
    // greater(x, 0) as it is stored -- this node then stands for ReLUGrad(x, MaxPool2DGrad(...)), the pair that
    // every conv -> relu -> pool block back-propagates through (relu_grad_node builds it).
    bool relu_masked;
    explicit MaxPool2DGrad(PoolHyper h, bool masked = false) : PoolHyper(h), relu_masked(masked) {}
    const char *name() const override { return relu_masked ? "MaxPool2DGradReLU" : "MaxPool2DGrad"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray gy = ctx.input(0), argmax = ctx.input(1), idx = ctx.input(2);
        int in_h = -1, in_w = -1;
        const size_t plain_inputs = ctx.num_inputs() - (relu_masked ? 1 : 0);
        if (plain_inputs > 3) {
            const NdArray like = ctx.input(3);
            if (like.ndim() == 4) {
                in_h = (int)like.shape()[2];
                in_w = (int)like.shape()[3];
            }
        }
        const int B = (int)gy.shape()[0], C = (int)gy.shape()[1], yh = (int)gy.shape()[2], yw = (int)gy.shape()[3];
        const int xh = in_h >= 0 ? in_h : ag_pool_grad_in_size(yh, size, pad, stride);
        const int xw = in_w >= 0 ? in_w : ag_pool_grad_in_size(yw, size, pad, stride);
        NdArray gx = NdArray::empty({B, C, xh, xw});
        OpError e;
        if (relu_masked) {
            const NdArray mask = ctx.input(ctx.num_inputs() - 1);
            if (mask.shape() != gx.shape()) return OpError::make(ErrorKind::IncompatibleShape, "relu grad: shapes differ");
            e = from_status(ag_maxpool2d_bwd_relu_f32(ctx.stream(), gy.ptr(), argmax.ptr(), reinterpret_cast<const uint8_t *>(idx.ptr()),
                                                      mask.ptr(), gx.ptr(), B, C, xh, xw, size, pad, stride));
        } else {
            e = from_status(ag_maxpool2d_bwd_f32(ctx.stream(), gy.ptr(), argmax.ptr(), reinterpret_cast<const uint8_t *>(idx.ptr()),
                                                 gx.ptr(), B, C, xh, xw, size, pad, stride));
        }
        if (!e.ok()) return e;
        ctx.append_output(gx);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override;
};

struct MaxPool2D : Op, PoolHyper {  // max_pool2d.rs:166-243
    explicit MaxPool2D(PoolHyper h) : PoolHyper(h) {}
    const char *name() const override { return "MaxPool2D"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0);
        if (x.ndim() != 4) return OpError::make(ErrorKind::IncompatibleShape, "max_pool2d: input must be 4D (got " + shape_str(x.shape()) + ")");
        const int B = (int)x.shape()[0], C = (int)x.shape()[1], H = (int)x.shape()[2], W = (int)x.shape()[3];
        const int OH = ag_pool_out_size(H, size, pad, stride), OW = ag_pool_out_size(W, size, pad, stride);
        const Shape ys{B, C, std::max(OH, 0), std::max(OW, 0)};
        NdArray y = NdArray::empty(ys), argmax = NdArray::empty(ys);
        NdArray idx = NdArray::empty({(int64_t)((y.len() + 3) / 4 + 1)});
        const OpError e = from_status(ag_maxpool2d_fwd_f32(ctx.stream(), x.ptr(), y.ptr(), argmax.ptr(),
                                                           reinterpret_cast<uint8_t *>(idx.ptr()), B, C, H, W, size, pad, stride));
        if (!e.ok()) return e;
        ctx.append_output(y);
        ctx.append_output(argmax);
        ctx.append_output(idx);
        return OpError::none();
    }
    // relu(x) or relu(a + b) in front of a 2 x 2 pooling at stride 2: one pass writes the activation and pools it
    // (ag_relu_maxpool2d_2x2_f32); defined behind the ReLU ops below.
    bool fuses_with_producer(const Op &producer) const override;
    bool compute_with_producer(ComputeContext &ctx, const Op &producer, std::vector<NdArray> *producer_outputs,
                               OpError *status) const override;
    void grad(GradientContext &ctx) const override
    {
        // max_pool2d.rs:229-242, with the input extent taken from x instead of being reconstructed
        const Tensor gy = ctx.output_grad(), y = ctx.output();
        const Tensor indices = tensor_ops::nth_tensor(y, 1), exact = tensor_ops::nth_tensor(y, 2);
        const Tensor gx = build(ctx.graph(), {gy, indices, exact, extents_of(ctx.input(0))},
                                std::make_unique<MaxPool2DGrad>(PoolHyper{pad, stride, size}));
        ctx.append_input_grad(gx);
    }
};

// ------------------------------------------------------------------------------------------
// MatMul / BatchMatMul                                                     dot_ops.rs:554-718
// ------------------------------------------------------------------------------------------
struct MatMul : Op {
    bool transpose_a, transpose_b;
    MatMul(bool ta, bool tb) : transpose_a(ta), transpose_b(tb) {}
    const char *name() const override { return "MatMul"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray a = ctx.input(0), b = ctx.input(1);
        if (a.ndim() != 2) throw Panic("lhs input for MatMul must be 2D");  // `expect` panics, dot_ops.rs:566-573
        if (b.ndim() != 2) throw Panic("rhs input for MatMul must be 2D");
        const int64_t m = transpose_a ? a.shape()[1] : a.shape()[0], k = transpose_a ? a.shape()[0] : a.shape()[1];
        const int64_t k2 = transpose_b ? b.shape()[1] : b.shape()[0], n = transpose_b ? b.shape()[0] : b.shape()[1];
        if (k != k2)
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "ndarray: inputs " + std::to_string(m) + " \xc3\x97 " + std::to_string(k) + " and " +
                                     std::to_string(k2) + " \xc3\x97 " + std::to_string(n) +
                                     " are not compatible for matrix multiplication");
        NdArray c = NdArray::empty({m, n});
        NdArray ws = workspace(ag_matmul_f32_workspace((int)m, (int)n, (int)k));
        const OpError e = from_status(ag_matmul_f32(ctx.stream(), transpose_a, transpose_b, (int)m, (int)n, (int)k, a.ptr(),
                                                    (int)std::max<int64_t>(a.shape()[1], 1), b.ptr(),
                                                    (int)std::max<int64_t>(b.shape()[1], 1), c.ptr(),
                                                    (int)std::max<int64_t>(n, 1), ws.ptr(), ws.len() * 4));
        if (!e.ok()) return e;
        ctx.append_output(c);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        // dot_ops.rs:608-628
        const Tensor gy = ctx.output_grad();
        ctx.append_input_grad(build(ctx.graph(), {gy, ctx.input(1)}, std::make_unique<MatMul>(false, true)));
        ctx.append_input_grad(build(ctx.graph(), {ctx.input(0), gy}, std::make_unique<MatMul>(true, false)));
    }
};

struct BatchMatMul : Op {
    bool transpose_a, transpose_b;
    BatchMatMul(bool ta, bool tb) : transpose_a(ta), transpose_b(tb) {}
    const char *name() const override { return "BatchMatMul"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x0 = ctx.input(0), x1 = ctx.input(1);
        const int r0 = x0.ndim(), r1 = x1.ndim();
        if (r0 < 2)
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "BatchMatMul: Left-hand-side input's ndim must be >= 2, actual: " + std::to_string(r0));
        if (r1 < 2)
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "BatchMatMul: Right-hand-side input's ndim must be >= 2, actual: " + std::to_string(r1));
        Shape s0 = x0.shape(), s1 = x1.shape();
        if (transpose_a) std::swap(s0[r0 - 2], s0[r0 - 1]);
        if (transpose_b) std::swap(s1[r1 - 2], s1[r1 - 1]);
        if (r0 != r1 || !std::equal(s0.begin(), s0.end() - 2, s1.begin()) || s0[r0 - 1] != s1[r1 - 2])
            return OpError::make(ErrorKind::IncompatibleShape, "Input shapes mismatch: " + shape_str(s0) + " vs " + shape_str(s1));
        const int64_t m = s0[r0 - 2], k = s0[r0 - 1], n = s1[r1 - 1];
        int64_t batch = 1;
        for (int i = 0; i < r0 - 2; ++i) batch *= s0[i];
        Shape out(s0.begin(), s0.end() - 2);
        out.push_back(m);
        out.push_back(n);
        NdArray c = NdArray::empty(out);
        const int64_t lda = x0.shape()[r0 - 1], ldb = x1.shape()[r1 - 1];
        const OpError e = from_status(ag_gemm_f32(ctx.stream(), transpose_a, transpose_b, (int)m, (int)n, (int)k, 1.f, x0.ptr(),
                                                  (int)std::max<int64_t>(lda, 1), x0.shape()[r0 - 2] * lda, x1.ptr(),
                                                  (int)std::max<int64_t>(ldb, 1), x1.shape()[r1 - 2] * ldb, 0.f, c.ptr(),
                                                  (int)std::max<int64_t>(n, 1), m * n, (int)batch));
        if (!e.ok()) return e;
        ctx.append_output(c);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        // dot_ops.rs:697-717
        const Tensor gy = ctx.output_grad();
        ctx.append_input_grad(build(ctx.graph(), {gy, ctx.input(1)}, std::make_unique<BatchMatMul>(false, true)));
        ctx.append_input_grad(build(ctx.graph(), {ctx.input(0), gy}, std::make_unique<BatchMatMul>(true, false)));
    }
};

// ------------------------------------------------------------------------------------------
// reductions                                                               reduction_ops.rs
// ------------------------------------------------------------------------------------------
std::vector<int> normalize_axes(const std::vector<int> &axes, int rank)
{
    std::vector<int> r;
    for (int a : axes) r.push_back(a < 0 ? a + rank : a);
    return r;
}

// ReduceGradCommon (:459-512): broadcast gy back to the shape of x.  The reference passes
// shape(x) as a tensor; here x itself is the second input and only its extents are read.
struct ReduceGradCommon : Op {
    std::vector<int> axes;
    float divide_by_len;  // != 0: additionally divide by the reduced length (ReduceMean::grad, :217-238)
    bool should_make_broadcast_dims;  // = !keep_dims of the reduction this is the gradient of (:221-232)
    ReduceGradCommon(std::vector<int> a, bool mean, bool make_dims)
        : axes(std::move(a)), divide_by_len(mean ? 1.f : 0.f), should_make_broadcast_dims(make_dims) {}
    const char *name() const override { return "ReduceGradCommon"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray gy = ctx.input(0), x = ctx.input(1);
        const int rank = x.ndim();
        std::vector<int> shape(x.shape().begin(), x.shape().end());
        const std::vector<int> ax = normalize_axes(axes, rank);
        NdArray gx = NdArray::empty(x.shape());
        OpError e = from_status(ag_broadcast_grad_f32(ctx.stream(), gy.ptr(), gx.ptr(), shape.data(), rank, ax.data(), (int)ax.size()));
        if (!e.ok()) return e;
        if (divide_by_len != 0.f) {
            float len = 1.f;  // reduce_prod of the gathered extents, as f32
            for (int a : ax) len *= (float)shape[(size_t)a];
            e = from_status(ag_div_scalar_f32(ctx.stream(), gx.ptr(), len, gx.ptr(), gx.len()));
            if (!e.ok()) return e;
        }
        ctx.append_output(gx);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        // the gradient of a broadcast is the matching sum, with keep_dims = should_make_broadcast_dims
        // as the reference has it (:498-511); the division by the reduced length that this op
        // fuses (a separate Div node in the reference, :231-234) passes through as the mean's 1/len
        Tensor s = divide_by_len != 0.f ? tensor_ops::reduce_mean(ctx.output_grad(), axes, should_make_broadcast_dims)
                                        : tensor_ops::reduce_sum(ctx.output_grad(), axes, should_make_broadcast_dims);
        ctx.append_input_grad(s);
        ctx.append_input_grad(std::nullopt);
    }
};

struct ReduceSum : Op {
    std::vector<int> axes;
    bool keep_dims, mean;
    ReduceSum(std::vector<int> a, bool k, bool m) : axes(std::move(a)), keep_dims(k), mean(m) {}
    const char *name() const override { return mean ? "ReduceMean" : "ReduceSum"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0);
        const int rank = x.ndim();
        std::vector<int> ax = normalize_axes(axes, rank);
        for (int a : ax)
            if (a < 0 || a >= rank) return OpError::make(ErrorKind::OutOfBounds, "reduce: axis out of range");
        if (rank == 0 || ax.empty()) {  // the reference returns a view of x (:63-70, :192-195)
            ctx.append_output_view(x);
            return OpError::none();
        }
        std::vector<int> shape(x.shape().begin(), x.shape().end());
        Shape out;
        for (int i = 0; i < rank; ++i) {
            const bool red = std::find(ax.begin(), ax.end(), i) != ax.end();
            if (!red) out.push_back(shape[(size_t)i]);
            else if (keep_dims) out.push_back(1);
        }
        NdArray y = NdArray::empty(out);
        const size_t nb = ag_reduce_sum_f32_workspace(shape.data(), rank, ax.data(), (int)ax.size());
        NdArray ws = workspace(nb);
        const OpError e = from_status(ag_reduce_sum_f32(ctx.stream(), x.ptr(), y.ptr(), shape.data(), rank, ax.data(),
                                                        (int)ax.size(), mean ? 1 : 0, ws.ptr(), ws.len() * 4));
        if (!e.ok()) return e;
        ctx.append_output(y);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        if (const auto c = constant_broadcast(ctx.graph(), ctx.output_grad(), ctx.input(0), mean ? &axes : nullptr)) {
            ctx.append_input_grad(*c);
            return;
        }
        const Tensor gx = build(ctx.graph(), {ctx.output_grad(), ctx.input(0)}, std::make_unique<ReduceGradCommon>(axes, mean, !keep_dims));
        ctx.append_input_grad(gx);
    }
};

struct ReduceSumToScalarGrad;

struct ReduceSumToScalar : Op {  // :123-137
    const char *name() const override { return "ReduceSumToScalar"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0);
        NdArray out = NdArray::empty({});
        NdArray ws = workspace(ag_sum_all_f32_workspace(x.len()));
        const OpError e = from_status(ag_sum_all_f32(ctx.stream(), x.ptr(), x.len(), out.ptr(), ws.ptr(), ws.len() * 4));
        if (!e.ok()) return e;
        ctx.append_output(out);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override;
};

struct ReduceSumToScalarGrad : Op {  // :139-159; input 1 is x (for its extents) instead of shape(x)
    const char *name() const override { return "ReduceSumToScalarGrad"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray gy = ctx.input(0), x = ctx.input(1);
        const int rank = x.ndim();
        std::vector<int> shape(x.shape().begin(), x.shape().end()), ax((size_t)rank);
        for (int i = 0; i < rank; ++i) ax[(size_t)i] = i;
        NdArray gx = NdArray::empty(x.shape());
        const OpError e = from_status(ag_broadcast_grad_f32(ctx.stream(), gy.ptr(), gx.ptr(), shape.data(), rank, ax.data(), rank));
        if (!e.ok()) return e;
        ctx.append_output(gx);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        ctx.append_input_grad(build(ctx.graph(), {ctx.output_grad()}, std::make_unique<ReduceSumToScalar>()));
        ctx.append_input_grad(std::nullopt);
    }
};

void ReduceSumToScalar::grad(GradientContext &ctx) const
{
    if (const auto c = constant_broadcast(ctx.graph(), ctx.output_grad(), ctx.input(0), nullptr)) {
        ctx.append_input_grad(*c);
        return;
    }
    ctx.append_input_grad(build(ctx.graph(), {ctx.output_grad(), ctx.input(0)}, std::make_unique<ReduceSumToScalarGrad>()));
}

// ------------------------------------------------------------------------------------------
// elementwise and loss glue
// ------------------------------------------------------------------------------------------
struct ReLUGrad : Op {  // greater(x, 0) * gy as one kernel (activation_ops.rs:161-166)
    const char *name() const override { return "ReLUGrad"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0), gy = ctx.input(1);
        if (x.shape() != gy.shape()) return OpError::make(ErrorKind::IncompatibleShape, "relu grad: shapes differ");
        NdArray gx = NdArray::empty(x.shape());
        const OpError e = from_status(ag_relu_grad_f32(ctx.stream(), x.ptr(), gy.ptr(), gx.ptr(), x.len()));
        if (!e.ok()) return e;
        ctx.append_output(gx);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        // second order: d/dgy (mask * gy) = mask * ggx; the mask itself has zero gradient
        ctx.append_input_grad(std::nullopt);
        ctx.append_input_grad(build(ctx.graph(), {ctx.input(0), ctx.output_grad()}, std::make_unique<ReLUGrad>()));
    }
};

// ReLUGrad(x, gy) as a node; when gy is the gradient of a max pooling, as one node with it (the MaxPool2DGrad node
// that gy names is then evaluated only if something else asks for it).
Tensor relu_grad_node(Graph *g, Tensor x, Tensor gy)
{
    const TensorInternal &n = g->node(gy.id);
    const auto *pool = dynamic_cast<const MaxPool2DGrad *>(n.op.get());
    if (pool && !pool->relu_masked && n.incoming_nodes.size() >= 3) {
        TensorBuilder b = g->builder();
        for (const IncomingTensor &in : n.incoming_nodes) b.append_input_with_selector(g->tensor(in.id), false, in.array_selector);
        b.append_input(x, false);
        return b.build(std::make_unique<MaxPool2DGrad>(PoolHyper{pool->pad, pool->stride, pool->size}, true));
    }
    return build(g, {x, gy}, std::make_unique<ReLUGrad>());
}

void MaxPool2DGrad::grad(GradientContext &ctx) const
{
    // second order: gx is linear in gy; the mask of the fused form multiplies the incoming gradient first
    Tensor ggx = ctx.output_grad();
    const size_t n = ctx.num_inputs();
    if (relu_masked) ggx = build(ctx.graph(), {ctx.input(n - 1), ggx}, std::make_unique<ReLUGrad>());
    const Tensor argmax = ctx.input(1), idx = ctx.input(2);
    const Tensor ggy = build(ctx.graph(), {ggx, argmax, idx}, std::make_unique<MaxPool2DGradGrad>(PoolHyper{pad, stride, size}));
    ctx.append_input_grad(ggy);
    for (size_t i = 1; i < n; ++i) ctx.append_input_grad(std::nullopt);
}

struct ReLU : Op {  // activation_ops.rs:154-167
    const char *name() const override { return "ReLU"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0);
        NdArray y = NdArray::empty(x.shape());
        const OpError e = from_status(ag_relu_f32(ctx.stream(), x.ptr(), y.ptr(), x.len()));
        if (!e.ok()) return e;
        ctx.append_output(y);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        ctx.append_input_grad(relu_grad_node(ctx.graph(), ctx.input(0), ctx.output_grad()));
    }
};

// MaybeReduceSum (binary_ops.rs:39-105): reduce gy to the shape of the operand it belongs to.
// Input 1 is that operand (only its extents are read).
// True when `b` is `a` without its leading axis, or with a leading axis of extent 1: the bias
// shapes of the reference's examples ([1, classes] on [batch, classes], [1, C, H, W] on NCHW).
static bool broadcasts_over_rows(const Shape &a, const Shape &b)
{
    if (a.empty() || a[0] == 0) return false;
    if (b.size() == a.size()) return b[0] == 1 && std::equal(a.begin() + 1, a.end(), b.begin() + 1);
    return b.size() + 1 == a.size() && std::equal(a.begin() + 1, a.end(), b.begin());
}

// True when `b` has `a`'s rank and every axis of `b` is either `a`'s or 1 (ndarray broadcasting of
// operands of equal rank); a one-element `b` of any rank counts as all ones (binary_ops.rs:54-60).
static bool broadcasts_along_axes(const Shape &a, const Shape &b, std::vector<int> *bshape)
{
    size_t blen = 1;
    for (const int64_t d : b) blen *= (size_t)d;
    if (a.empty() || a.size() > 8) return false;
    bshape->assign(a.size(), 1);
    if (blen == 1) return true;
    if (b.size() != a.size()) return false;
    for (size_t i = 0; i < a.size(); ++i) {
        if (b[i] != a[i] && b[i] != 1) return false;
        if (a[i] > 0x7fffffff) return false;
        (*bshape)[i] = (int)b[i];
    }
    return true;
}

struct MaybeReduceSum : Op {
    const char *name() const override { return "MaybeReduceSum"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray gy = ctx.input(0), x = ctx.input(1);
        if (gy.shape() == x.shape()) {
            ctx.append_output_view(gy);
            return OpError::none();
        }
        if (broadcasts_over_rows(gy.shape(), x.shape())) {
            NdArray out = NdArray::empty(x.shape());
            const size_t rows = (size_t)gy.shape()[0];
            OpError e;
            if (gy.len() >= ((size_t)1 << 20) && rows <= 0x7fffffff && gy.len() / rows <= 0x7fffffff) {
                // large gradients: the streaming fold over axis 0 instead of one sequential chain per column
                const int shape[2] = {(int)rows, (int)(gy.len() / rows)}, axis = 0;
                NdArray ws = workspace(ag_reduce_sum_f32_workspace(shape, 2, &axis, 1));
                e = from_status(ag_reduce_sum_f32(ctx.stream(), gy.ptr(), out.ptr(), shape, 2, &axis, 1, 0, ws.ptr(), ws.len() * 4));
            } else {
                e = from_status(ag_bias_grad_f32(ctx.stream(), gy.ptr(), out.ptr(), rows, gy.len() / rows));
            }
            if (!e.ok()) return e;
            ctx.append_output(out);
            return OpError::none();
        }
        std::vector<int> xshape;
        if (broadcasts_along_axes(gy.shape(), x.shape(), &xshape)) {
            // sum over every axis the operand was broadcast along (binary_ops.rs:69-87)
            std::vector<int> shape(gy.shape().begin(), gy.shape().end()), axes;
            for (int i = 0; i < (int)shape.size(); ++i)
                if (xshape[(size_t)i] == 1 && shape[(size_t)i] > 1) axes.push_back(i);
            if (axes.empty()) {  // same elements, other extents of 1 (binary_ops.rs:62-66)
                ctx.append_output_view(gy.reshaped(x.shape()));
                return OpError::none();
            }
            NdArray out = NdArray::empty(x.shape());
            const size_t nb = ag_reduce_sum_f32_workspace(shape.data(), (int)shape.size(), axes.data(), (int)axes.size());
            NdArray ws = workspace(nb);
            const OpError e = from_status(ag_reduce_sum_f32(ctx.stream(), gy.ptr(), out.ptr(), shape.data(), (int)shape.size(),
                                                            axes.data(), (int)axes.size(), 0, ws.ptr(), ws.len() * 4));
            if (!e.ok()) return e;
            ctx.append_output(out);
            return OpError::none();
        }
        return OpError::make(ErrorKind::IncompatibleShape,
                             "MaybeReduceSum: cannot reduce " + shape_str(gy.shape()) + " to " + shape_str(x.shape()));
    }
    void grad(GradientContext &ctx) const override
    {
        ctx.append_input_grad(std::nullopt);
        ctx.append_input_grad(std::nullopt);
    }
};

struct AddOp : Op {  // binary_ops.rs:147-166, 304-346
    const char *name() const override { return "AddOp"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray a = ctx.input(0), b = ctx.input(1);
        NdArray y = NdArray::empty(a.shape());
        OpError e;
        if (a.shape() == b.shape()) {
            const float *xs[2] = {a.ptr(), b.ptr()};
            e = from_status(ag_add_n_f32(ctx.stream(), xs, 2, y.ptr(), a.len()));
        } else if (broadcasts_over_rows(a.shape(), b.shape())) {
            const size_t rows = (size_t)a.shape()[0];
            e = from_status(ag_add_bias_f32(ctx.stream(), a.ptr(), b.ptr(), y.ptr(), rows, a.len() / rows));
        } else if (std::vector<int> bshape; broadcasts_along_axes(a.shape(), b.shape(), &bshape)) {
            const std::vector<int> shape(a.shape().begin(), a.shape().end());
            e = from_status(ag_add_broadcast_f32(ctx.stream(), a.ptr(), b.ptr(), y.ptr(), shape.data(), bshape.data(), (int)shape.size()));
        } else {
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "AddOp: unsupported broadcast " + shape_str(a.shape()) + " + " + shape_str(b.shape()));
        }
        if (!e.ok()) return e;
        ctx.append_output(y);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        const Tensor gy = ctx.output_grad();
        ctx.append_input_grad(build(ctx.graph(), {gy, ctx.input(0)}, std::make_unique<MaybeReduceSum>()));
        ctx.append_input_grad(build(ctx.graph(), {gy, ctx.input(1)}, std::make_unique<MaybeReduceSum>()));
    }
};

// AddOp followed by ReLU as one node: what tensor_ops::relu builds when its argument is an AddOp node, with
// that node's two operands as inputs.  The value is relu(a + b) bit for bit; the AddOp node stays in the graph and
// is evaluated only if something else asks for it.  For back-propagation the node's only input is the AddOp
// node itself (`backprop_inputs`): the gradient it hands on is the mask taken from this node's own OUTPUT
// (y > 0 exactly where a + b > 0) -- what ReLU::grad hands to its argument (activation_ops.rs:154-167) -- and
// AddOp::grad carries it on to the operands, so that the sum stays differentiable like any other node
// (grad(loss, [a + b]) and everything else that names the sum see the graph of the two operations).
struct AddReLU : Op {
    const char *name() const override { return "AddReLU"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray a = ctx.input(0), b = ctx.input(1);
        std::vector<int> bshape;
        if (a.shape() == b.shape()) {
            bshape.assign(a.shape().begin(), a.shape().end());
        } else if (broadcasts_over_rows(a.shape(), b.shape())) {
            bshape.assign(a.shape().begin(), a.shape().end());
            bshape[0] = 1;
        } else if (!broadcasts_along_axes(a.shape(), b.shape(), &bshape)) {
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "AddOp: unsupported broadcast " + shape_str(a.shape()) + " + " + shape_str(b.shape()));
        }
        if (a.shape().size() > 8)
            return OpError::make(ErrorKind::IncompatibleShape, "AddOp: rank " + std::to_string(a.shape().size()) + " not in 0..8");
        NdArray y = NdArray::empty(a.shape());
        if (a.shape().empty()) {
            // 0-dimensional operands whose rank was not known when the graph was built: the two operations in turn
            const float *xs[2] = {a.ptr(), b.ptr()};
            OpError e0 = from_status(ag_add_n_f32(ctx.stream(), xs, 2, y.ptr(), a.len()));
            if (e0.ok()) e0 = from_status(ag_relu_f32(ctx.stream(), y.ptr(), y.ptr(), y.len()));
            if (!e0.ok()) return e0;
            ctx.append_output(y);
            return OpError::none();
        }
        const std::vector<int> shape(a.shape().begin(), a.shape().end());
        const OpError e = from_status(ag_add_broadcast_relu_f32(ctx.stream(), a.ptr(), b.ptr(), y.ptr(), shape.data(),
                                                                bshape.data(), (int)shape.size()));
        if (!e.ok()) return e;
        ctx.append_output(y);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        // one back-prop input: the AddOp node
        ctx.append_input_grad(relu_grad_node(ctx.graph(), ctx.output(), ctx.output_grad()));
    }
};

bool MaxPool2D::fuses_with_producer(const Op &producer) const
{
    if (size != 2 || stride != 2 || pad != 0) return false;
    return dynamic_cast<const ReLU *>(&producer) != nullptr || dynamic_cast<const AddReLU *>(&producer) != nullptr;
}

bool MaxPool2D::compute_with_producer(ComputeContext &ctx, const Op &producer, std::vector<NdArray> *producer_outputs,
                                      OpError *status) const
{
    const bool with_sum = dynamic_cast<const AddReLU *>(&producer) != nullptr;
    if (ctx.num_inputs() != (with_sum ? 2u : 1u)) return false;
    const Shape &as = ctx.input_shape(0);
    if (as.size() != 4 || as[2] < 2 || as[3] < 2 || as[2] % 2 != 0 || as[3] % 2 != 0 || as[0] * as[1] == 0) return false;
    std::vector<int> bshape;
    if (with_sum) {  // the operand patterns of AddReLU::compute, for rank 4
        const Shape &bs = ctx.input_shape(1);
        if (as == bs) {
            bshape.assign(as.begin(), as.end());
        } else if (broadcasts_over_rows(as, bs)) {
            bshape.assign(as.begin(), as.end());
            bshape[0] = 1;
        } else if (!broadcasts_along_axes(as, bs, &bshape)) {
            return false;
        }
        if (bshape.size() != 4) return false;
    }
    const NdArray a = ctx.input(0);
    const NdArray b = with_sum ? ctx.input(1) : NdArray();
    if ((reinterpret_cast<uintptr_t>(a.ptr()) & 7u) != 0) {  // (never with arrays of the arena; the kernel asks for it)
        *status = OpError::make(ErrorKind::NdArrayError, "max_pool2d: misaligned input");
        return true;
    }
    const int B = (int)as[0], C = (int)as[1], H = (int)as[2], W = (int)as[3];
    const Shape ys{B, C, H / 2, W / 2};
    NdArray r = NdArray::empty(as), y = NdArray::empty(ys), argmax = NdArray::empty(ys);
    NdArray idx = NdArray::empty({(int64_t)((y.len() + 3) / 4 + 1)});
    *status = from_status(ag_relu_maxpool2d_2x2_f32(ctx.stream(), a.ptr(), with_sum ? b.ptr() : nullptr,
                                                    with_sum ? bshape.data() : nullptr, r.ptr(), y.ptr(), argmax.ptr(),
                                                    reinterpret_cast<uint8_t *>(idx.ptr()), B, C, H, W));
    if (!status->ok()) return true;
    producer_outputs->push_back(r);
    ctx.append_output(y);
    ctx.append_output(argmax);
    ctx.append_output(idx);
    return true;
}

struct MulOp : Op {  // binary_ops.rs:209-237 (same-shape operands)
    const char *name() const override { return "MulOp"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray a = ctx.input(0), b = ctx.input(1);
        if (a.shape() != b.shape())
            return OpError::make(ErrorKind::IncompatibleShape, "MulOp: shapes " + shape_str(a.shape()) + " and " + shape_str(b.shape()) + " differ");
        NdArray y = NdArray::empty(a.shape());
        const OpError e = from_status(ag_mul_f32(ctx.stream(), a.ptr(), b.ptr(), y.ptr(), a.len()));
        if (!e.ok()) return e;
        ctx.append_output(y);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        const Tensor gy = ctx.output_grad();
        ctx.append_input_grad(tensor_ops::mul(gy, ctx.input(1)));
        ctx.append_input_grad(tensor_ops::mul(gy, ctx.input(0)));
    }
};

struct AddN : Op {  // array_ops.rs:503-535
    const char *name() const override { return "AddN"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const size_t n = ctx.num_inputs();
        if (n == 0) throw Panic("add_n: no inputs");
        std::vector<NdArray> xs;
        for (size_t i = 0; i < n; ++i) xs.push_back(ctx.input(i));
        if (n == 1) {
            ctx.append_output_view(xs[0]);
            return OpError::none();
        }
        // the empty outputs of in-place updates (one zero scalar shared by all of them) add up to that zero
        bool all_empty = true;
        for (const NdArray &x : xs) all_empty = all_empty && x.allocation() == NdArray::shared_zero().allocation();
        if (all_empty) {
            ctx.append_empty_output();
            return OpError::none();
        }
        for (size_t i = 1; i < n; ++i)
            if (xs[i].shape() != xs[0].shape()) return OpError::make(ErrorKind::IncompatibleShape, "add_n: shapes differ");
        NdArray acc = NdArray::empty(xs[0].shape());
        // ((x0 + x1) + x2) + ... in groups of at most 8 operands per launch
        size_t done = 0;
        bool have_acc = false;
        while (done < n) {
            const float *ptrs[8];
            int cnt = 0;
            if (have_acc) ptrs[cnt++] = acc.ptr();
            while (cnt < 8 && done < n) ptrs[cnt++] = xs[done++].ptr();
            const OpError e = from_status(ag_add_n_f32(ctx.stream(), ptrs, cnt, acc.ptr(), acc.len()));
            if (!e.ok()) return e;
            have_acc = true;
        }
        ctx.append_output(acc);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        for (size_t i = 0; i < ctx.num_inputs(); ++i) ctx.append_input_grad(ctx.output_grad());
    }
};

struct ReshapeLike : Op {  // gradient of Reshape: back to the extents of input 1
    const char *name() const override { return "Reshape"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray gy = ctx.input(0), x = ctx.input(1);
        if (gy.len() != x.len()) return OpError::make(ErrorKind::IncompatibleShape, "reshape: element counts differ");
        ctx.append_output_view(gy.reshaped(x.shape()));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        // a reshape again (array_ops.rs:226-238); the input that only lends its extents gets none
        ctx.append_input_grad(build(ctx.graph(), {ctx.output_grad(), ctx.input(0)}, std::make_unique<ReshapeLike>()));
        ctx.append_input_grad(std::nullopt);
    }
};

struct Reshape : Op {  // array_ops.rs:183-239: a view when the input is contiguous (always, here)
    Shape target;
    explicit Reshape(Shape s) : target(std::move(s)) {}
    const char *name() const override { return "Reshape"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0);
        Shape s = target;
        int64_t known = 1;
        int unknown = -1;
        for (size_t i = 0; i < s.size(); ++i) {
            if (s[i] == -1) {
                if (unknown >= 0) return OpError::make(ErrorKind::IncompatibleShape, "reshape: more than one -1 in " + shape_str(target));
                unknown = (int)i;
            } else {
                known *= s[i];
            }
        }
        if (unknown >= 0) {
            if (known == 0 || x.len() % (size_t)known) return OpError::make(ErrorKind::IncompatibleShape, "reshape: cannot infer -1");
            s[(size_t)unknown] = (int64_t)(x.len() / (size_t)known);
        }
        size_t n = 1;
        for (int64_t d : s) n *= (size_t)d;
        if (n != x.len())
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "reshape: cannot reshape " + shape_str(x.shape()) + " into " + shape_str(target));
        ctx.append_output_view(x.reshaped(s));
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        ctx.append_input_grad(build(ctx.graph(), {ctx.output_grad(), ctx.input(0)}, std::make_unique<ReshapeLike>()));
    }
};

struct SparseSoftmaxCrossEntropyGrad : Op {  // xent_ops.rs:139-158
    const char *name() const override { return "SparseSoftmaxCrossEntropyGrad"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray lsm = ctx.input(0), t = ctx.input(1), gy = ctx.input(2);
        NdArray gx = NdArray::empty(lsm.shape());
        const OpError e = from_status(ag_sparse_softmax_xent_grad_f32(ctx.stream(), lsm.ptr(), t.ptr(), gy.ptr(), gx.ptr(),
                                                                      (size_t)lsm.shape()[0], (size_t)lsm.shape()[1]));
        if (!e.ok()) return e;
        ctx.append_output(gx);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        ctx.append_input_grad(std::nullopt);
        ctx.append_input_grad(std::nullopt);
    }
};

// The same gradient computed from the logits, so that an evaluation that never asks for the loss does not run the
// forward at all.  Inputs (logits, labels, gy); or, when the upstream gradient is a constant (a FilledLike node: the
// mean of a batch loss), (logits, labels, the inputs of that node), with the constant resolved on the host and handed
// to the kernel as an argument -- no array is filled for it.
struct SparseSoftmaxCrossEntropyGradLogits : Op {
    std::optional<FilledLike> constant;
    explicit SparseSoftmaxCrossEntropyGradLogits(std::optional<FilledLike> c) : constant(std::move(c)) {}
    const char *name() const override { return "SparseSoftmaxCrossEntropyGradLogits"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0), t = ctx.input(1);
        if (x.ndim() != 2)
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "SparseSoftmaxCrossEntropy: given first argument's ndim is not 2: shape=" + shape_str(x.shape()));
        if (t.len() != (size_t)x.shape()[0]) throw Panic("Batch size mismatch: inputs vs labels");
        float value = 0.f;
        const float *gy = nullptr;
        NdArray gy_array;
        if (constant) {
            const OpError e = constant->resolve(ctx, 3, &value);  // input 2 is the constant's shape source
            if (!e.ok()) return e;
        } else {
            gy_array = ctx.input(2);
            if (gy_array.len() != (size_t)x.shape()[0]) return OpError::make(ErrorKind::IncompatibleShape, "SparseSoftmaxCrossEntropyGrad: one upstream gradient per row expected");
            gy = gy_array.ptr();
        }
        NdArray gx = NdArray::empty(x.shape());
        const OpError e = from_status(ag_sparse_softmax_xent_grad_logits_f32(ctx.stream(), x.ptr(), t.ptr(), gy, value, gx.ptr(),
                                                                             (size_t)x.shape()[0], (size_t)x.shape()[1]));
        if (!e.ok()) return e;
        ctx.append_output(gx);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        for (size_t i = 0; i < ctx.num_inputs(); ++i) ctx.append_input_grad(std::nullopt);
    }
};

struct SparseSoftmaxCrossEntropy : Op {  // xent_ops.rs:63-137
    const char *name() const override { return "SparseSoftmaxCrossEntropy"; }
    OpError compute(ComputeContext &ctx) const override
    {
        const NdArray x = ctx.input(0), t = ctx.input(1);
        if (x.ndim() != 2)
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "SparseSoftmaxCrossEntropy: given first argument's ndim is not 2: shape=" + shape_str(x.shape()));
        if (!(t.ndim() == 1 || (t.ndim() == 2 && t.shape()[1] == 1)))
            return OpError::make(ErrorKind::IncompatibleShape,
                                 "SparseSoftmaxCrossEntropy: second argument's shape must be (batch_size, 1) or (batch_size,). given shape=" +
                                     shape_str(t.shape()));
        if (t.len() != (size_t)x.shape()[0]) throw Panic("Batch size mismatch: inputs vs labels");
        NdArray loss = NdArray::empty({x.shape()[0], 1}), lsm = NdArray::empty(x.shape());
        const OpError e = from_status(ag_sparse_softmax_xent_f32(ctx.stream(), x.ptr(), t.ptr(), loss.ptr(), lsm.ptr(),
                                                                 (size_t)x.shape()[0], (size_t)x.shape()[1]));
        if (!e.ok()) return e;
        ctx.append_output(loss);
        ctx.append_output(lsm);
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        // from the logits rather than from this node's log-softmax (same bits): the forward then runs only when
        // something asks for the loss
        const Tensor x = ctx.input(0), t = ctx.input(1), gy = ctx.output_grad();
        Graph *g = ctx.graph();
        const TensorInternal &gn = g->node(gy.id);
        TensorBuilder b = g->builder();
        b.append_input(x, false);
        b.append_input(t, false);
        std::optional<FilledLike> constant;
        if (const auto *f = dynamic_cast<const FilledLike *>(gn.op.get())) {
            constant.emplace(f->value, f->mean_axes);
            // The constant usually takes its extents from this node's own loss [rows, 1] (the mean over the batch of
            // the loss): the logits [rows, classes] stand in wherever only the row count is read, so that the
            // gradient does not depend on the forward.
            const TensorID self = ctx.output().id;
            for (size_t i = 0; i < gn.incoming_nodes.size(); ++i) {
                const IncomingTensor &in = gn.incoming_nodes[i];
                bool rows_only = true;  // input 0 gives the fill's shape, which nothing reads here
                if (i >= 1)
                    for (int a : f->mean_axes[i - 1]) rows_only = rows_only && (a == 0 || a == -2);
                if (in.id == self && in.array_selector == 0 && rows_only) b.append_input(x, false);
                else b.append_input_with_selector(g->tensor(in.id), false, in.array_selector);
            }
        } else {
            b.append_input(gy, false);
        }
        ctx.append_input_grad(b.build(std::make_unique<SparseSoftmaxCrossEntropyGradLogits>(std::move(constant))));
        ctx.append_input_grad(std::nullopt);  // the reference builds a label gradient "that won't be used in most cases"
    }
};

// ------------------------------------------------------------------------------------------
// AdamOp                                                  gradient_descent_ops/adam.rs:3-67
// ------------------------------------------------------------------------------------------
struct AdamOp : Op {
    float alpha, eps, b1, b2;
    AdamOp(float a, float e, float x, float y) : alpha(a), eps(e), b1(x), b2(y) {}
    const char *name() const override { return "AdamOp"; }
    OpError compute(ComputeContext &ctx) const override
    {
        NdArray t = ctx.input_mut(4);
        const NdArray g = ctx.input(1);
        NdArray m = ctx.input_mut(2), v = ctx.input_mut(3), p = ctx.input_mut(0);
        if (g.len() != p.len() || m.len() != p.len() || v.len() != p.len())
            return OpError::make(ErrorKind::IncompatibleShape, "AdamOp: parameter, gradient and moment shapes differ");
        if (t.len() < 1) return OpError::make(ErrorKind::IncompatibleShape, "AdamOp: empty step counter");
        ctx.adam_update(AdamJob{p, g, m, v, t, alpha, eps, b1, b2});
        ctx.append_empty_output();
        return OpError::none();
    }
    void grad(GradientContext &ctx) const override
    {
        for (int i = 0; i < 5; ++i) ctx.append_input_grad(std::nullopt);
    }
};

}  // namespace

// ---------------------------------------------------------------------------------------------
// tensor_ops                                                          src/tensor_ops/mod.rs
// ---------------------------------------------------------------------------------------------
namespace tensor_ops {

Tensor nth_tensor(Tensor x, int n)
{
    return x.graph->builder().append_input_with_selector(x, false, n).build(std::make_unique<Identity>());
}

Tensor dilated_conv2d(Tensor x, Tensor w, int pad, int stride, int dilate)
{
    return build(x.graph, {x, w}, std::make_unique<Conv2D>(ConvHyper{pad, stride, dilate}));
}
Tensor conv2d(Tensor x, Tensor w, int pad, int stride) { return dilated_conv2d(x, w, pad, stride, 1); }
Tensor conv2d_with_columns(Tensor x, Tensor w, int pad, int stride, int dilate)
{
    return build(x.graph, {x, w}, std::make_unique<Conv2D>(ConvHyper{pad, stride, dilate}, true));
}

Tensor dilated_conv2d_transpose(Tensor x, Tensor w, int pad, int stride, int dilate)
{
    return build(x.graph, {x, w}, std::make_unique<Conv2DTranspose>(ConvHyper{pad, stride, dilate}));
}
Tensor conv2d_transpose(Tensor x, Tensor w, int pad, int stride) { return dilated_conv2d_transpose(x, w, pad, stride, 1); }

Tensor max_pool2d(Tensor x, int pool_size, int pad, int stride)
{
    return build(x.graph, {x}, std::make_unique<MaxPool2D>(PoolHyper{pad, stride, pool_size}));
}

Tensor matmul(Tensor a, Tensor b) { return build(a.graph, {a, b}, std::make_unique<MatMul>(false, false)); }
Tensor batch_matmul_t(Tensor a, Tensor b, bool ta, bool tb) { return build(a.graph, {a, b}, std::make_unique<BatchMatMul>(ta, tb)); }
Tensor batch_matmul(Tensor a, Tensor b) { return batch_matmul_t(a, b, false, false); }

Tensor reduce_sum(Tensor x, const std::vector<int> &axes, bool keep_dims)
{
    return build(x.graph, {x}, std::make_unique<ReduceSum>(axes, keep_dims, false));
}
Tensor reduce_mean(Tensor x, const std::vector<int> &axes, bool keep_dims)
{
    return build(x.graph, {x}, std::make_unique<ReduceSum>(axes, keep_dims, true));
}
Tensor sum_all(Tensor x) { return build(x.graph, {x}, std::make_unique<ReduceSumToScalar>()); }
Tensor relu(Tensor x)
{
    // relu(a + b): one fused node over a and b (the bias-activation step after a convolution)
    const TensorInternal &n = x.graph->node(x.id);
    // (the sum itself is the node's back-prop input; operands known to be 0-dimensional keep the two nodes: the fused
    // kernel takes ranks 1..8)
    if (dynamic_cast<const AddOp *>(n.op.get()) && n.incoming_nodes.size() == 2 && n.incoming_nodes[0].array_selector == 0 &&
        n.incoming_nodes[1].array_selector == 0 && !n.incoming_nodes[0].allow_mut && !n.incoming_nodes[1].allow_mut) {
        const TensorInternal &lhs = x.graph->node(n.incoming_nodes[0].id);
        const bool rank0 = lhs.known_shape && lhs.known_shape->empty();
        if (!rank0)
            return x.graph->builder()
                .append_input(x.graph->tensor(n.incoming_nodes[0].id), false)
                .append_input(x.graph->tensor(n.incoming_nodes[1].id), false)
                .append_backprop_input(x)
                .build(std::make_unique<AddReLU>());
    }
    return build(x.graph, {x}, std::make_unique<ReLU>());
}
Tensor add(Tensor a, Tensor b) { return build(a.graph, {a, b}, std::make_unique<AddOp>()); }
Tensor mul(Tensor a, Tensor b) { return build(a.graph, {a, b}, std::make_unique<MulOp>()); }

Tensor add_n(const std::vector<Tensor> &xs)
{
    if (xs.empty()) throw Panic("add_n: no inputs");
    if (xs.size() == 1) return xs[0];  // mod.rs:831-847
    TensorBuilder b = xs[0].graph->builder();
    for (const Tensor &t : xs) b.append_input(t, false);
    return b.build(std::make_unique<AddN>());
}

Tensor reshape(Tensor x, const Shape &shape) { return build(x.graph, {x}, std::make_unique<Reshape>(shape)); }

Tensor sparse_softmax_cross_entropy(Tensor logits, Tensor labels)
{
    return build(logits.graph, {logits, labels}, std::make_unique<SparseSoftmaxCrossEntropy>());
}

Tensor scalar(float v, Graph *g) { return g->builder().set_known_shape(Shape{}).build(std::make_unique<ScalarOp>(v)); }

Tensor zeros_like(Tensor x)
{
    return x.graph->builder().append_input(x, false).set_differentiable(false).build(std::make_unique<ZerosLike>());
}

Tensor stop_gradient(Tensor x)
{
    return x.graph->builder().append_input(x, false).set_differentiable(false).build(std::make_unique<StopGradient>());
}

}  // namespace tensor_ops

// ---------------------------------------------------------------------------------------------
// Adam                                                              src/optimizers/adam.rs
// ---------------------------------------------------------------------------------------------
namespace optimizers {

Adam::Adam(float alpha, float eps, float b1, float b2, const std::vector<VariableID> &vars, VariableEnvironment &env,
           std::string adam_namespace_id)
    : alpha_(alpha), eps_(eps), b1_(b1), b2_(b2), ns_(std::move(adam_namespace_id))
{
    for (VariableID vid : vars) {
        const Shape shape = env.array(vid).shape();
        env.set(ns_, std::to_string(vid) + "m", NdArray::zeros(shape));
        env.set(ns_, std::to_string(vid) + "v", NdArray::zeros(shape));
        env.set(ns_, std::to_string(vid) + "t", NdArray::scalar(1.f));
    }
}

std::vector<Tensor> Adam::compute_updates(const std::vector<Tensor> &params, const std::vector<Tensor> &grads,
                                          Context &ctx) const
{
    if (params.size() != grads.size()) throw Panic("assertion failed: num_params == grads.len()");
    std::vector<Tensor> ret;
    for (size_t i = 0; i < params.size(); ++i) {
        const VariableID vid = ctx.node(params[i].id).variable_id;
        if (vid < 0) throw Panic("Got non-variable tensor");
        const Tensor m = ctx.variable(std::to_string(vid) + "m", ns_);
        const Tensor v = ctx.variable(std::to_string(vid) + "v", ns_);
        const Tensor t = ctx.variable(std::to_string(vid) + "t", ns_);
        ret.push_back(ctx.builder()
                          .append_input(params[i], true)
                          .append_input(grads[i], false)
                          .append_input(m, true)
                          .append_input(v, true)
                          .append_input(t, true)
                          .build(std::make_unique<AdamOp>(alpha_, eps_, b1_, b2_)));
    }
    return ret;
}

void Adam::update(const std::vector<Tensor> &params, const std::vector<Tensor> &grads, Context &ctx,
                  const std::vector<std::pair<std::string, NdArray>> &feeds) const
{
    const std::vector<Tensor> ops = compute_updates(params, grads, ctx);
    for (const EvalResult &r : ctx.eval(ops, feeds))
        if (!r.error.ok()) throw Panic("called `Result::unwrap()` on an `Err` value: " + r.error.message);
}

Tensor Adam::get_update_op(const std::vector<Tensor> &params, const std::vector<Tensor> &grads, Context &ctx) const
{
    return tensor_ops::add_n(compute_updates(params, grads, ctx));
}

}  // namespace optimizers

}  // namespace host
}  // namespace ag
