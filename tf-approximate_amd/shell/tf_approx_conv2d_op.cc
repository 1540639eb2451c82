// TensorFlow registration of ApproxConv2DWithMinMaxVars on top of axconv::ApproxConv2DOp.
//
// Built only with -DAXCONV_WITH_TENSORFLOW against a TensorFlow (ROCm) installation; TensorFlow is not part of
// this repository's toolchain, so this translation unit is NOT compiled by build.py and its build is unverified.
// The op's registered interface is the reference's (tf2/src/approx_nn_ops.cpp:38-54): six inputs (input,
// filter and the four min/max scalars), one output, attrs T, strides, num_bits, mul_map_file, padding,
// explicit_paddings, data_format, dilations, and the Conv2D shape function with explicit padding.  A graph or
// a Python caller (tf2/test/test_table_approx_conv_2d.py:47-49) that used the reference's library loads this
// one instead and sees the same op.
#ifdef AXCONV_WITH_TENSORFLOW

#include <hip/hip_runtime.h>

#include "approx_conv2d_op.h"
#include "tensorflow/core/framework/common_shape_fns.h"
#include "tensorflow/core/framework/op.h"
#include "tensorflow/core/framework/op_kernel.h"
#include "tensorflow/core/util/padding.h"

namespace tensorflow {

REGISTER_OP("ApproxConv2DWithMinMaxVars")
    .Input("input: T")
    .Input("filter: T")
    .Input("input_min: T")
    .Input("input_max: T")
    .Input("filter_min: T")
    .Input("filter_max: T")
    .Output("output: T")
    .Attr("T: {half, bfloat16, float, double}")
    .Attr("strides: list(int)")
    .Attr("num_bits: int")
    .Attr("mul_map_file: string")
    .Attr(GetPaddingAttrStringWithExplicit())
    .Attr(GetExplicitPaddingsAttrString())
    .Attr(GetConvnetDataFormatAttrString())
    .Attr("dilations: list(int) = [1, 1, 1, 1]")
    .SetShapeFn(shape_inference::Conv2DShapeWithExplicitPadding);

namespace {

// allocate_output / allocate_temp of the TensorFlow context behind the shell's allocator interface.
class TfContext : public axconv::OpContext {
public:
    explicit TfContext(OpKernelContext *ctx) : m_ctx(ctx) {}
    float *allocate_output(const std::vector<int64_t> &shape) override
    {
        TensorShape s;
        for (int64_t d : shape)
            s.AddDim(d);
        Tensor *out = nullptr;
        m_status = m_ctx->allocate_output(0, s, &out);
        return m_status.ok() ? out->flat<float>().data() : nullptr;
    }
    void *allocate_temp(size_t bytes) override
    {
        m_temps.emplace_back();
        m_status = m_ctx->allocate_temp(DT_UINT8, TensorShape({(int64)bytes}), &m_temps.back());
        return m_status.ok() ? m_temps.back().flat<uint8>().data() : nullptr;
    }
    void *stream() override
    {
        // the ROCm stream TensorFlow runs this op on
        return reinterpret_cast<void *>(m_ctx->eigen_gpu_device().stream());
    }
    const Status &status() const { return m_status; }

private:
    OpKernelContext *m_ctx;
    std::vector<Tensor> m_temps; // kept alive until Compute returns; TensorFlow defers the free to the stream
    Status m_status;
};

Status ToTf(const axconv::Status &s)
{
    switch (s.code) {
    case AXC_OK: return Status::OK();
    case AXC_INVALID_ARGUMENT: return errors::InvalidArgument(s.message);
    case AXC_UNIMPLEMENTED: return errors::Unimplemented(s.message);
    default: return errors::Internal(s.message);
    }
}

class ApproxConv2DWithMinMaxVarsOp : public OpKernel {
public:
    explicit ApproxConv2DWithMinMaxVarsOp(OpKernelConstruction *ctx) : OpKernel(ctx)
    {
        axconv::ApproxConv2DAttrs attrs;
        OP_REQUIRES_OK(ctx, ctx->GetAttr("strides", &attrs.strides));
        OP_REQUIRES_OK(ctx, ctx->GetAttr("num_bits", &attrs.num_bits));
        OP_REQUIRES_OK(ctx, ctx->GetAttr("mul_map_file", &attrs.mul_map_file));
        OP_REQUIRES_OK(ctx, ctx->GetAttr("padding", &attrs.padding));
        if (ctx->HasAttr("explicit_paddings")) {
            std::vector<int64> ep;
            OP_REQUIRES_OK(ctx, ctx->GetAttr("explicit_paddings", &ep));
            attrs.explicit_paddings.assign(ep.begin(), ep.end());
        }
        OP_REQUIRES_OK(ctx, ctx->GetAttr("data_format", &attrs.data_format));
        OP_REQUIRES_OK(ctx, ctx->GetAttr("dilations", &attrs.dilations));
        m_op.reset(new axconv::ApproxConv2DOp(attrs));
        OP_REQUIRES_OK(ctx, ToTf(m_op->status()));
    }

    void Compute(OpKernelContext *ctx) override
    {
        const Tensor &input = ctx->input(0);
        const Tensor &filter = ctx->input(1);
        axconv::DeviceTensor in, flt, out;
        in.data = const_cast<float *>(input.flat<float>().data());
        flt.data = const_cast<float *>(filter.flat<float>().data());
        for (int i = 0; i < input.dims(); ++i)
            in.shape.push_back(input.dim_size(i));
        for (int i = 0; i < filter.dims(); ++i)
            flt.shape.push_back(filter.dim_size(i));
        // the four scalars live in host memory (HostMemory below), as in approx_nn_conv_ops.cpp:691-694
        const float input_min = ctx->input(2).scalar<float>()();
        const float input_max = ctx->input(3).scalar<float>()();
        const float filter_min = ctx->input(4).scalar<float>()();
        const float filter_max = ctx->input(5).scalar<float>()();
        TfContext shell_ctx(ctx);
        const axconv::Status s = m_op->Compute(&shell_ctx, in, flt, input_min, input_max, filter_min, filter_max, &out);
        OP_REQUIRES_OK(ctx, shell_ctx.status());
        OP_REQUIRES_OK(ctx, ToTf(s));
    }

private:
    std::unique_ptr<axconv::ApproxConv2DOp> m_op;
};

REGISTER_KERNEL_BUILDER(Name("ApproxConv2DWithMinMaxVars")
                            .Device(DEVICE_GPU)
                            .TypeConstraint<float>("T")
                            .HostMemory("input_min")
                            .HostMemory("input_max")
                            .HostMemory("filter_min")
                            .HostMemory("filter_max"),
                        ApproxConv2DWithMinMaxVarsOp);

} // namespace
} // namespace tensorflow

#endif // AXCONV_WITH_TENSORFLOW
