// See approx_conv2d_op.h.
#include "approx_conv2d_op.h"

#include <algorithm>

namespace axconv {

static Status FromLibrary(int code)
{
    if (code == AXC_OK)
        return Status::OK();
    const char *detail = axc_last_error();
    return Status{code, detail && *detail ? detail : axc_status_string(code)};
}

Status InitApproxConv2DParameters(const ApproxConv2DAttrs &attrs, ApproxConv2DParameters *params)
{
    params->dilations = attrs.dilations;
    params->strides = attrs.strides;
    params->explicitPaddings = attrs.explicit_paddings;

    if (attrs.padding == "SAME")
        params->padding = AXC_PAD_SAME;
    else if (attrs.padding == "VALID")
        params->padding = AXC_PAD_VALID;
    else if (attrs.padding == "EXPLICIT")
        params->padding = AXC_PAD_EXPLICIT;
    else
        return Status::InvalidArgument("Unknown padding type: " + attrs.padding);

    if (attrs.data_format == "NHWC")
        params->dataFormat = AXC_FORMAT_NHWC;
    else if (attrs.data_format == "NCHW")
        params->dataFormat = AXC_FORMAT_NCHW;
    else
        return Status::InvalidArgument("Invalid data format");

    if (params->dilations.size() != 4)
        return Status::InvalidArgument("Sliding window dilations field must specify 4 dimensions");
    if (params->strides.size() != 4)
        return Status::InvalidArgument("Sliding window strides must specify 4 dimensions");

    const bool nhwc = params->dataFormat == AXC_FORMAT_NHWC;
    const int iN = 0, iC = nhwc ? 3 : 1, iH = nhwc ? 1 : 2, iW = nhwc ? 2 : 3;
    if (params->strides[iN] != 1 || params->strides[iC] != 1)
        return Status::InvalidArgument(
            "Current implementation does not yet support strides in the batch and depth dimensions.");
    if (params->strides[iH] <= 0 || params->strides[iW] <= 0)
        return Status::InvalidArgument("Row and column strides should be larger than 0.");
    if (params->dilations[iN] != 1 || params->dilations[iC] != 1)
        return Status::InvalidArgument(
            "Current implementation does not yet support dilations in the batch and depth dimensions.");
    if (params->dilations[iH] <= 0 || params->dilations[iW] <= 0)
        return Status::InvalidArgument("Dilated rates should be larger than 0.");

    // CheckValidPadding: explicit_paddings must be empty unless padding is EXPLICIT, and then hold 8 values
    if (params->padding == AXC_PAD_EXPLICIT) {
        if (params->explicitPaddings.size() != 8)
            return Status::InvalidArgument("explicit_paddings attribute must contain 8 values, but got: " +
                                           std::to_string(params->explicitPaddings.size()));
    } else if (!params->explicitPaddings.empty()) {
        return Status::InvalidArgument("explicit_paddings attribute must be empty if the padding attribute is not EXPLICIT");
    }
    return Status::OK();
}

void ApproxConv2DOp::Init(const ApproxConv2DAttrs &attrs, const uint16_t *host_table)
{
    m_numBits = attrs.num_bits;
    m_depthwise = attrs.depthwise;
    m_status = InitApproxConv2DParameters(attrs, &m_params);
    if (!m_status.ok())
        return;
    if (host_table)
        m_status = FromLibrary(axc_table_create(host_table, &m_table));
    else
        m_status = FromLibrary(axc_table_create_from_file(attrs.mul_map_file.c_str(), attrs.num_bits, &m_table));
}

ApproxConv2DOp::ApproxConv2DOp(const ApproxConv2DAttrs &attrs) { Init(attrs, nullptr); }

ApproxConv2DOp::ApproxConv2DOp(const ApproxConv2DAttrs &attrs, const uint16_t *host_table) { Init(attrs, host_table); }

ApproxConv2DOp::~ApproxConv2DOp()
{
    if (m_table)
        axc_table_destroy(m_table);
}

Status ApproxConv2DOp::Compute(OpContext *ctx, const DeviceTensor &input, const DeviceTensor &filter,
                               float input_min, float input_max, float filter_min, float filter_max,
                               DeviceTensor *output)
{
    if (!m_status.ok())
        return m_status;
    if (input.shape.size() != 4)
        return Status::InvalidArgument("input must be 4-dimensional");
    if (filter.shape.size() != 4)
        return Status::InvalidArgument("filter must be 4-dimensional");

    axc_conv2d_desc desc = {};
    for (int i = 0; i < 4; ++i) {
        desc.input_shape[i] = input.shape[i];
        desc.filter_shape[i] = filter.shape[i];
        desc.strides[i] = m_params.strides[i];
        desc.dilations[i] = m_params.dilations[i];
    }
    desc.padding = m_params.padding;
    desc.data_format = m_params.dataFormat;
    desc.num_bits = m_numBits;
    for (size_t i = 0; i < m_params.explicitPaddings.size() && i < 8; ++i)
        desc.explicit_paddings[i] = m_params.explicitPaddings[i];

    // ComputeApproxConv2DDimensions (approx_nn_conv_ops.cpp:311-404): done by the library, which the
    // workspace query runs as well.
    axc_conv2d_dims dims;
    int rc;
    if (m_depthwise) {
        axc_conv2d_desc probe = desc;             // geometry of the dense op with one input channel per group
        probe.input_shape[3] = 1;
        probe.filter_shape[2] = 1;
        rc = axc_conv2d_geometry(&probe, &dims);
        if (rc == AXC_OK && (filter.shape[3] != 1 || filter.shape[2] != input.shape[3]))
            return Status::InvalidArgument("depthwise filter must be [rows, cols, in_depth, 1]");
        dims.out_depth = (int32_t)input.shape[3];
    } else {
        rc = axc_conv2d_geometry(&desc, &dims);
    }
    if (rc != AXC_OK)
        return FromLibrary(rc);

    output->shape = {dims.batch, dims.out_rows, dims.out_cols, dims.out_depth};
    output->data = ctx->allocate_output(output->shape);
    if (output->num_elements() == 0)
        return Status::OK();
    if (!output->data)
        return Status{AXC_RUNTIME_ERROR, "allocate_output failed"};

    size_t ws_bytes = 0;
    rc = m_depthwise ? axc_depthwise_conv2d_workspace_bytes(&desc, &ws_bytes) : axc_conv2d_workspace_bytes(&desc, &ws_bytes);
    if (rc != AXC_OK)
        return FromLibrary(rc);
    void *ws = ws_bytes ? ctx->allocate_temp(ws_bytes) : nullptr;
    if (ws_bytes && !ws)
        return Status{AXC_RUNTIME_ERROR, "allocate_temp failed"};

    rc = m_depthwise
             ? axc_depthwise_conv2d_minmax(m_table, &desc, input.data, filter.data, input_min, input_max, filter_min,
                                           filter_max, output->data, ws, ws_bytes, ctx->stream())
             : axc_conv2d_minmax(m_table, &desc, input.data, filter.data, input_min, input_max, filter_min,
                                 filter_max, output->data, ws, ws_bytes, ctx->stream());
    return FromLibrary(rc);
}

} // namespace axconv
