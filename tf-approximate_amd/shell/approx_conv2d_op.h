// Host-side shell of the ApproxConv2DWithMinMaxVars op over the C-ABI library (include/axconv.h).
//
// It mirrors the reference's op class for this path, minus TensorFlow:
//   ApproxConv2DParameters / InitApproxConv2DParameters   tf2/src/approx_nn_conv_ops.cpp:254-303
//   ApproxConv2DOp (constructor + Compute)                 tf2/src/approx_nn_conv_ops.cpp:411-468
//   the table member (mul_map_file attr, loaded once)      tf2/src/approx_ops_types.h:99-122,205-216
// Same attribute names, same checks in the same order, same error text.  Tensors are device pointers plus
// shapes; the caller supplies output and scratch memory through an allocator, as TensorFlow's context does
// (allocate_output / allocate_temp, approx_nn_conv_ops.cpp:131-148,433).
#pragma once

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "axconv.h"

namespace axconv {

struct Status {
    int code = AXC_OK;          // AXC_* of axconv.h
    std::string message;
    bool ok() const { return code == AXC_OK; }
    static Status OK() { return Status(); }
    static Status InvalidArgument(const std::string &m) { return Status{AXC_INVALID_ARGUMENT, m}; }
    static Status Unimplemented(const std::string &m) { return Status{AXC_UNIMPLEMENTED, m}; }
};

// A dense float tensor in device memory.
struct DeviceTensor {
    float *data = nullptr;
    std::vector<int64_t> shape;
    int64_t num_elements() const
    {
        int64_t n = 1;
        for (int64_t d : shape)
            n *= d;
        return n;
    }
};

// What the op needs from its host framework.
class OpContext {
public:
    virtual ~OpContext() {}
    // Device memory for the op's output / for scratch that lives until the stream has run the op.
    virtual float *allocate_output(const std::vector<int64_t> &shape) = 0;
    virtual void *allocate_temp(size_t bytes) = 0;
    virtual void *stream() = 0; // hipStream_t
};

// The op's attributes (REGISTER_OP("ApproxConv2DWithMinMaxVars"), tf2/src/approx_nn_ops.cpp:38-54).
struct ApproxConv2DAttrs {
    std::vector<int32_t> strides;
    int num_bits = 8;
    std::string mul_map_file;
    std::string padding;                         // "SAME" | "VALID" | "EXPLICIT"
    std::vector<int64_t> explicit_paddings;
    std::string data_format = "NHWC";
    std::vector<int32_t> dilations = {1, 1, 1, 1};
    bool depthwise = false;                      // filter [kh, kw, C, 1], channel multiplier 1 (not in the reference)
};

struct ApproxConv2DParameters {
    std::vector<int32_t> dilations, strides;
    int padding = AXC_PAD_VALID;
    std::vector<int64_t> explicitPaddings;
    int dataFormat = AXC_FORMAT_NHWC;
};

Status InitApproxConv2DParameters(const ApproxConv2DAttrs &attrs, ApproxConv2DParameters *params);

class ApproxConv2DOp {
public:
    // Construction validates the attributes and loads the table; check status() before Compute().
    explicit ApproxConv2DOp(const ApproxConv2DAttrs &attrs);
    // A table handed over as 65536 uint16 in host memory (index (input_code << 8) | filter_code) instead of a file.
    ApproxConv2DOp(const ApproxConv2DAttrs &attrs, const uint16_t *host_table);
    ~ApproxConv2DOp();
    ApproxConv2DOp(const ApproxConv2DOp &) = delete;
    ApproxConv2DOp &operator=(const ApproxConv2DOp &) = delete;

    const Status &status() const { return m_status; }

    // input NHWC, filter HWIO, min/max as host scalars (the reference reads them from host memory,
    // approx_nn_conv_ops.cpp:691-694).  Enqueues on ctx->stream() and returns; *output is allocated through ctx.
    Status Compute(OpContext *ctx, const DeviceTensor &input, const DeviceTensor &filter, float input_min,
                   float input_max, float filter_min, float filter_max, DeviceTensor *output);

private:
    void Init(const ApproxConv2DAttrs &attrs, const uint16_t *host_table);
    ApproxConv2DParameters m_params;
    int m_numBits = 8;
    bool m_depthwise = false;
    axc_table *m_table = nullptr;
    Status m_status;
};

} // namespace axconv
