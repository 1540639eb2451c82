/*
 * axconv -- C ABI of the MI355X (gfx950) implementation of TFApprox's
 * ApproxConv2DWithMinMaxVars hot path.
 *
 * Plain C: opaque handles, raw device pointers, sizes, int status codes.  No C++ or
 * framework types cross this boundary.  All tensor pointers are DEVICE pointers
 * (hipMalloc'd or owned by any framework that hands out HIP device memory); the four
 * min/max values are host scalars passed by value, as the reference pins them to host
 * memory (tf2/src/approx_nn_conv_ops.cpp:691-694).  `stream` is a hipStream_t passed as
 * void* (NULL = the default stream).  Launch calls are asynchronous on that stream, allocate
 * nothing and keep no state between calls (tile plans are cached by layer shape, which callers cannot observe):
 * the caller owns the workspace.  A table belongs to the device that was current at its creation; launches with
 * another device current are refused.
 *
 * Each declaration cites the reference interface (paths under tf2/src/) it replaces.
 */
#ifndef AXCONV_H
#define AXCONV_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status codes; the reference reports the same conditions through tensorflow::Status
 * (errors::InvalidArgument / errors::Unimplemented, approx_nn_conv_ops.cpp:120,162,224,231,287-303). */
enum {
    AXC_OK = 0,
    AXC_INVALID_ARGUMENT = 1,
    AXC_UNIMPLEMENTED = 2,
    AXC_RUNTIME_ERROR = 3 /* a HIP call failed; the reference ignores CUDA return codes */
};

enum { AXC_PAD_VALID = 0, AXC_PAD_SAME = 1, AXC_PAD_EXPLICIT = 2 };
enum { AXC_FORMAT_NHWC = 0, AXC_FORMAT_NCHW = 1 };

/* Attributes and shapes of one op invocation: the op's attrs (approx_nn_ops.cpp:46-53,
 * parsed at approx_nn_conv_ops.cpp:254-309) plus the input/filter shapes read in Compute
 * (approx_nn_conv_ops.cpp:311-404).  strides/dilations are given in the data_format's own
 * order, four entries each, exactly as the attrs hold them. */
typedef struct axc_conv2d_desc {
    int64_t input_shape[4];   /* in data_format order (NHWC: N,H,W,C) */
    int64_t filter_shape[4];  /* HWIO: rows, cols, in_depth, out_depth */
    int32_t strides[4];
    int32_t dilations[4];
    int32_t padding;          /* AXC_PAD_* */
    int32_t data_format;      /* AXC_FORMAT_* */
    int32_t num_bits;         /* only 8 is supported (approx_ops_types.h:218) */
    int64_t explicit_paddings[8];
} axc_conv2d_desc;

/* Mirrors tensorflow::ApproxConv2DDimensions (approx_nn_conv_ops.h:56-79). */
typedef struct axc_conv2d_dims {
    int32_t batch, input_rows, input_cols, in_depth;
    int32_t filter_rows, filter_cols, patch_depth, out_depth;
    int32_t stride_rows, stride_cols, dilation_rows, dilation_cols;
    int64_t out_rows, out_cols;
    int64_t pad_rows_before, pad_rows_after, pad_cols_before, pad_cols_after;
} axc_conv2d_dims;

/* Mirrors BaseTableApproxOpType_t::OpQuantProps_t (approx_ops_types.h:79-97). */
typedef struct axc_quant_props {
    float input_scale, input_inv_scale, input_offset;
    float filter_scale, filter_inv_scale, filter_offset;
    float s1xs2, m1, m2, m1xm2;
    int32_t input_zero_code; /* code of the value 0.0f: what padding taps look up */
} axc_quant_props;

/* Device-resident truth table.  Immutable after creation; may be shared by concurrent calls. */
typedef struct axc_table axc_table;

const char *axc_status_string(int status);
/* Message of the last failing call on this thread (the reference's error text where it has one). */
const char *axc_last_error(void);

/* Replaces the GPU table upload, TableApproxOpType_t<GpuDevice> ctor (cuda/approx_ops_types.cu:20-42):
 * host_table is uint16[65536], index (input_code << 8) | filter_code (approx_nn_conv_kernels.cpp:245). */
int axc_table_create(const uint16_t *host_table, axc_table **out);
/* Replaces BaseTableApproxOpType_t ctor + LoadLookupTable (approx_ops_types.h:99-122,205-216):
 * empty or NULL filename -> exact products; short read -> AXC_INVALID_ARGUMENT
 * "ApproxTF: Couldn't read the lookup table!"; num_bits != 8 -> AXC_INVALID_ARGUMENT. */
int axc_table_create_from_file(const char *filename, int num_bits, axc_table **out);
/* Replaces ~TableApproxOpType_t<GpuDevice> (cuda/approx_ops_types.cu:44-49). */
int axc_table_destroy(axc_table *table);

/* Replaces BaseTableApproxOpType_t::Update / UpdateVarQuantProps / Nudge
 * (approx_ops_types.h:29-49,135-197), stateless. */
int axc_quant_props_compute(float input_min, float input_max, float filter_min, float filter_max,
                            axc_quant_props *out);

/* Replaces InitApproxConv2DParameters + ComputeApproxConv2DDimensions
 * (approx_nn_conv_ops.cpp:254-404), including their argument checks. */
int axc_conv2d_geometry(const axc_conv2d_desc *desc, axc_conv2d_dims *dims);

/* Scratch the launch calls below need for this desc (replaces the three allocate_temp calls at
 * approx_nn_conv_ops.cpp:590-613). */
int axc_conv2d_workspace_bytes(const axc_conv2d_desc *desc, size_t *bytes);

/* The reference's Keras layer around the op, FakeApproxConv2D.call
 * (tf2/python/keras/layers/fake_approx_convolutional.py:223-261), as one call that never leaves the device:
 * min / max of the input batch and of the kernel (reduce_min / reduce_max, :233-241), fake quantization of both
 * with them (fake_quant_with_min_max_vars, :235,242: here fused into the kernels that read the tensors), the op,
 * then bias_add and the activation of Conv.call (:261).  bias may be null; activation is AXC_ACT_*.
 * Workspace: axc_conv2d_workspace_bytes.  axc_fake_approx_depthwise_conv2d is the same layer call around the
 * depthwise variant (filter [rows, cols, C, 1], bias one value per channel; workspace:
 * axc_depthwise_conv2d_workspace_bytes): the Keras layer wraps whichever convolution it is given. */
enum { AXC_ACT_NONE = 0, AXC_ACT_RELU = 1 };
int axc_fake_approx_conv2d(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                           const float *filter, const float *bias, int activation, float *output, void *workspace,
                           size_t workspace_bytes, void *stream);
int axc_fake_approx_depthwise_conv2d(const axc_table *table, const axc_conv2d_desc *desc, const float *input,
                                     const float *filter, const float *bias, int activation, float *output,
                                     void *workspace, size_t workspace_bytes, void *stream);

/* The tf1 integer op AxConv2D (tf1/axqconv/axqconv.cc:66-94 registration, :113-278 ReferenceAxConvFunctor,
 * :286-441 AxQuantizedConv2DOp): quint8 input and filter codes in, qint32 out,
 *   out = sum over the patch of  T[a][b] - a*offset_filter - b*offset_input + offset_input*offset_filter,
 * taps outside the image reading a = offset_input; padding origin by that functor's own rule (:153-163).
 * offset_* are what the reference derives with FloatToQuantizedUnclamped(0, min, max) (TensorFlow, third party).
 * Strides must be equal, dilations 1.  Workspace: axc_conv2d_workspace_bytes. */
int axc_axconv2d_quint8(const axc_table *table, const axc_conv2d_desc *desc, const uint8_t *input,
                        const uint8_t *filter, int32_t offset_input, int32_t offset_filter, int32_t *output,
                        void *workspace, size_t workspace_bytes, void *stream);

/* AxTune of ApproximateSelector::init (tf1/axqconv/approximate_selector.h:52-85), host side: tuned[i][w] =
 * table[i][w2(w)] with w2 the weight whose column is closest to exact multiplication by w.  table and tuned are
 * uint16[65536] in host memory and may be the same buffer. */
int axc_table_tune_weights(const uint16_t *table, uint16_t *tuned);

/* The two TensorFlow quantization helpers AxQuantizedConv2DOp::Compute calls around the functor
 * (tf1/axqconv/axqconv.cc:364-367,427-431), as the reference's copy of them defines them
 * (tf1/axqconv/quantization_utils.h:49-64,114-140): the quint8 code of 0.0f for a float range (offset_input /
 * offset_filter of axc_axconv2d_quint8), and the float range the qint32 output stands for. */
int axc_quint8_zero_point(float range_min, float range_max, int32_t *zero_point);
int axc_qint32_range_for_multiplication(float min_a, float max_a, float min_b, float max_b, float *min_c,
                                        float *max_c);

/* How the dense kernel would cut this layer on the current device (for tools and tests; the reference has no
 * counterpart, its launch shapes are fixed in cuda/approx_nn_conv_kernels.cu:296-627):
 * plan = { columns per tile (16/32/64), rows per tile, row tiles, column tiles, K splits, workgroups,
 *          fills of 64 filter entries per K split, how the layer runs given a workspace of the size
 *          axc_conv2d_workspace_bytes reports: 0 = table rows expanded inside every tile, 1 = out of pre-expanded
 *          rows, 2 = out of pre-expanded rows by the kernel whose wavefronts do not meet at a barrier between fills }. */
int axc_conv2d_tile_plan(const axc_conv2d_desc *desc, int32_t plan[8]);
/* Pins the tile width the planner uses (16, 32 or 64 columns; 0 = its own choice, the default), process-wide, for
 * tests and timing of the wider-tile kernel variants.  The environment variable AXC_TILE_COLUMNS gives the initial
 * value and is read once, when the library is loaded.  Like axc_set_preexpand it is process-wide; a workspace query and
 * the launch it is for must see the same value. */
int axc_set_tile_columns(int columns);
/* Layers with many output pixels per filter element (16-column tiles, an even number of channel quads, whole pairs
 * of fills per K split where K is split, at most 2 GiB of rows) run out of pre-expanded rows: the table rows of
 * every filter element are laid out in the workspace once per call instead of inside every tile.  mode 0 = the planner decides (the default), 1 = every
 * layer that can run that way does, -1 = none does; process-wide, for tests and timing, initial value from the
 * environment variable AXC_PREEXPAND (read once, when the library is loaded).  Results do not depend on it.  The
 * workspace query counts the rows; a launch whose workspace lacks room for them runs without them, with the tile
 * plan of the kernel that expands inside its tiles when the workspace holds what that plan needs.  No counterpart
 * in the reference. */
int axc_set_preexpand(int mode);
/* The wavefronts of the kernel that plan code 2 stands for wait for each other by polling counters, every wait a bounded
 * number of polls (the default, 2^20 of ~150 cycles each, is far beyond any legitimate wait).  A wait that runs out ends
 * the launch early - every wavefront leaves the kernel, nothing hangs - and the NEXT launch call on that GPU returns
 * AXC_RUNTIME_ERROR once instead of launching: the earlier launch's output is incomplete.  This sets the number of
 * polls, process-wide; 0 makes every wait that is not satisfied at once give up (tests of the report).  No counterpart
 * in the reference. */
int axc_set_wait_limit(uint32_t polls);
int axc_depthwise_conv2d_workspace_bytes(const axc_conv2d_desc *desc, size_t *bytes);

/* The op: replaces ApproxConv2DOp::Compute -> LaunchApproxConv2DOp<GPUDevice> and the kernels it
 * launches (approx_nn_conv_ops.cpp:420-460,510-664; cuda/approx_nn_conv_kernels.cu:296-627).
 * input: float NHWC, filter: float HWIO, output: float NHWC [N,out_rows,out_cols,out_depth]. */
int axc_conv2d_minmax(const axc_table *table, const axc_conv2d_desc *desc,
                      const float *input, const float *filter,
                      float input_min, float input_max, float filter_min, float filter_max,
                      float *output, void *workspace, size_t workspace_bytes, void *stream);

/* The op followed by the tail of the Keras layer's call, bias_add and the activation of Conv.call
 * (tf2/python/keras/layers/fake_approx_convolutional.py:261), fused into the op's store, for callers that hold the
 * ranges themselves (fake-quantization variables fixed after training or calibration) and so have no use for
 * the per-batch min / max pass of axc_fake_approx_conv2d.  Unlike that entry it does not fake-quantize: like the op,
 * it expects tensors that already lie on their grids.  bias may be null (out_depth floats otherwise; in_depth for
 * the depthwise variant); activation is AXC_ACT_*.  Results equal axc_conv2d_minmax / axc_depthwise_conv2d_minmax
 * followed by `+ bias` and `max(x, 0)`, each rounded on its own. */
int axc_conv2d_minmax_bias_act(const axc_table *table, const axc_conv2d_desc *desc,
                               const float *input, const float *filter,
                               float input_min, float input_max, float filter_min, float filter_max,
                               const float *bias, int activation,
                               float *output, void *workspace, size_t workspace_bytes, void *stream);
int axc_depthwise_conv2d_minmax_bias_act(const axc_table *table, const axc_conv2d_desc *desc,
                                         const float *input, const float *filter,
                                         float input_min, float input_max, float filter_min, float filter_max,
                                         const float *bias, int activation,
                                         float *output, void *workspace, size_t workspace_bytes, void *stream);

/* axc_conv2d_minmax for callers that cannot allocate or own a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The workspace is a fixed array of
 * axc_conv2d_static_workspace_limit() bytes (32 MiB) inside the library's device image, one copy per GPU, held
 * until the process ends; the call itself allocates and frees nothing.  Layers whose
 * axc_conv2d_workspace_bytes exceeds the limit are refused with AXC_INVALID_ARGUMENT.  All calls on one GPU
 * share the array: calls that overlap on one GPU (two streams, two threads) race; issue them on one stream.
 * Results are identical to axc_conv2d_minmax. */
int axc_conv2d_static_workspace_limit(size_t *bytes);
int axc_conv2d_minmax_static(const axc_table *table, const axc_conv2d_desc *desc,
                             const float *input, const float *filter,
                             float input_min, float input_max, float filter_min, float filter_max,
                             float *output, void *stream);

/* Depthwise variant (filter [rows, cols, C, 1]).  The reference has none: its CPU launcher rejects
 * in_depth != filter in_depth (approx_nn_conv_ops.cpp:229-232).  Defined as the dense op applied to
 * every channel on its own with the tensor-wide min/max. */
int axc_depthwise_conv2d_minmax(const axc_table *table, const axc_conv2d_desc *desc,
                                const float *input, const float *filter,
                                float input_min, float input_max, float filter_min, float filter_max,
                                float *output, void *workspace, size_t workspace_bytes, void *stream);

/* ---- parity entry points (stages of the op, exposed so each can be checked bit for bit) ---- */

/* The quantize expression (approx_nn_conv_kernels.cpp:193,197,243,293) on n floats:
 * codes[i] = uint8((v[i] - offset) * inv_scale + 0.5f), offset/inv_scale from (min, max). */
int axc_quantize(const float *values, int64_t n, float min, float max, uint8_t *codes, void *stream);

/* Same as axc_conv2d_minmax / axc_depthwise_conv2d_minmax but stores the int32 sums of table
 * entries (the `total` of approx_nn_conv_kernels.cpp:235-247 before the epilogue) instead of floats. */
int axc_conv2d_minmax_acc_i32(const axc_table *table, const axc_conv2d_desc *desc,
                              const float *input, const float *filter,
                              float input_min, float input_max, float filter_min, float filter_max,
                              int32_t *acc, void *workspace, size_t workspace_bytes, void *stream);
int axc_depthwise_conv2d_minmax_acc_i32(const axc_table *table, const axc_conv2d_desc *desc,
                                        const float *input, const float *filter,
                                        float input_min, float input_max, float filter_min, float filter_max,
                                        int32_t *acc, void *workspace, size_t workspace_bytes, void *stream);

/* LUT-GEMM on caller-supplied codes: input_codes uint8 NHWC, filter_codes uint8 HWIO,
 * input_zero_code is what out-of-bounds taps look up.  acc: int32 [N,out_rows,out_cols,out_depth]. */
int axc_conv2d_codes_acc_i32(const axc_table *table, const axc_conv2d_desc *desc,
                             const uint8_t *input_codes, const uint8_t *filter_codes, int input_zero_code,
                             int32_t *acc, void *workspace, size_t workspace_bytes, void *stream);

/* ---- measurement -------------------------------------------------------------------------- */

/* Per-kernel timing with HIP events recorded on the launch stream.  While enabled, every kernel the
 * launch calls enqueue is bracketed by two events; axc_profile_read synchronizes them and returns the
 * accumulated milliseconds and launch count per kernel name since the last reset. */
int axc_profile_enable(int enable);
int axc_profile_reset(void);
int axc_profile_read(int index, char *name, size_t name_bytes, double *total_ms, int64_t *launches);

/* Conflict-free ds_read_u16 gather rate of this GPU (lookups per second over all CUs): the measured
 * ceiling of the LDS-lookup roofline. */
int axc_lds_gather_peak(double *lookups_per_second, void *stream);

/* Conflict-free streaming ds_read_b128 rate of this GPU (bytes per second over all CUs): the ceiling of the
 * LDS read port for 16-byte accesses, the width the LUT-GEMM reads its expanded table rows with.  A lookup
 * moves at least its 2-byte table entry through that port. */
int axc_lds_read_peak(double *bytes_per_second, void *stream);

/* Issue rate of the LUT-GEMM's accumulate instructions on this GPU, in lane operations per second over all CUs,
 * measured with a kernel that contains nothing else, in the LUT-GEMM's occupancy (two wavefronts per SIMD).
 * The LUT-GEMM spends axc_dense_accumulate_ops_per_lookup() of these operations per table entry, so
 * rate / ops_per_lookup is the ceiling the vector ALUs put on lookups per second. */
int axc_valu_issue_peak(double *lane_ops_per_second, void *stream);
int axc_dense_accumulate_ops_per_lookup(double *ops);
/* Rate, in table entries per second over all CUs, of a kernel that contains nothing but the instruction mix of a
 * LUT-GEMM lookup - address (v_perm_b32), 16-byte LDS read of eight entries, their six accumulate instructions - in
 * the LUT-GEMM's occupancy.  The LDS read port and the vector ALUs each allow more on their own; a pair of wavefronts
 * that has to issue both kinds gets this.  No counterpart in the reference (measurement only). */
int axc_lookup_mix_peak(double *lookups_per_second, void *stream);

/* Properties of the current device the planner uses. */
int axc_device_info(int *compute_units, int *lds_bytes_per_workgroup, int *clock_khz);

#ifdef __cplusplus
}
#endif
#endif /* AXCONV_H */
