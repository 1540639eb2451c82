// Internal declarations shared by the HIP translation units of libaxconv_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <map>
#include <mutex>
#include <utility>
#include <stdint.h>
#include <stddef.h>

#include "axconv.h"

namespace axc {

constexpr int kTableBytes = 131072;            // 256 x 256 uint16, weight-code major
constexpr int kTableRows = 257;                // row 256 is all zeros: the row of the null weight
constexpr int kTableAllocBytes = kTableRows * 512;
constexpr int kExpandBytes = 32768;            // one expanded-row buffer: 256 activation rows x 64 slots x uint16
constexpr int kDenseLdsBytes = 4 * kExpandBytes; // dense kernel: 2 buffers of expanded rows + 2 of staged table rows
constexpr int kDenseThreads = 512;             // dense kernel: 8 wavefronts x 256 VGPRs, one workgroup per CU
constexpr int kDenseWaves = kDenseThreads / 64;
constexpr int kDenseParkBytes = 16 * 4 * kDenseThreads; // per-thread pixel geometry parked behind the buffers
constexpr int kPxMaxTileWaveRows = 8 * kDenseWaves - 1;  // lutgemm_pxf_kernel: the last wavefront's last pixel slot holds
                                                         // the kernel's wait counters instead of geometry
constexpr int kBlockThreads = 1024;            // depthwise kernel / LDS probe: 16 wavefronts per CU
constexpr int kWaves = kBlockThreads / 64;
// Accumulate instruction mix of the dense kernel's generated phase body (gen_lookup_asm.py emits the same):
// 0 = one VALU add per table entry (v_add_u32 of a whole dword + v_add_u32_sdwa of its high half);
// 1 = three per four entries (two dwords of one column pair folded by one v_add3_u32, the high halves by SDWA adds).
constexpr int kDenseAccumulateMix = 1;   // what the 16- and 32-column tiles run (64-column tiles: mix 0)
constexpr uint16_t kNullWeight = 256;          // slot that contributes nothing (padding channel / column)

// Geometry of one dense layer after validation.
struct ConvGeom {
    int N, H, W, C;        // input NHWC
    int KH, KW, Co;        // filter HWIO (in depth == C)
    int OH, OW;
    int sh, sw, dh, dw, ph, pw;
    int C4;                // ceil(C / 4): channel quads in the quantized activation layout
    int64_t M;             // N * OH * OW
    int K;                 // KH * KW * C
};

// How the dense LUT-GEMM is cut into workgroup tiles.
struct DensePlan {
    int nt;                // columns per tile: 16, 32 or 64
    int rows_per_tile;     // multiple of 64, <= 1024 * (64 / nt)
    int n_row_tiles, n_col_tiles;
    int fills;             // expanded-row refills over the whole K: KH*KW * C4 * (4 / (64/nt))
    int k_splits;          // tiles along K: each computes fills_per_split fills into its own int32 partial sums
    int fills_per_split;
    int grid;
    int px;                // 1: the layer suits the kernel that reads pre-expanded rows (lutgemm_px_kernel.hip)
    float cost;            // what the planner's model expects of the LUT-GEMM launches, in cycles
};

// Quantization of one tensor as the pre-pass kernels see it.
struct TensorQuant {
    float offset;       // nudged minimum
    float inv_scale;
    float scale;
    float nudged_max;
    uint32_t fq;        // 1: snap every value to the 8-bit grid first (the Keras layer's fake quantization)
    uint32_t zp4;       // row-permuted code of 0.0f, replicated in all four bytes (input tensor only)
};

// Everything the kernels need to know about a layer's quantization.  The op entry points pass it by value
// (min/max are host scalars there); the layer entry point computes it on the device from the tensors' own
// min/max, so kernels take both a value and a device pointer and use the pointer when it is not null.
struct LayerQuant {
    TensorQuant in, flt;
    float s1xs2, m1, m2, k_m1xm2;
};

// fake_quant_with_min_max_vars on one value (clamp to the nudged range, round half up to the grid), in the
// float32 operations of TensorFlow's functor; identity unless q.fq.
__device__ inline float fake_quant_value(float v, const TensorQuant &q)
{
    if (!q.fq)
        return v;
    if (q.scale == 0.0f)
        return 0.0f;                       // min == max == 0: the whole tensor quantizes to 0
    const float c = fmaxf(fminf(v, q.nudged_max), q.offset);
    const float t = floorf(__fadd_rn(__fmul_rn(__fsub_rn(c, q.offset), q.inv_scale), 0.5f));
    return __fadd_rn(__fmul_rn(t, q.scale), q.offset);
}

struct DenseParams {
    ConvGeom g;
    DensePlan plan;
    const uint32_t *xq;     // [N][H][C4][W] dwords of 4 row-permuted activation codes, then one more
                            // [C4][W] row holding the zero-point code (read by taps outside the image)
    const float *psum;      // [M] sum of the raw input over each output pixel's patch (float epilogue only)
    const uint16_t *wq;     // [n_col_tiles][fills][64] packed filter codes (kNullWeight = none)
    const float *fsum;      // [Co] sum over (h, w, c) of the raw filter
    const uint16_t *tableT; // [257 filter code (256 = null)][256 input code]
    float *out_f;
    int32_t *out_i;         // with k_splits > 1: [k_splits][M][Co] partial sums, reduced by launch_splitk_epilogue
    float s1xs2, m1, m2, k_m1xm2; // epilogue constants; k_m1xm2 = float(K) * m1xM2
    uint32_t zp4;           // row-permuted zero code replicated in all four bytes
    uint32_t xq_bytes, wq_bytes; // sizes of the two streams (buffer-descriptor bounds)
    int step_n, step_oh, step_ow; // 64 * kDenseWaves / 2 output pixels (the distance between a lane's pixels) as
                                  // images, output rows and output columns
    const LayerQuant *lq_dev;    // not null: epilogue constants come from here instead of the four floats above
    const float *bias;           // not null: added to every output column after the epilogue
    int relu;                    // 1: max(x, 0) last
    int stagger_sleeps;          // s_sleep(127) periods by which group g of the workgroups starts late, times g (0: none)
    int stagger_groups;          // g = 0 .. stagger_groups - 1 in turn (2: every second group, the only form lutgemm_expand has)
    const uint16_t *px_rows;     // pre-expanded rows [n_col_tiles][fills / 2][256][128] (lutgemm_px_kernel only)
    uint32_t px_bytes;
    // Addressing of xq.  Usual layout: dwords of four channels, [N][H][C4][W].  Flat layout (channel counts that are
    // no multiple of four, see prepare_dense): bytes, [N][H][row], a row = the pixels' channels one after the other
    // with the horizontal padding written out; g then describes a filter of KH taps whose "channels" are the
    // KW * C bytes a filter row covers.
    int row_step;                // between input rows, in address units
    int addr_unit;               // bytes per address unit: 4 (dwords) or 1 (flat)
    uint32_t quad_bytes;         // between the channel quads that one tap of a pixel reads
    uint32_t zp_tail_bytes;      // size of the zero-point row behind xq
    int flat_col_bytes;          // flat: bytes between horizontally neighbouring output pixels (sw * C); 0 = usual layout
    // lutgemm_pxf_kernel: its wavefronts wait for each other through counters in LDS, every wait a bounded number of
    // polls.  A wait that runs out writes a nonzero word to *wait_error (host-visible memory) and the wavefront leaves
    // the kernel; so do the others at their next wait.
    uint32_t spin_limit;
    uint32_t *wait_error;
};

struct DepthwiseParams {
    int N, H, W, C, KH, KW, OH, OW, sh, sw, dh, dw, ph, pw;
    int64_t M;
    const float *x;         // NHWC raw input
    const uint8_t *wcodes;  // [KH*KW][C] filter codes
    const float *fsum;      // [C]
    const uint16_t *tableT;
    float *out_f;
    int32_t *out_i;
    TensorQuant in_q;            // quantization of the input (op entry points: from the host scalars)
    float s1xs2, m1, m2, k_m1xm2;
    const LayerQuant *lq_dev;    // not null (layer entry point): input quantization and epilogue constants from here
    const float *bias;           // not null: added per channel after the epilogue
    int relu;                    // 1: max(x, 0) last
    int stagger_sleeps;          // s_sleep(127) periods by which every second group of workgroups starts late (0: none)
};

// Row permutation of the expanded table: logical activation code a lives in physical row
// (a >> 2) | ((a & 3) << 6), so that the four codes one lane transposes land in rows of
// alternating bank parity.
__host__ __device__ inline uint32_t phys_row(uint32_t a) { return (a >> 2) | ((a & 3u) << 6); }

// Device-side quantize: three separately rounded fp32 operations, truncation, clamp.
__device__ inline uint32_t quantize_code(float v, float offset, float inv_scale)
{
    float t = __fadd_rn(__fmul_rn(__fsub_rn(v, offset), inv_scale), 0.5f);
    t = t > 0.0f ? t : 0.0f;          // also maps NaN to 0
    t = t < 255.0f ? t : 255.0f;      // truncation of [255,256) is 255 as well
    return (uint32_t)t;
}

// Function attributes belong to a (kernel, device) pair and never change here: they are set on first use instead
// of before every launch (the runtime calls cost a few microseconds of host time each).
inline hipError_t set_max_dynamic_lds_once(const void *kernel, int bytes, bool require_no_static_lds = false)
{
    static std::mutex mu;
    static std::map<std::pair<const void *, int>, int> done;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return e;
    const std::pair<const void *, int> key(kernel, dev);
    {
        std::lock_guard<std::mutex> lock(mu);
        auto it = done.find(key);
        if (it != done.end() && it->second >= bytes)
            return hipSuccess;
    }
    if (require_no_static_lds) {
        hipFuncAttributes attr;
        e = hipFuncGetAttributes(&attr, kernel);
        if (e != hipSuccess)
            return e;
        if (attr.sharedSizeBytes != 0)
            return hipErrorInvalidConfiguration;
    }
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess)
        return e;
    std::lock_guard<std::mutex> lock(mu);
    done[key] = bytes;
    return hipSuccess;
}

int device_cus();   // compute units of the current device (cached)
int device_lds_bytes();    // LDS one workgroup may take on the current device (cached)
double device_clock_hz();  // shader clock of the current device (cached)

// ---- launchers (each enqueues on `stream`; returns hipError_t of the launch) -----------------
hipError_t launch_quantize_relayout(const float *x, const ConvGeom &g, const TensorQuant &tq, const LayerQuant *lq_dev,
                                    uint32_t *xq, float *chsum, hipStream_t stream);
// With xq_fused / fused given, 1x1 stride-1 layers also get their quantized activations from this pass
// (*fused = true); the caller then skips launch_quantize_relayout.
// The filter pre-pass of the same layer (what launch_filter_pack would do), for a launch that can take it along.
struct FilterJob {
    const float *filter;
    const uint8_t *filter_codes;
    const DensePlan *plan;
    TensorQuant tq;
    uint16_t *wq;
    float *fsum;
    const uint16_t *tableT;   // with px_rows: the transposed table the pre-expanded rows are built from
    uint16_t *px_rows;        // nullptr: the layer does not run out of pre-expanded rows
};
// xq_fused / fused: the launch may also quantize the input into xq (then *fused is set);
// filter_job / filter_done: it may also do the filter pre-pass (then *filter_done is set), and with it build the
// pre-expanded rows that filter_job names (then *px_done is set).
hipError_t launch_patch_sums(const float *x, const ConvGeom &g, const TensorQuant &tq, const LayerQuant *lq_dev,
                             float *psum, hipStream_t stream, uint32_t *xq_fused = nullptr, bool *fused = nullptr,
                             const FilterJob *filter_job = nullptr, bool *filter_done = nullptr,
                             int flat_row_bytes = 0,   // > 0: a fused xq is written in the flat layout
                             bool *px_done = nullptr);
hipError_t launch_layer_quant(const float *input, int64_t n_input, const float *filter, int64_t n_filter, int K,
                              float *partials, LayerQuant *lq_dev, hipStream_t stream);
constexpr int kMinMaxBlocks = 2048;   // partial (min, max) pairs per tensor in launch_layer_quant's scratch
// out[n][oh][ow][:] = in[n][oh * sh][ow * sw][:] for tensors of element_bytes-wide elements (C per pixel)
hipError_t launch_subsample(const void *in, int element_bytes, int N, int H, int W, int C, int sh, int sw, int OH, int OW,
                            void *out, hipStream_t stream);
hipError_t launch_codes_relayout(const uint8_t *codes, const ConvGeom &g, uint32_t zp4, uint32_t *xq,
                                 hipStream_t stream);
// Flat layout of xq: rows of row_bytes bytes, pad_left pixels of the zero-point code, the W pixels' codes, zero-point
// codes up to the end of the row; one more row of zero-point codes behind the last image.  From floats (x) or codes.
hipError_t launch_quantize_flat_rows(const float *x, const uint8_t *codes, const ConvGeom &g, int pad_left,
                                     int row_bytes, const TensorQuant &tq, const LayerQuant *lq_dev, uint8_t *xq,
                                     hipStream_t stream);
// tableT / px_rows / px_done: the launch may also build the pre-expanded rows of the layer (then *px_done is set)
hipError_t launch_filter_pack(const float *filter, const uint8_t *filter_codes, const ConvGeom &g,
                              const DensePlan &plan, const TensorQuant &tq, const LayerQuant *lq_dev,
                              uint16_t *wq, float *fsum, hipStream_t stream, const uint16_t *tableT = nullptr,
                              uint16_t *px_rows = nullptr, bool *px_done = nullptr);
hipError_t launch_quantize_flat(const float *v, int64_t n, float offset, float inv_scale, uint8_t *codes,
                                hipStream_t stream);
hipError_t launch_dense(const DenseParams &p, bool out_i32, hipStream_t stream);
// the same layer out of pre-expanded rows: launch_px_expand_rows builds p.px_rows from the packed filter codes
hipError_t launch_px_expand_rows(const uint16_t *wq, const uint16_t *tableT, const DensePlan &plan, uint16_t *rows,
                                 hipStream_t stream);
hipError_t launch_dense_px(const DenseParams &p, bool out_i32, hipStream_t stream);
bool px_free_running(const DensePlan &plan, int taps);   // the plan runs lutgemm_pxf_kernel (no barrier between fills)
hipError_t launch_splitk_epilogue(const DenseParams &p, const int32_t *partials, float *out_f, int32_t *out_i,
                                  hipStream_t stream);
hipError_t launch_axconv_correction(const uint8_t *codes, const uint8_t *fcodes, const ConvGeom &g, int offset_input,
                                    int offset_filter, int32_t *asum, int32_t *bsum, int32_t *out, hipStream_t stream);
hipError_t launch_fill_u32(uint32_t *dst, int64_t n, uint32_t value, hipStream_t stream);
hipError_t launch_depthwise_filter(const float *filter, int taps, int C, const TensorQuant &tq,
                                   const LayerQuant *lq_dev, uint8_t *wcodes, float *fsum, hipStream_t stream);
hipError_t launch_depthwise(const DepthwiseParams &p, bool out_i32, int grid, hipStream_t stream);
hipError_t run_lds_gather_peak(double *lookups_per_second, hipStream_t stream, bool stream_b128);
hipError_t run_valu_issue_peak(double *lane_ops_per_second, int mix, hipStream_t stream);
hipError_t run_lookup_mix_peak(double *lookups_per_second, hipStream_t stream);

} // namespace axc
