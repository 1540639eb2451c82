/*
 * CPU oracle for the ApproxConv2DWithMinMaxVars hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a TensorFlow-free restatement, in plain C,
 * of the arithmetic the reference's CPU kernels perform.  It is the checker the
 * HIP library is compared with; it is never part of the shipped product path.
 * Only tests, the smoke check and the benchmark's cpu_baseline leg may use it.
 *
 * Every function names the reference lines (paths under tf2/src/) it restates.
 *
 * Pinning status (what fixes each function's results independently of this file):
 *   axo_nudge / axo_update_quant_props  closed forms + golden hex floats (tests/test_oracle_quant.py)
 *   axo_quantize                        grid invariant q(nudged_min + i*scale) == i, q(0) == zero point
 *   axo_table_load / axo_table_exact    the reference's 37 .bin tables and its 36 C multiplier models
 *   axo_conv_geometry                   closed forms for SAME/VALID (third-party TF helper): the reference's
 *                                       only test runs one shape (256x256, 8x8, stride 1, SAME)
 *   axo_im2col / axo_gemm_table / axo_gemm_combined / axo_conv2d
 *                                       brute force, integer matmul with the exact table,
 *                                       conv2d(fq(X), fq(F)) by a library routine, direct 7-loop form
 *   axo_axconv2d_tf1                    exact table => integer convolution of (code - offset) by numpy
 *   axo_table_tune_weights              exact table is a fixed point; brute-force argmin in numpy
 *   axo_depthwise_conv2d                no counterpart in the reference (it rejects grouped convolutions);
 *                                       defined here as the dense op applied per channel
 */
#ifndef AXCONV_ORACLE_H
#define AXCONV_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* approx_ops_types.h:79-97 (VarQuantProps_t x2 + OpQuantProps_t), flattened. */
typedef struct {
    float in_scale, in_inv_scale, in_offset;
    float f_scale, f_inv_scale, f_offset;
    float s1xs2, m1, m2, m1xm2;
} axo_quant_props;

enum { AXO_PAD_VALID = 0, AXO_PAD_SAME = 1, AXO_PAD_EXPLICIT = 2 };

enum {
    AXO_OK = 0,
    AXO_INVALID_ARGUMENT = 1,
    AXO_UNIMPLEMENTED = 2
};

typedef struct {
    int batch, in_rows, in_cols, in_depth;
    int filter_rows, filter_cols, patch_depth, out_depth;
    int stride_rows, stride_cols, dilation_rows, dilation_cols;
    int padding; /* AXO_PAD_* */
    /* filled by axo_conv_geometry */
    int64_t out_rows, out_cols, pad_rows_before, pad_rows_after, pad_cols_before, pad_cols_after;
} axo_conv_desc;

/* approx_ops_types.h:29-49 */
void axo_nudge(float min, float max, int quant_min, int quant_max,
               float *nudged_min, float *nudged_max, float *scale);
/* approx_ops_types.h:135-152 */
void axo_update_var_quant_props(float min_value, float max_value,
                                float *scale, float *inv_scale, float *offset);
/* approx_ops_types.h:158-197 */
void axo_update_quant_props(float in_min, float in_max, float f_min, float f_max, axo_quant_props *qp);

/* approx_ops_types.h:112-117 */
void axo_table_exact(uint16_t table[65536]);
/* approx_ops_types.h:205-216; returns AXO_OK or AXO_INVALID_ARGUMENT (short read / missing file) */
int axo_table_load(const char *filename, uint16_t table[65536]);

/* The quantize expression at approx_nn_conv_kernels.cpp:193,197,243,293.  Out-of-range
 * inputs are undefined behaviour in the reference; here they clamp to [0,255]. */
uint8_t axo_quantize(float value, float offset, float inv_scale);
void axo_quantize_array(const float *values, int64_t n, float offset, float inv_scale, uint8_t *codes);

/* approx_nn_conv_ops.cpp:311-404 with TF's GetWindowedOutputSizeVerboseV2 restated. */
int axo_conv_geometry(axo_conv_desc *d);

/* approx_nn_conv_kernels.cpp:260-296 */
void axo_im2col(const axo_quant_props *qp, const float *in,
                int c, int w, int h, int ow, int oh, int kw, int kh, int pw, int ph,
                int sw, int sh, int dw, int dh, int po, int pc,
                uint8_t *out, float *out_coeffs);
/* approx_nn_conv_kernels.cpp:300-306 (summation order: h, w, c ascending per output channel) */
void axo_filter_sums(const float *filter, int kh, int kw, int c, int co, float *sums);
/* approx_nn_conv_kernels.cpp:215-256; acc_i32 (optional, may be NULL) receives the exact integer sums */
void axo_gemm_table(const axo_quant_props *qp, const uint16_t *table,
                    int m, int n, int k, const uint8_t *a, int lda, const float *b, int ldb,
                    const float *a_coeffs, const float *b_coeffs, float *c, int ldc, int32_t *acc_i32);
/* approx_nn_conv_kernels.cpp:167-211 */
void axo_gemm_combined(const axo_quant_props *qp, const uint16_t *table,
                       int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                       float *c, int ldc, int32_t *acc_i32);

/* approx_nn_conv_ops.cpp:70-206 (dispatch + chunking) behind :420-460 (Compute).
 * input NHWC float, filter HWIO float, output NHWC float.  acc_i32 optional. */
int axo_conv2d(const uint16_t *table, axo_conv_desc *d,
               const float *input, const float *filter,
               float in_min, float in_max, float f_min, float f_max,
               float *output, int32_t *acc_i32);

/* approx_nn_conv_ops_ref.cpp:231-317, the reference's second statement of the same formula
 * as a direct 7-deep loop (no dilation).  Used to cross-check axo_conv2d. */
int axo_conv2d_direct(const uint16_t *table, axo_conv_desc *d,
                      const float *input, const float *filter,
                      float in_min, float in_max, float f_min, float f_max, float *output);

/* Same results as axo_conv2d's integer sums, computed with pre-quantized filter codes and
 * int32 accumulation (optionally OpenMP over output pixels).  out = epilogue(float(acc)).
 * Used for parity at sizes where the reference-order loop would take minutes. */
int axo_conv2d_fast(const uint16_t *table, axo_conv_desc *d,
                    const float *input, const float *filter,
                    float in_min, float in_max, float f_min, float f_max,
                    float *output, int32_t *acc_i32, int threads);

/* Depthwise (channel multiplier 1): filter [kh,kw,C,1]; for each channel the dense op on that
 * channel alone, with tensor-wide min/max.  No counterpart in the reference. */
int axo_depthwise_conv2d(const uint16_t *table, axo_conv_desc *d,
                         const float *input, const float *filter,
                         float in_min, float in_max, float f_min, float f_max,
                         float *output, int32_t *acc_i32);

/* Integer-only LUT GEMM on given codes: acc[m][n] = sum_k table[(a[m][k] << 8) | b[k][n]]. */
void axo_lut_gemm_codes(const uint16_t *table, int m, int n, int k,
                        const uint8_t *a, const uint8_t *b, int32_t *acc);

/* Times the reference-faithful single-thread path (im2col chunk + table GEMM) on the first
 * `patches` output pixels of the described layer; returns seconds. */
double axo_time_reference_chunk(const uint16_t *table, axo_conv_desc *d,
                                const float *input, const float *filter,
                                float in_min, float in_max, float f_min, float f_max,
                                int patches, float *out_chunk);

/* tf1 AxConv2D, ReferenceAxConvFunctor (tf1/axqconv/axqconv.cc:113-278) for quint8 x quint8 -> qint32 with
 * offset_output 0, mult 1, shift 0 (:354-356): the seven loops, the per-product zero-point correction (:228-247),
 * taps outside the image reading the input offset (:213-216), the functor's own padding origin (:153-163).
 * table is indexed [input_code * 256 + filter_code] (approximate_selector.h:101-103).  Pinned by brute force
 * against the exact table (then it is the plain integer convolution of the offset-corrected codes).
 * padding: AXO_PAD_SAME / AXO_PAD_VALID; output [batches][out_h][out_w][filter_count]. */
void axo_axconv2d_tf1(const uint16_t *table, const uint8_t *input, int batches, int in_h, int in_w, int in_depth,
                      int input_offset, const uint8_t *filter, int filter_h, int filter_w, int filter_count,
                      int filter_offset, int stride, int padding, int32_t *output, int out_h, int out_w);

/* AxTune column remap of ApproximateSelector::init (tf1/axqconv/approximate_selector.h:52-85). */
void axo_table_tune_weights(const uint16_t *table, uint16_t *tuned);

#ifdef __cplusplus
}
#endif
#endif
