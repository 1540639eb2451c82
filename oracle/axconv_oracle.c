/*
 * CPU oracle for the ApproxConv2DWithMinMaxVars hot path -- TEST INFRASTRUCTURE ONLY.
 * See axconv_oracle.h for what each function restates and what pins it.
 *
 * Build with -O2 -ffp-contract=off and without -march=native: the reference is built
 * without FMA contraction, and every float expression below is meant to round after
 * each operation exactly as written.
 */
#include "axconv_oracle.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

/* ---- quantization parameters ------------------------------------------------------- */

/* approx_ops_types.h:29-49 */
void axo_nudge(float min, float max, int quant_min, int quant_max,
               float *nudged_min, float *nudged_max, float *scale)
{
    const float qmin_f = (float)quant_min;
    const float qmax_f = (float)quant_max;
    *scale = (max - min) / (qmax_f - qmin_f);
    const float zp_from_min = qmin_f - min / *scale;
    uint16_t nudged_zp;
    if (zp_from_min < qmin_f)
        nudged_zp = (uint16_t)quant_min;
    else if (zp_from_min > qmax_f)
        nudged_zp = (uint16_t)quant_max;
    else
        nudged_zp = (uint16_t)roundf(zp_from_min);
    *nudged_min = (qmin_f - (float)nudged_zp) * (*scale);
    *nudged_max = (qmax_f - (float)nudged_zp) * (*scale);
}

/* approx_ops_types.h:135-152 */
void axo_update_var_quant_props(float min_value, float max_value,
                                float *scale, float *inv_scale, float *offset)
{
    float nudged_scale = 0.0f, inv_nudged_scale = 0.0f, nudged_min = 0.0f, nudged_max = 0.0f;
    if (min_value != 0.0f || max_value != 0.0f) {
        axo_nudge(min_value, max_value, 0, 255, &nudged_min, &nudged_max, &nudged_scale);
        inv_nudged_scale = 1.0f / nudged_scale;
    }
    (void)nudged_max;
    *scale = nudged_scale;
    *inv_scale = inv_nudged_scale;
    *offset = nudged_min;
}

/* approx_ops_types.h:158-197 */
void axo_update_quant_props(float in_min, float in_max, float f_min, float f_max, axo_quant_props *qp)
{
    axo_update_var_quant_props(in_min, in_max, &qp->in_scale, &qp->in_inv_scale, &qp->in_offset);
    axo_update_var_quant_props(f_min, f_max, &qp->f_scale, &qp->f_inv_scale, &qp->f_offset);
    qp->s1xs2 = qp->in_scale * qp->f_scale;
    qp->m1 = qp->in_offset;
    qp->m2 = qp->f_offset;
    qp->m1xm2 = qp->m1 * qp->m2;
}

/* ---- lookup table ------------------------------------------------------------------ */

/* approx_ops_types.h:112-117 */
void axo_table_exact(uint16_t table[65536])
{
    for (uint32_t i = 0; i < 65536u; ++i)
        table[i] = (uint16_t)((i >> 8) * (i & 0xFFu));
}

/* approx_ops_types.h:205-216: zero-fill, read 65536 little-endian uint16, fail on a short read. */
int axo_table_load(const char *filename, uint16_t table[65536])
{
    memset(table, 0, 65536 * sizeof(uint16_t));
    FILE *f = fopen(filename, "rb");
    if (!f)
        return AXO_INVALID_ARGUMENT;
    unsigned char *raw = (unsigned char *)malloc(131072);
    size_t got = fread(raw, 1, 131072, f);
    fclose(f);
    if (got != 131072) {
        free(raw);
        return AXO_INVALID_ARGUMENT;
    }
    for (int i = 0; i < 65536; ++i)
        table[i] = (uint16_t)(raw[2 * i] | (raw[2 * i + 1] << 8));
    free(raw);
    return AXO_OK;
}

/* ---- quantize ---------------------------------------------------------------------- */

/* approx_nn_conv_kernels.cpp:193,197,243,293: AT((v - offset) * invScale + 0.5), AT = uint8.
 * The float->uint8 cast truncates toward zero.  Values that would land outside [0,255]
 * (undefined in the reference) clamp. */
uint8_t axo_quantize(float value, float offset, float inv_scale)
{
    volatile float d = value - offset;   /* volatile: force a rounding after every step */
    volatile float p = d * inv_scale;
    volatile float t = p + 0.5f;
    float tt = t;
    if (!(tt > 0.0f))
        return 0;
    if (tt >= 256.0f)
        return 255;
    return (uint8_t)tt;
}

void axo_quantize_array(const float *values, int64_t n, float offset, float inv_scale, uint8_t *codes)
{
    for (int64_t i = 0; i < n; ++i)
        codes[i] = axo_quantize(values[i], offset, inv_scale);
}

/* ---- geometry ---------------------------------------------------------------------- */

/* TF GetWindowedOutputSizeVerboseV2 (third-party; closed forms) */
static int windowed_output_size(int64_t in, int64_t filter, int64_t dilation, int64_t stride, int padding,
                                int64_t *out, int64_t *pad_before, int64_t *pad_after)
{
    if (stride <= 0 || dilation < 1)
        return AXO_INVALID_ARGUMENT;
    const int64_t eff = (filter - 1) * dilation + 1;
    if (padding == AXO_PAD_VALID) {
        *out = (in - eff + stride) / stride;
        *pad_before = *pad_after = 0;
    } else if (padding == AXO_PAD_SAME) {
        *out = (in + stride - 1) / stride;
        int64_t needed = (*out - 1) * stride + eff - in;
        if (needed < 0)
            needed = 0;
        *pad_before = needed / 2;
        *pad_after = needed - *pad_before;
    } else {
        *out = (in + *pad_before + *pad_after - eff + stride) / stride;
    }
    if (*out < 0)
        return AXO_INVALID_ARGUMENT;
    return AXO_OK;
}

/* approx_nn_conv_ops.cpp:311-404 */
int axo_conv_geometry(axo_conv_desc *d)
{
    if (d->patch_depth <= 0 || d->in_depth % d->patch_depth != 0)
        return AXO_INVALID_ARGUMENT; /* :338-341 */
    if (d->stride_rows <= 0 || d->stride_cols <= 0 || d->dilation_rows <= 0 || d->dilation_cols <= 0)
        return AXO_INVALID_ARGUMENT; /* :290-303 */
    if (d->padding != AXO_PAD_EXPLICIT) {
        d->pad_rows_before = d->pad_rows_after = d->pad_cols_before = d->pad_cols_after = 0;
    }
    int rc = windowed_output_size(d->in_rows, d->filter_rows, d->dilation_rows, d->stride_rows, d->padding,
                                  &d->out_rows, &d->pad_rows_before, &d->pad_rows_after);
    if (rc != AXO_OK)
        return rc;
    return windowed_output_size(d->in_cols, d->filter_cols, d->dilation_cols, d->stride_cols, d->padding,
                                &d->out_cols, &d->pad_cols_before, &d->pad_cols_after);
}

/* ---- kernels ----------------------------------------------------------------------- */

/* approx_nn_conv_kernels.cpp:260-296 */
void axo_im2col(const axo_quant_props *qp, const float *in,
                int c, int w, int h, int ow, int oh, int kw, int kh, int pw, int ph,
                int sw, int sh, int dw, int dh, int po, int pc,
                uint8_t *out, float *out_coeffs)
{
    const int pl = c * kw * kh;
    for (int i = 0; i < pc; ++i)
        out_coeffs[i] = 0.0f;
    for (int tId = 0; tId < pc * pl; ++tId) {
        int patchId = (tId + po * pl) / pl;
        int outB = (patchId / ow) / oh;
        int outH = (patchId / ow) % oh;
        int outW = patchId % ow;

        int valueId = (tId + po * pl) % pl;
        int offsetH = valueId / (kw * c);
        int offsetW = (valueId / c) % kw;
        int offsetC = valueId % c;

        int inH = outH * sh - ph + offsetH * dh;
        int inW = outW * sw - pw + offsetW * dw;

        float value = 0.0f;
        if (inH >= 0 && inW >= 0 && inH < h && inW < w)
            value = in[(((size_t)outB * h + inH) * w + inW) * c + offsetC];

        out[tId] = axo_quantize(value, qp->in_offset, qp->in_inv_scale);
        volatile float s = out_coeffs[patchId - po] + value;
        out_coeffs[patchId - po] = s;
    }
}

/* approx_nn_conv_kernels.cpp:300-306.  The reference uses an Eigen reduction whose order is
 * unspecified; here the order is h, w, c ascending. */
void axo_filter_sums(const float *filter, int kh, int kw, int c, int co, float *sums)
{
    const int k = kh * kw * c;
    for (int j = 0; j < co; ++j) {
        volatile float s = 0.0f;
        for (int l = 0; l < k; ++l)
            s = s + filter[(size_t)l * co + j];
        sums[j] = s;
    }
}

static inline float epilogue(const axo_quant_props *qp, float total, float a_sum, float b_sum, int k)
{
    /* approx_nn_conv_kernels.cpp:250-253 / :205-208, left to right, one rounding per operation */
    volatile float t0 = total * qp->s1xs2;
    volatile float t1 = qp->m2 * a_sum;
    volatile float t2 = t0 + t1;
    volatile float t3 = qp->m1 * b_sum;
    volatile float t4 = t2 + t3;
    volatile float t5 = (float)k * qp->m1xm2;
    volatile float t6 = t4 - t5;
    return t6;
}

/* approx_nn_conv_kernels.cpp:215-256 */
void axo_gemm_table(const axo_quant_props *qp, const uint16_t *table,
                    int m, int n, int k, const uint8_t *a, int lda, const float *b, int ldb,
                    const float *a_coeffs, const float *b_coeffs, float *c, int ldc, int32_t *acc_i32)
{
    for (size_t j = 0; j < (size_t)n; ++j) {
        for (size_t i = 0; i < (size_t)m; ++i) {
            float total = 0.0f;
            int32_t itotal = 0;
            for (size_t l = 0; l < (size_t)k; ++l) {
                const uint32_t aValue = a[i * (size_t)lda + l];
                const uint32_t bValue = axo_quantize(b[l * (size_t)ldb + j], qp->f_offset, qp->f_inv_scale);
                const uint32_t cValue = table[(aValue << 8) | bValue];
                total += (float)cValue;
                itotal += (int32_t)cValue;
            }
            c[i * (size_t)ldc + j] = epilogue(qp, total, a_coeffs[i], b_coeffs[j], k);
            if (acc_i32)
                acc_i32[i * (size_t)ldc + j] = itotal;
        }
    }
}

/* approx_nn_conv_kernels.cpp:167-211 */
void axo_gemm_combined(const axo_quant_props *qp, const uint16_t *table,
                       int m, int n, int k, const float *a, int lda, const float *b, int ldb,
                       float *c, int ldc, int32_t *acc_i32)
{
    for (size_t j = 0; j < (size_t)n; ++j) {
        for (size_t i = 0; i < (size_t)m; ++i) {
            float total = 0.0f, aSum = 0.0f, bSum = 0.0f;
            int32_t itotal = 0;
            for (size_t l = 0; l < (size_t)k; ++l) {
                const float av = a[i * (size_t)lda + l];
                const uint32_t aValue = axo_quantize(av, qp->in_offset, qp->in_inv_scale);
                aSum += av;
                const float bv = b[l * (size_t)ldb + j];
                const uint32_t bValue = axo_quantize(bv, qp->f_offset, qp->f_inv_scale);
                bSum += bv;
                const uint32_t cValue = table[(aValue << 8) | bValue];
                total += (float)cValue;
                itotal += (int32_t)cValue;
            }
            c[i * (size_t)ldc + j] = epilogue(qp, total, aSum, bSum, k);
            if (acc_i32)
                acc_i32[i * (size_t)ldc + j] = itotal;
        }
    }
}

/* ---- op ---------------------------------------------------------------------------- */

#define AXO_MAX_CHUNK ((int64_t)(16 * 1024 * 1024) / (int64_t)sizeof(float)) /* approx_nn_conv_ops.cpp:118 */

/* approx_nn_conv_ops.cpp:420-460 (Compute) + :211-247 (CPU launcher checks) + :70-206 (LaunchGeneric) */
int axo_conv2d(const uint16_t *table, axo_conv_desc *d,
               const float *input, const float *filter,
               float in_min, float in_max, float f_min, float f_max,
               float *output, int32_t *acc_i32)
{
    int rc = axo_conv_geometry(d);
    if (rc != AXO_OK)
        return rc;
    if ((int64_t)d->batch * d->out_rows * d->out_cols * d->out_depth == 0)
        return AXO_OK; /* :449 */
    if (d->in_depth != d->patch_depth)
        return AXO_UNIMPLEMENTED; /* :229-232 grouped convolution */

    axo_quant_props qp;
    axo_update_quant_props(in_min, in_max, f_min, f_max, &qp);

    const int N = d->batch, H = d->in_rows, W = d->in_cols, C = d->in_depth;
    const int KH = d->filter_rows, KW = d->filter_cols, CO = d->out_depth;
    const int OH = (int)d->out_rows, OW = (int)d->out_cols;

    if (KH == 1 && KW == 1 && d->stride_rows == 1 && d->stride_cols == 1 &&
        (d->padding == AXO_PAD_SAME || d->padding == AXO_PAD_VALID)) {
        /* :81-97 */
        axo_gemm_combined(&qp, table, N * H * W, CO, C, input, C, filter, CO, output, CO, acc_i32);
        return AXO_OK;
    }
    if (KH == H && KW == W && d->dilation_rows == 1 && d->dilation_cols == 1 && d->padding == AXO_PAD_VALID) {
        /* :98-115 */
        axo_gemm_combined(&qp, table, N, CO, H * W * C, input, H * W * C, filter, CO, output, CO, acc_i32);
        return AXO_OK;
    }

    /* :116-204 */
    const int64_t patch_len = (int64_t)KH * KW * C;
    if (patch_len > AXO_MAX_CHUNK)
        return AXO_INVALID_ARGUMENT; /* :120-121 */
    if (d->padding == AXO_PAD_EXPLICIT)
        return AXO_UNIMPLEMENTED; /* :160-163 */

    const int64_t total = (int64_t)N * OH * OW;
    const int64_t per_chunk = AXO_MAX_CHUNK / patch_len;
    uint8_t *im2col = (uint8_t *)malloc((size_t)AXO_MAX_CHUNK);
    float *patch_coeff = (float *)malloc((size_t)per_chunk * sizeof(float));
    float *filter_coeff = (float *)malloc((size_t)CO * sizeof(float));
    axo_filter_sums(filter, KH, KW, C, CO, filter_coeff);

    float *out = output;
    int32_t *acc = acc_i32;
    for (int64_t i = 0; i < total; i += per_chunk) {
        int64_t batch = i / ((int64_t)OH * OW);
        int patch_offset = (int)(i % ((int64_t)OH * OW));
        int count = (int)((per_chunk < total - i) ? per_chunk : (total - i));
        const float *in = input + (size_t)batch * H * W * C;
        axo_im2col(&qp, in, C, W, H, OW, OH, KW, KH, (int)d->pad_cols_before, (int)d->pad_rows_before,
                   d->stride_cols, d->stride_rows, d->dilation_cols, d->dilation_rows,
                   patch_offset, count, im2col, patch_coeff);
        axo_gemm_table(&qp, table, count, CO, (int)patch_len, im2col, (int)patch_len, filter, CO,
                       patch_coeff, filter_coeff, out, CO, acc);
        out += per_chunk * CO;
        if (acc)
            acc += per_chunk * CO;
    }
    free(im2col);
    free(patch_coeff);
    free(filter_coeff);
    return AXO_OK;
}

/* approx_nn_conv_ops_ref.cpp:231-317 */
int axo_conv2d_direct(const uint16_t *table, axo_conv_desc *d,
                      const float *input, const float *filter,
                      float in_min, float in_max, float f_min, float f_max, float *output)
{
    int rc = axo_conv_geometry(d);
    if (rc != AXO_OK)
        return rc;
    if (d->dilation_rows != 1 || d->dilation_cols != 1 || d->in_depth != d->patch_depth)
        return AXO_UNIMPLEMENTED;
    axo_quant_props qp;
    axo_update_quant_props(in_min, in_max, f_min, f_max, &qp);
    const int N = d->batch, H = d->in_rows, W = d->in_cols, C = d->in_depth;
    const int KH = d->filter_rows, KW = d->filter_cols, CO = d->out_depth;
    const int OH = (int)d->out_rows, OW = (int)d->out_cols;
    int left, top;
    if (d->padding == AXO_PAD_VALID) {
        left = ((OW - 1) * d->stride_cols + KW - W + 1) / 2;
        top = ((OH - 1) * d->stride_rows + KH - H + 1) / 2;
    } else {
        left = ((OW - 1) * d->stride_cols + KW - W) / 2;
        top = ((OH - 1) * d->stride_rows + KH - H) / 2;
    }
    for (int b = 0; b < N; ++b)
        for (int oy = 0; oy < OH; ++oy)
            for (int ox = 0; ox < OW; ++ox)
                for (int oc = 0; oc < CO; ++oc) {
                    const int x0 = ox * d->stride_cols - left;
                    const int y0 = oy * d->stride_rows - top;
                    float total = 0.0f, in_total = 0.0f, f_total = 0.0f;
                    for (int fy = 0; fy < KH; ++fy)
                        for (int fx = 0; fx < KW; ++fx)
                            for (int ic = 0; ic < C; ++ic) {
                                const int ix = x0 + fx, iy = y0 + fy;
                                float iv = 0.0f;
                                if (ix >= 0 && ix < W && iy >= 0 && iy < H)
                                    iv = input[(((size_t)b * H + iy) * W + ix) * C + ic];
                                const float fv = filter[(((size_t)fy * KW + fx) * C + ic) * CO + oc];
                                in_total += iv;
                                f_total += fv;
                                const uint32_t qa = axo_quantize(iv, qp.in_offset, qp.in_inv_scale);
                                const uint32_t qb = axo_quantize(fv, qp.f_offset, qp.f_inv_scale);
                                total += (float)table[(qa << 8) | qb];
                            }
                    output[(((size_t)b * OH + oy) * OW + ox) * CO + oc] =
                        epilogue(&qp, total, in_total, f_total, KH * KW * C);
                }
    return AXO_OK;
}

/* Integer sums with pre-quantized codes; see header. */
int axo_conv2d_fast(const uint16_t *table, axo_conv_desc *d,
                    const float *input, const float *filter,
                    float in_min, float in_max, float f_min, float f_max,
                    float *output, int32_t *acc_i32, int threads)
{
    int rc = axo_conv_geometry(d);
    if (rc != AXO_OK)
        return rc;
    if (d->in_depth != d->patch_depth)
        return AXO_UNIMPLEMENTED;
    if (d->padding == AXO_PAD_EXPLICIT)
        return AXO_UNIMPLEMENTED;
    axo_quant_props qp;
    axo_update_quant_props(in_min, in_max, f_min, f_max, &qp);
    const int N = d->batch, H = d->in_rows, W = d->in_cols, C = d->in_depth;
    const int KH = d->filter_rows, KW = d->filter_cols, CO = d->out_depth;
    const int OH = (int)d->out_rows, OW = (int)d->out_cols;
    const int K = KH * KW * C;
    const int64_t M = (int64_t)N * OH * OW;
    if (M * CO == 0)
        return AXO_OK;

    uint8_t *fq = (uint8_t *)malloc((size_t)K * CO);
    float *fsum = (float *)malloc((size_t)CO * sizeof(float));
    for (size_t i = 0; i < (size_t)K * CO; ++i)
        fq[i] = axo_quantize(filter[i], qp.f_offset, qp.f_inv_scale);
    axo_filter_sums(filter, KH, KW, C, CO, fsum);
    /* transpose codes to [CO][K] so the inner loop is contiguous */
    uint8_t *fqt = (uint8_t *)malloc((size_t)K * CO);
    for (int l = 0; l < K; ++l)
        for (int j = 0; j < CO; ++j)
            fqt[(size_t)j * K + l] = fq[(size_t)l * CO + j];
    const uint8_t zp = axo_quantize(0.0f, qp.in_offset, qp.in_inv_scale);
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel num_threads(threads > 0 ? threads : 1)
#endif
    {
        uint8_t *patch = (uint8_t *)malloc((size_t)K);
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
        for (int64_t p = 0; p < M; ++p) {
            int b = (int)(p / ((int64_t)OH * OW));
            int oy = (int)((p / OW) % OH);
            int ox = (int)(p % OW);
            float psum = 0.0f;
            int l = 0;
            for (int fy = 0; fy < KH; ++fy)
                for (int fx = 0; fx < KW; ++fx) {
                    int iy = oy * d->stride_rows - (int)d->pad_rows_before + fy * d->dilation_rows;
                    int ix = ox * d->stride_cols - (int)d->pad_cols_before + fx * d->dilation_cols;
                    if (iy >= 0 && ix >= 0 && iy < H && ix < W) {
                        const float *src = input + (((size_t)b * H + iy) * W + ix) * C;
                        for (int ic = 0; ic < C; ++ic, ++l) {
                            patch[l] = axo_quantize(src[ic], qp.in_offset, qp.in_inv_scale);
                            volatile float s = psum + src[ic];
                            psum = s;
                        }
                    } else {
                        for (int ic = 0; ic < C; ++ic, ++l) {
                            patch[l] = zp;
                            volatile float s = psum + 0.0f;
                            psum = s;
                        }
                    }
                }
            for (int j = 0; j < CO; ++j) {
                const uint8_t *wj = fqt + (size_t)j * K;
                int32_t acc = 0;
                for (int q = 0; q < K; ++q)
                    acc += table[((uint32_t)patch[q] << 8) | wj[q]];
                if (acc_i32)
                    acc_i32[(size_t)p * CO + j] = acc;
                if (output)
                    output[(size_t)p * CO + j] = epilogue(&qp, (float)acc, psum, fsum[j], K);
            }
        }
        free(patch);
    }
    free(fq);
    free(fqt);
    free(fsum);
    return AXO_OK;
}

/* Depthwise: the dense op per channel (see header). */
int axo_depthwise_conv2d(const uint16_t *table, axo_conv_desc *d,
                         const float *input, const float *filter,
                         float in_min, float in_max, float f_min, float f_max,
                         float *output, int32_t *acc_i32)
{
    if (d->patch_depth != d->in_depth || d->out_depth != d->in_depth)
        return AXO_INVALID_ARGUMENT; /* filter [kh,kw,C,1] is described as patch_depth = out_depth = C */
    const int C = d->in_depth;
    axo_conv_desc g = *d;
    int rc = axo_conv_geometry(&g);
    if (rc != AXO_OK)
        return rc;
    *d = g;
    const int N = d->batch, H = d->in_rows, W = d->in_cols;
    const int KH = d->filter_rows, KW = d->filter_cols;
    const int OH = (int)d->out_rows, OW = (int)d->out_cols;
    const size_t M = (size_t)N * OH * OW;
    if (M * C == 0)
        return AXO_OK;
    float *xin = (float *)malloc((size_t)N * H * W * sizeof(float));
    float *fin = (float *)malloc((size_t)KH * KW * sizeof(float));
    float *yout = (float *)malloc(M * sizeof(float));
    int32_t *aout = (int32_t *)malloc(M * sizeof(int32_t));
    for (int c = 0; c < C; ++c) {
        for (size_t p = 0; p < (size_t)N * H * W; ++p)
            xin[p] = input[p * C + c];
        for (int t = 0; t < KH * KW; ++t)
            fin[t] = filter[(size_t)t * C + c];
        axo_conv_desc one = *d;
        one.in_depth = one.patch_depth = one.out_depth = 1;
        /* force the generic (im2col) path for every shape: 1x1 and full-image filters give the
         * same sums through either path */
        rc = axo_conv2d_fast(table, &one, xin, fin, in_min, in_max, f_min, f_max, yout, aout, 1);
        if (rc != AXO_OK)
            break;
        for (size_t p = 0; p < M; ++p) {
            if (output)
                output[p * C + c] = yout[p];
            if (acc_i32)
                acc_i32[p * C + c] = aout[p];
        }
    }
    free(xin);
    free(fin);
    free(yout);
    free(aout);
    return rc;
}

void axo_lut_gemm_codes(const uint16_t *table, int m, int n, int k,
                        const uint8_t *a, const uint8_t *b, int32_t *acc)
{
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            int32_t s = 0;
            for (int l = 0; l < k; ++l)
                s += table[((uint32_t)a[(size_t)i * k + l] << 8) | b[(size_t)l * n + j]];
            acc[(size_t)i * n + j] = s;
        }
}

static double now_s(void)
{
    struct timespec ts;
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}

double axo_time_reference_chunk(const uint16_t *table, axo_conv_desc *d,
                                const float *input, const float *filter,
                                float in_min, float in_max, float f_min, float f_max,
                                int patches, float *out_chunk)
{
    if (axo_conv_geometry(d) != AXO_OK)
        return -1.0;
    axo_quant_props qp;
    axo_update_quant_props(in_min, in_max, f_min, f_max, &qp);
    const int H = d->in_rows, W = d->in_cols, C = d->in_depth;
    const int KH = d->filter_rows, KW = d->filter_cols, CO = d->out_depth;
    const int OH = (int)d->out_rows, OW = (int)d->out_cols;
    const int K = KH * KW * C;
    uint8_t *im2col = (uint8_t *)malloc((size_t)patches * K);
    float *patch_coeff = (float *)malloc((size_t)patches * sizeof(float));
    float *filter_coeff = (float *)malloc((size_t)CO * sizeof(float));
    double t0 = now_s();
    axo_filter_sums(filter, KH, KW, C, CO, filter_coeff);
    axo_im2col(&qp, input, C, W, H, OW, OH, KW, KH, (int)d->pad_cols_before, (int)d->pad_rows_before,
               d->stride_cols, d->stride_rows, d->dilation_cols, d->dilation_rows, 0, patches, im2col, patch_coeff);
    axo_gemm_table(&qp, table, patches, CO, K, im2col, K, filter, CO, patch_coeff, filter_coeff, out_chunk, CO, NULL);
    double t1 = now_s();
    free(im2col);
    free(patch_coeff);
    free(filter_coeff);
    return t1 - t0;
}

/* tf1/axqconv/axqconv.cc:113-278 */
void axo_axconv2d_tf1(const uint16_t *table, const uint8_t *input, int batches, int in_h, int in_w, int in_depth,
                      int input_offset, const uint8_t *filter, int filter_h, int filter_w, int filter_count,
                      int filter_offset, int stride, int padding, int32_t *output, int out_h, int out_w)
{
    int left, top;
    if (padding == AXO_PAD_VALID) { /* :153-157 */
        left = ((out_w - 1) * stride + filter_w - in_w + 1) / 2;
        top = ((out_h - 1) * stride + filter_h - in_h + 1) / 2;
    } else {                        /* :158-163 */
        left = ((out_w - 1) * stride + filter_w - in_w) / 2;
        top = ((out_h - 1) * stride + filter_h - in_h) / 2;
    }
    for (int batch = 0; batch < batches; ++batch)
        for (int oy = 0; oy < out_h; ++oy)
            for (int ox = 0; ox < out_w; ++ox)
                for (int oc = 0; oc < filter_count; ++oc) {
                    const int x0 = ox * stride - left, y0 = oy * stride - top;
                    int32_t total = 0;
                    for (int fy = 0; fy < filter_h; ++fy)
                        for (int fx = 0; fx < filter_w; ++fx)
                            for (int ic = 0; ic < in_depth; ++ic) {
                                const int ix = x0 + fx, iy = y0 + fy;
                                int32_t a;
                                if (ix >= 0 && ix < in_w && iy >= 0 && iy < in_h)
                                    a = input[(((size_t)batch * in_h + iy) * in_w + ix) * in_depth + ic];
                                else
                                    a = (uint8_t)input_offset; /* :215: stored into the quint8 source value */
                                const int32_t b = filter[(((size_t)fy * filter_w + fx) * in_depth + ic) * filter_count + oc];
                                const int32_t axm = table[a * 256 + b];
                                total += axm - a * filter_offset - b * input_offset + input_offset * filter_offset;
                            }
                    output[(((size_t)batch * out_h + oy) * out_w + ox) * filter_count + oc] = total;
                }
}

/* tf1/axqconv/approximate_selector.h:52-85 */
void axo_table_tune_weights(const uint16_t *table, uint16_t *tuned)
{
    for (int w = 0; w < 256; ++w) {
        int wpos = -1, werr = 0;
        for (int w2 = 0; w2 < 256; ++w2) {
            int sumerr = 0;
            for (int i = 0; i < 256; ++i)
                sumerr += abs(i * w - (int)table[i * 256 + w2]);
            if (sumerr < werr || (werr == sumerr && w2 == w) || wpos < 0) {
                werr = sumerr;
                wpos = w2;
            }
        }
        for (int i = 0; i < 256; ++i)
            tuned[i * 256 + w] = table[i * 256 + wpos];
    }
}
