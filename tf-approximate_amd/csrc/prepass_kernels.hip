// Pre-pass kernels: quantize + relayout of the input, filter quantize/pack/sums, flat quantize.
#include "axconv_internal.h"
#include "px_expand.h"
#include <type_traits>

namespace axc {

// Keeps the LDS reads and the adds (into `sum`) around it in program order, in the compiler's own passes and in its
// scheduler: the empty statement claims to read and write both memory and the running sum.
__device__ __forceinline__ void chain_fence(float &sum)
{
    __asm__ volatile("" : "+v"(sum) : : "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Waits until at most `pending` LDS reads of this wavefront are outstanding (they return in order).  A lone wavefront
// issues about one instruction per four cycles whatever its kind, so one wait per batch of reads instead of one per
// read is time the chain gets back.
template <int PENDING>
__device__ __forceinline__ void wait_lds_reads()
{
    static_assert(PENDING >= 0 && PENDING <= 15, "lgkmcnt is a 4-bit counter");
    __builtin_amdgcn_s_waitcnt(0xC07F | (PENDING << 8)); // vmcnt and expcnt left at their maxima
}

// Input pre-pass.  Restates the quantize and the channel part of the patch sum of
// ApproxConvIm2ColKernel (tf2/src/approx_nn_conv_kernels.cpp:288-294) once per input element
// instead of once per patch element.
//   xq   [N][H][C4][W]  one dword = codes of channels 4*c4 .. 4*c4+3 of one pixel, each code stored as
//                       its expanded-row index phys_row(code)
//   chsum[N][H][W]      sum over channels of the raw floats, c ascending
// One thread per pixel: the channel loop is sequential so the sum has the reference's order within a pixel.
__global__ void __launch_bounds__(256) quantize_relayout_kernel(const float *__restrict__ x, int64_t pixels,
                                                                 int H, int W, int C, int C4, const TensorQuant tq,
                                                                 const LayerQuant *__restrict__ lq_dev,
                                                                 uint32_t *__restrict__ xq,
                                                                 float *__restrict__ chsum)
{
    const TensorQuant q = lq_dev ? lq_dev->in : tq;
    const uint32_t zp4 = q.zp4;
    const int64_t pix = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    // the extra [C4][W] row behind the image rows: every dword is the zero-point code x4
    for (int64_t i = pix; i < (int64_t)C4 * W; i += (int64_t)gridDim.x * blockDim.x)
        xq[pixels * C4 + i] = zp4;
    if (pix >= pixels)
        return;
    const int w = (int)(pix % W);
    const int64_t nh = pix / W; // n * H + h
    const float *src = x + pix * C;
    float sum = 0.0f;
    for (int c4 = 0; c4 < C4; ++c4) {
        uint32_t packed = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = c4 * 4 + i;
            if (c < C) {
                const float v = fake_quant_value(src[c], q);
                sum = __fadd_rn(sum, v);
                packed |= phys_row(quantize_code(v, q.offset, q.inv_scale)) << (8 * i);
            }
        }
        xq[(nh * C4 + c4) * W + w] = packed;
    }
    if (chsum)
        chsum[pix] = sum;
}

// Same result as quantize_relayout_kernel for C % 4 == 0, with fully coalesced reads: consecutive lanes
// read consecutive float4 of the NHWC input (one float4 = the four channels of one xq dword).
__global__ void __launch_bounds__(256) quantize_relayout_vec4_kernel(const float4 *__restrict__ x4, int64_t quads,
                                                                      int W, int C4, const TensorQuant tq,
                                                                      const LayerQuant *__restrict__ lq_dev,
                                                                      uint32_t *__restrict__ xq)
{
    const TensorQuant q = lq_dev ? lq_dev->in : tq;
    const uint32_t zp4 = q.zp4;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    // the extra [C4][W] row behind the image rows: every dword is the zero-point code x4
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < (int64_t)C4 * W; i += stride)
        xq[quads + i] = zp4;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < quads; i += stride) {
        const float4 v = x4[i];
        const int64_t pix = i / C4;
        const int c4 = (int)(i - pix * C4);
        const int64_t nh = pix / W;
        const int w = (int)(pix - nh * W);
        const uint32_t packed = phys_row(quantize_code(fake_quant_value(v.x, q), q.offset, q.inv_scale)) |
                                (phys_row(quantize_code(fake_quant_value(v.y, q), q.offset, q.inv_scale)) << 8) |
                                (phys_row(quantize_code(fake_quant_value(v.z, q), q.offset, q.inv_scale)) << 16) |
                                (phys_row(quantize_code(fake_quant_value(v.w, q), q.offset, q.inv_scale)) << 24);
        xq[(nh * C4 + c4) * W + w] = packed;
    }
}

// Patch sums (the outCoeffs of ApproxConvIm2ColKernel, tf2/src/approx_nn_conv_kernels.cpp:294): for each
// output pixel the fp32 sum of the raw input over its patch, accumulated strictly in the reference's order
// (kh, kw, c ascending; taps outside the image add 0.0f, which leaves the sum unchanged).  fp32 addition is
// not associative and this sum is multiplied by the filter offset in the epilogue, so any other order
// shows up in the output at the 1e-4 level for inputs with a large mean.  One thread per output pixel.
__device__ __forceinline__ float4 fake_quant_value4(float4 v, const TensorQuant &q)
{
    return make_float4(fake_quant_value(v.x, q), fake_quant_value(v.y, q), fake_quant_value(v.z, q),
                       fake_quant_value(v.w, q));
}

__global__ void __launch_bounds__(256) patch_sums_kernel(const float *__restrict__ x, ConvGeom g, const TensorQuant tq,
                                                          const LayerQuant *__restrict__ lq_dev,
                                                          float *__restrict__ psum)
{
    const TensorQuant q = lq_dev ? lq_dev->in : tq;
    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= g.M)
        return;
    const int n = (int)(m / ((int64_t)g.OH * g.OW));
    const int rem = (int)(m - (int64_t)n * g.OH * g.OW);
    const int oh = rem / g.OW, ow = rem - oh * g.OW;
    const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
    float s = 0.0f;
    for (int kh = 0; kh < g.KH; ++kh) {
        const int ih = ih0 + kh * g.dh;
        if ((unsigned)ih >= (unsigned)g.H)
            continue;
        for (int kw = 0; kw < g.KW; ++kw) {
            const int iw = iw0 + kw * g.dw;
            if ((unsigned)iw >= (unsigned)g.W)
                continue;
            const float *src = x + (((int64_t)n * g.H + ih) * g.W + iw) * g.C;
            if ((g.C & 3) == 0) {
                const float4 *src4 = reinterpret_cast<const float4 *>(src);
                for (int c4 = 0; c4 < g.C / 4; ++c4) {
                    const float4 v = fake_quant_value4(src4[c4], q);
                    s = __fadd_rn(s, v.x);
                    s = __fadd_rn(s, v.y);
                    s = __fadd_rn(s, v.z);
                    s = __fadd_rn(s, v.w);
                }
            } else {
                for (int c = 0; c < g.C; ++c)
                    s = __fadd_rn(s, fake_quant_value(src[c], q));
            }
        }
    }
    psum[m] = s;
}

// Patch sums for C % 4 == 0, same order and same results as patch_sums_kernel.  One thread per output
// pixel still owns the sequential chain, but the floats arrive through LDS: for each tap and 32-channel
// slice the block loads the 256 input pixels of its 256 output pixels cooperatively (8 lanes read the 128
// contiguous bytes of one pixel's slice), so a wavefront touches 8 memory lines per load instead of 64.
// The loads of the next slice are in flight while the block adds up the current one.
constexpr int kPsTile = 256;  // output pixels per block
constexpr int kPsCh = 32;     // channels per LDS slice
constexpr int kPsRow = kPsCh + 4; // padded row (floats): conflict-free 16-byte accesses
constexpr int kPsLoads = kPsCh / 4 * kPsTile / kPsTile; // float4 loads per thread per slice

__global__ void __launch_bounds__(kPsTile) patch_sums_tiled_kernel(const float *__restrict__ x, ConvGeom g,
                                                                    const TensorQuant tq,
                                                                    const LayerQuant *__restrict__ lq_dev,
                                                                    float *__restrict__ psum)
{
    const TensorQuant qt = lq_dev ? lq_dev->in : tq;
    __shared__ int pix_base[kPsTile];  // (n * H) of the pixel's image, or -1 when the pixel does not exist
    __shared__ int pix_hw[kPsTile];    // input row / column of tap (0, 0), 16 bits each
    __shared__ __align__(16) float tile[kPsTile * kPsRow];
    constexpr int kQuads = kPsCh / 4;  // float4 per pixel per slice
    const int t = threadIdx.x;
    const int64_t m = (int64_t)blockIdx.x * kPsTile + t;
    const bool valid = m < g.M;
    {
        int n = 0, ih0 = 0, iw0 = 0;
        if (valid) {
            n = (int)(m / ((int64_t)g.OH * g.OW));
            const int rem = (int)(m - (int64_t)n * g.OH * g.OW);
            const int oh = rem / g.OW, ow = rem - oh * g.OW;
            ih0 = oh * g.sh - g.ph;
            iw0 = ow * g.sw - g.pw;
        }
        pix_base[t] = valid ? n * g.H : -1;
        pix_hw[t] = (ih0 << 16) | (iw0 & 0xffff);
    }
    __syncthreads();
    // this thread fetches quad j of the pixels pl0, pl0 + 32, ... of every slice
    const int j = t % kQuads, pl0 = t / kQuads;
    int lbase[kPsLoads], lih[kPsLoads], liw[kPsLoads];
#pragma unroll
    for (int i = 0; i < kPsLoads; ++i) {
        const int pl = pl0 + i * (kPsTile / kQuads);
        lbase[i] = pix_base[pl];
        lih[i] = pix_hw[pl] >> 16;
        liw[i] = (int)(int16_t)(pix_hw[pl] & 0xffff);
    }
    const int slices = (g.C + kPsCh - 1) / kPsCh;
    const int iters = g.KH * g.KW * slices;
    float4 v[kPsLoads];
    auto fetch = [&](int it) {
        const int tap = it / slices, c0 = (it - tap * slices) * kPsCh;
        const int kh = tap / g.KW, kw = tap - kh * g.KW;
#pragma unroll
        for (int i = 0; i < kPsLoads; ++i) {
            const int ih = lih[i] + kh * g.dh, iw = liw[i] + kw * g.dw;
            v[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (lbase[i] >= 0 && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W && c0 + j * 4 < g.C)
                v[i] = *reinterpret_cast<const float4 *>(x + ((int64_t)(lbase[i] + ih) * g.W + iw) * g.C + c0 + j * 4);
        }
    };
    float s = 0.0f;
    fetch(0);
    for (int it = 0; it < iters; ++it) {
        __syncthreads(); // previous slice consumed
#pragma unroll
        for (int i = 0; i < kPsLoads; ++i)   // 0.0f (a tap outside the image) lies on the grid: snapping keeps it 0.0f
            *reinterpret_cast<float4 *>(&tile[(pl0 + i * (kPsTile / kQuads)) * kPsRow + j * 4]) =
                qt.fq ? fake_quant_value4(v[i], qt) : v[i];
        __syncthreads();
        if (it + 1 < iters)
            fetch(it + 1);
        const int c0 = (it % slices) * kPsCh;
        const int nq = (g.C - c0 < kPsCh ? g.C - c0 : kPsCh) / 4;
        // taps outside the image were stored as 0.0f: x + 0.0f == x (the sum never is -0.0f after a real term,
        // and 0.0f + 0.0f stays +0.0f as in the reference, which starts from +0.0f)
        for (int q = 0; q < nq; ++q) {
            const float4 w = *reinterpret_cast<const float4 *>(&tile[t * kPsRow + q * 4]);
            s = __fadd_rn(s, w.x);
            s = __fadd_rn(s, w.y);
            s = __fadd_rn(s, w.z);
            s = __fadd_rn(s, w.w);
        }
    }
    if (valid)
        psum[m] = s;
}

// The filter pre-pass of a layer is independent of its input pre-pass: as two launches they would run one after
// the other, so the launch below carries both: the filter work of filter_prep_kernel in workgroups of its own
// (ordered as described at the members below), the patch sums in the others.
struct FilterWork {
    const float *filter;
    const uint8_t *filter_codes;
    int taps, C, C4, Co, nt, n_col_tiles;
    TensorQuant tq;
    uint16_t *wq;
    int sum_blocks;
    float *fsum;
    // Order of the workgroups of a launch: the filter sums (long chains: first), rounded up to a multiple of 8 so
    // that workgroup index mod 8 stays the XCD for the others; the patch sums; the workgroups that pack filter codes
    // (many and short: they fill the tail).
    int sum8;         // sum_blocks rounded up to a multiple of 8
    int work_blocks;  // patch-sum workgroups
    int pack_blocks;  // 0: no pack workgroups
    // pack_total > 0: no pack blocks; the threads of the patch-sum blocks that run no chain pack the codes,
    // each block its share of the pack_total elements
    int64_t pack_total;
    // expand_blocks > 0: the last workgroups of the launch build the pre-expanded rows of lutgemm_px_kernel.hip
    // (px_expand.h), blockDim.x / 4 activation codes of one (column tile, pair of fills) each: the rows depend on the
    // filter and the table only, so they need not wait for the patch sums in a launch of their own
    int expand_blocks;
    const uint16_t *tableT;
    uint16_t *px_rows;
};

__device__ __forceinline__ void filter_pack_element(const int64_t i, const float *__restrict__ filter,
                                                    const uint8_t *__restrict__ filter_codes, int taps, int C,
                                                    int C4, int Co, int nt, int n_col_tiles, const TensorQuant &qf,
                                                    uint16_t *__restrict__ wq);

// Patch sums for C % 4 == 0 when the input rows under a band of output rows fit in LDS: same order and same
// results as patch_sums_kernel.  A block owns `rb` consecutive output rows of one image (one thread per output
// pixel) and first copies the input rows they touch into LDS, so every input float is fetched from memory
// about once (plus the halo) instead of once per filter tap; the sequential chains then read LDS only.
// Pixels are padded to C + 4 floats so that the 16-byte reads of neighbouring threads fall into different banks.
// bid / nblocks: index of this workgroup among those that do this work (in dispatch order, so that bid & 7 is
// the XCD); nthreads: the threads of the workgroup that take part (the others only meet the barrier).
// wseg: output columns per workgroup.  wseg == OW: whole rows.  Less (wide rows of many channels, which would not
// fit LDS otherwise): a band is cut into column segments, each with the input columns under it in LDS (SEG; without
// it the code is the one for whole rows, with no trace of the segments).
template <bool SEG>
__device__ __forceinline__ void patch_sums_rows_body(const float *__restrict__ x, const ConvGeom &g, const int rb,
                                                     const int in_rows, const int wseg, const TensorQuant &tq,
                                                     const LayerQuant *__restrict__ lq_dev, float *__restrict__ psum,
                                                     uint32_t *__restrict__ xq, const int bid_in, const int nblocks,
                                                     const int nthreads, const FilterWork &fw)
{
    // xq != nullptr: the block also quantizes the input rows it owns among those it copies (the rows under its
    // own band of output rows; the launcher has checked that these lie inside every block's window and together
    // cover the image), which saves the separate quantize pass over the input.
    const TensorQuant qt = lq_dev ? lq_dev->in : tq;
    if (xq && bid_in == 0)
        for (int i = threadIdx.x; i < g.C4 * g.W; i += blockDim.x)
            xq[(int64_t)g.N * g.H * g.C4 * g.W + i] = qt.zp4;
    extern __shared__ __align__(16) unsigned char ps_lds[];
    float *const rows = reinterpret_cast<float *>(ps_lds);
    const int t = threadIdx.x;
    const int bands = (g.OH + rb - 1) / rb;
    // consecutive bands (which share input rows) go to the same XCD: blocks are dealt round-robin over 8 XCDs
    const int per_xcd = nblocks / 8, extra = nblocks % 8, xcd = bid_in & 7;
    const int bid = xcd * per_xcd + (xcd < extra ? xcd : extra) + (bid_in >> 3);
    const int segs = SEG ? (g.OW + wseg - 1) / wseg : 1;
    const int nb = SEG ? bid / segs : bid, seg = SEG ? bid - nb * segs : 0;   // nb: (image, band)
    const int n = nb / bands, band = nb - n * bands;
    const int oh0 = band * rb;
    const int ih_first = oh0 * g.sh - g.ph;  // input row held in LDS row 0 (may lie outside the image)
    const int own_lo = oh0 * g.sh;           // owned input rows: [own_lo, own_hi)
    const int own_hi = (oh0 + rb >= g.OH) ? g.H : (oh0 + rb) * g.sh;
    const int ow0 = SEG ? seg * wseg : 0, ow1 = (SEG && ow0 + wseg < g.OW) ? ow0 + wseg : g.OW;   // output columns [ow0, ow1)
    const int segw = ow1 - ow0;
    // input columns [iw_lo, iw_lo + wc) are held in LDS; [own_clo, own_chi) of them are this workgroup's to quantize
    int iw_lo = 0, wc = g.W, own_clo = 0, own_chi = g.W;
    if (SEG) {
        iw_lo = ow0 * g.sw - g.pw;
        iw_lo = iw_lo < 0 ? 0 : iw_lo;
        int iw_hi = (ow1 - 1) * g.sw - g.pw + (g.KW - 1) * g.dw + 1;
        iw_hi = iw_hi > g.W ? g.W : iw_hi;
        wc = iw_hi - iw_lo;
        own_clo = ow0 * g.sw;
        own_chi = ow1 == g.OW ? g.W : ow1 * g.sw;
    }
    const int pitch = g.C + 4;
    if (t >= nthreads) {
        // not taking part in the copy
    } else if (nthreads % g.C4 == 0) {
        // thread -> (pixel column, channel quad) once; then it walks down the rows and across the columns, sixteen
        // 16-byte loads in flight at a time.  The loads are unconditional (coordinates clamped into the image, the
        // result replaced by zeros afterwards) so that each store waits for its own load only.
        // A narrow image leaves most threads without a column: they then take further rows (rpar rows side by side).
        constexpr int kInFlight = 16;
        const int q = t % g.C4, wstep = nthreads / g.C4;
        const int rpar = wstep >= 2 * wc ? wstep / wc : 1;
        int w0 = t / g.C4, r0 = 0;
        if (rpar > 1) {
            r0 = w0 / wc;
            w0 = r0 < rpar ? w0 - r0 * wc : wc;   // threads beyond the last whole row: no column
        }
        const int wsteps = rpar > 1 ? 1 : (wc + wstep - 1) / wstep;
        const int iters = ((in_rows + rpar - 1) / rpar) * wsteps;
        const float *const xn = x + (int64_t)n * g.H * g.W * g.C + q * 4;
        int r_next = r0, ws_next = 0; // (row, column step) of the next item
        for (int it0 = 0; it0 < iters; it0 += kInFlight) {
            float4 v[kInFlight];
            int rr[kInFlight], ww[kInFlight];
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                rr[u] = r_next;
                ww[u] = w0 + ws_next * wstep;
                if (++ws_next == wsteps) {
                    ws_next = 0;
                    r_next += rpar;
                }
                int ih = ih_first + rr[u];
                ih = ih < 0 ? 0 : (ih >= g.H ? g.H - 1 : ih);
                const int wcl = iw_lo + (ww[u] < wc ? ww[u] : wc - 1);
                v[u] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                if (it0 + u < iters)   // the same for the whole workgroup: no load for items nobody has
                    v[u] = *reinterpret_cast<const float4 *>(xn + ((int64_t)ih * g.W + wcl) * g.C);
            }
#pragma unroll
            for (int u = 0; u < kInFlight; ++u) {
                const int ih = ih_first + rr[u];
                const bool in_image = (unsigned)ih < (unsigned)g.H;
                float4 f = fake_quant_value4(v[u], qt);
                if (!in_image)
                    f = make_float4(0.0f, 0.0f, 0.0f, 0.0f);   // rows outside the image are zeros
                if (it0 + u < iters && rr[u] < in_rows && ww[u] < wc) {
                    *reinterpret_cast<float4 *>(&rows[(rr[u] * wc + ww[u]) * pitch + q * 4]) = f;
                    const int iw = iw_lo + ww[u];
                    if (xq && in_image && ih >= own_lo && ih < own_hi && (!SEG || (iw >= own_clo && iw < own_chi)))
                        xq[(((int64_t)n * g.H + ih) * g.C4 + q) * g.W + iw] =
                            phys_row(quantize_code(f.x, qt.offset, qt.inv_scale)) |
                            (phys_row(quantize_code(f.y, qt.offset, qt.inv_scale)) << 8) |
                            (phys_row(quantize_code(f.z, qt.offset, qt.inv_scale)) << 16) |
                            (phys_row(quantize_code(f.w, qt.offset, qt.inv_scale)) << 24);
                }
            }
        }
    } else {
        const int quads_per_row = wc * g.C4;
        const int total = in_rows * quads_per_row;
        for (int i = t; i < total; i += nthreads) {
            const int r = i / quads_per_row, rem = i - r * quads_per_row;
            const int w = rem / g.C4, q = rem - w * g.C4;
            const int ih = ih_first + r;
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if ((unsigned)ih < (unsigned)g.H)
                v = fake_quant_value4(
                    *reinterpret_cast<const float4 *>(x + (((int64_t)n * g.H + ih) * g.W + iw_lo + w) * g.C + q * 4), qt);
            *reinterpret_cast<float4 *>(&rows[(r * wc + w) * pitch + q * 4]) = v;
        }
    }
    float *const zero_px = rows + (size_t)in_rows * wc * pitch; // one pixel of zeros behind the rows (see below)
    if (t < g.C4)
        *reinterpret_cast<float4 *>(zero_px + t * 4) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    __syncthreads();
    // Chains go to the wavefronts of the block starting from a different one in blocks that are likely to share a
    // CU (wavefronts of a block are spread over the SIMDs in order), so that their chains do not share a SIMD.
    const int rot = ((bid_in >> 8) + (bid_in >> 3)) & 3;
    const int tc = (t + (int)blockDim.x - rot * 64) % (int)blockDim.x;
    const int ohl = tc / segw, ow = ow0 + tc - ohl * segw;
    const int oh = oh0 + ohl;
    if (ohl >= rb) {
        // No chain for this thread.  If the launch asks for it, it packs filter codes meanwhile - but only from
        // wavefronts that share no SIMD with a chain (wavefront w of the block sits on SIMD w mod 4): a chain
        // runs as fast as its wavefront gets to issue, and any other work on its SIMD takes issue slots from it.
        const int chain_waves = (rb * segw + 63) / 64;
        const int wave = tc >> 6; // counted from the first chain wavefront
        if (fw.pack_total > 0 && (wave & 3) >= chain_waves) {
            const int waves = (int)blockDim.x >> 6;
            const int free_simds = 4 - chain_waves; // the launcher asks for this work only when chain_waves < 4
            const int workers = ((waves >> 2) * free_simds) * 64; // blockDim.x is 512 or 1024: 2 or 4 wavefronts per SIMD
            const int widx = (((wave >> 2) * free_simds + (wave & 3) - chain_waves) << 6) + (tc & 63);
            const int64_t share = (((fw.pack_total + nblocks - 1) / nblocks) + 63) & ~(int64_t)63;
            const int64_t first = (int64_t)bid_in * share;
            const int64_t last = first + share < fw.pack_total ? first + share : fw.pack_total;
            const TensorQuant qf = lq_dev ? lq_dev->flt : fw.tq;
            for (int64_t i = first + widx; i < last; i += workers)
                filter_pack_element(i, fw.filter, fw.filter_codes, fw.taps, fw.C, fw.C4, fw.Co, fw.nt,
                                    fw.n_col_tiles, qf, fw.wq);
        }
        return;
    }
    if (oh >= g.OH)
        return;
    const int iw0 = ow * g.sw - g.pw;
    float s = 0.0f;
    __builtin_amdgcn_s_setprio(3);   // the chain is the critical path: its wavefront issues ahead of the others on its SIMD
    const auto batched_chain = [&](auto batch_tag) {
        // The chain of K dependent adds is what takes the time here, so nothing else may wait on it: the taps and
        // their channels form one flat list of batches of 32 floats (16 where the channel quads are no multiple of 8), the LDS reads of a batch are issued a batch
        // ahead of its adds, and every lane takes every tap - a tap outside the image reads the pixel of zeros
        // (x + 0 == x; the sum starts at +0 and so is never -0) instead of branching around it.
        constexpr int kBatch = decltype(batch_tag)::value; // 16-byte reads per batch: 8, or 4 for 16 channels and the like
        const int bpt = g.C4 / kBatch, nb = g.KH * g.KW * bpt;
        int kh = 0, kw = 0, bi = 0;
        auto tap_src = [&]() -> const float4 * {
            const int iw = iw0 + kw * g.dw;
            const bool ok = kh < g.KH && (unsigned)iw < (unsigned)g.W;
            return reinterpret_cast<const float4 *>(ok ? rows + ((ohl * g.sh + kh * g.dh) * wc + iw - iw_lo) * pitch : zero_px);
        };
        const float4 *src = tap_src();
        auto read = [&](float4(&w)[kBatch]) {
#pragma unroll
            for (int i = 0; i < kBatch; ++i)
                w[i] = src[bi * kBatch + i];
            if (++bi == bpt) { // next tap (beyond the last one: the pixel of zeros, read but never added)
                bi = 0;
                if (++kw == g.KW) {
                    kw = 0;
                    ++kh;
                }
                src = tap_src();
            }
        };
        auto add = [&](const float4(&w)[kBatch]) {
#pragma unroll
            for (int i = 0; i < kBatch; ++i) {
                s = __fadd_rn(s, w[i].x);
                s = __fadd_rn(s, w[i].y);
                s = __fadd_rn(s, w[i].z);
                s = __fadd_rn(s, w[i].w);
            }
        };
        float4 w0[kBatch], w1[kBatch];
        read(w0);
        for (int b = 0; b < nb; b += 2) {
            // the scheduling fences keep each read behind the adds that free its registers: hoisted above them it
            // would need a third register set and a copy back at the end of every iteration
            read(w1);
            chain_fence(s);
            wait_lds_reads<kBatch>();
            add(w0);
            chain_fence(s);
            read(w0);
            chain_fence(s);
            wait_lds_reads<kBatch>();
            if (b + 1 < nb)
                add(w1);
            chain_fence(s);
        }
        psum[((int64_t)n * g.OH + oh) * g.OW + ow] = s;
    };
    if ((g.C4 & 7) == 0) {
        batched_chain(std::integral_constant<int, 8>());
        return;
    }
    if ((g.C4 & 3) == 0) {
        batched_chain(std::integral_constant<int, 4>());
        return;
    }
    for (int kh = 0; kh < g.KH; ++kh) {
        const int r = ohl * g.sh + kh * g.dh;        // LDS row of this tap; rows outside the image hold zeros,
        for (int kw = 0; kw < g.KW; ++kw) {          // and x + 0.0f == x, so they need no branch
            const int iw = iw0 + kw * g.dw;
            if ((unsigned)iw >= (unsigned)g.W)
                continue;
            const float *src = &rows[(r * wc + iw - iw_lo) * pitch];
#pragma unroll 8
            for (int q = 0; q < g.C4; ++q) {
                const float4 v = *reinterpret_cast<const float4 *>(src + q * 4);
                s = __fadd_rn(s, v.x);
                s = __fadd_rn(s, v.y);
                s = __fadd_rn(s, v.z);
                s = __fadd_rn(s, v.w);
            }
        }
    }
    psum[((int64_t)n * g.OH + oh) * g.OW + ow] = s;
}

// Patch sums for channel counts that are not a multiple of four (3-channel stems), same order and same results as
// patch_sums_kernel.  A block owns `rb` consecutive output rows of one image: it copies the input rows under them
// into LDS as they lie in memory (consecutive threads, consecutive floats), quantizes the rows it owns into the
// code layout when xq is given (same ownership rule as patch_sums_rows_body), and then runs one sequential chain
// per output pixel out of LDS, so every input float is fetched from memory about once instead of once per tap.
__global__ void __launch_bounds__(1024) patch_sums_smallc_kernel(const float *__restrict__ x, const ConvGeom g,
                                                                  const int rb, const int in_rows, const TensorQuant tq,
                                                                  const LayerQuant *__restrict__ lq_dev,
                                                                  float *__restrict__ psum, uint32_t *__restrict__ xq,
                                                                  const int flat_row_bytes, const int pad_left)
{
    // flat_row_bytes > 0: xq in the flat layout (see quantize_flat_rows_kernel), rows of that many bytes
    const TensorQuant qt = lq_dev ? lq_dev->in : tq;
    const int zp_row_dwords = flat_row_bytes ? flat_row_bytes / 4 : g.C4 * g.W;
    if (xq && blockIdx.x == 0)
        for (int i = threadIdx.x; i < zp_row_dwords; i += blockDim.x)
            xq[(int64_t)g.N * g.H * zp_row_dwords + i] = qt.zp4;
    extern __shared__ __align__(16) unsigned char ps_lds[];
    float *const rows = reinterpret_cast<float *>(ps_lds);
    const int t = threadIdx.x;
    const int bands = (g.OH + rb - 1) / rb;
    // consecutive bands (which share input rows) go to the same XCD: blocks are dealt round-robin over 8 XCDs
    const int nblocks = (int)gridDim.x;
    const int per_xcd = nblocks / 8, extra = nblocks % 8, xcd = (int)blockIdx.x & 7;
    const int bid = xcd * per_xcd + (xcd < extra ? xcd : extra) + ((int)blockIdx.x >> 3);
    const int n = bid / bands;
    const int oh0 = (bid - n * bands) * rb;
    const int ih_first = oh0 * g.sh - g.ph;  // input row held in LDS row 0 (may lie outside the image)
    const int row_floats = g.W * g.C;
    if ((row_floats & 3) == 0 && ((uintptr_t)x & 15) == 0) {   // rows of whole 16-byte pieces (3 x 224, 3 x 32 ...)
        const int row_quads = row_floats >> 2;
        for (int i = t; i < in_rows * row_quads; i += blockDim.x) {
            const int r = i / row_quads, e = i - r * row_quads;
            const int ih = ih_first + r;
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if ((unsigned)ih < (unsigned)g.H)
                v = fake_quant_value4(
                    *reinterpret_cast<const float4 *>(x + ((int64_t)n * g.H + ih) * row_floats + e * 4), qt);
            *reinterpret_cast<float4 *>(&rows[i * 4]) = v;
        }
    } else {
        for (int i = t; i < in_rows * row_floats; i += blockDim.x) {
            const int r = i / row_floats, e = i - r * row_floats;
            const int ih = ih_first + r;
            rows[i] = (unsigned)ih < (unsigned)g.H ? fake_quant_value(x[((int64_t)n * g.H + ih) * row_floats + e], qt) : 0.0f;
        }
    }
    __syncthreads();
    if (xq && flat_row_bytes) {
        const int own_lo = oh0 * g.sh;           // owned input rows: [own_lo, own_hi)
        const int own_hi = (oh0 + rb >= g.OH) ? g.H : (oh0 + rb) * g.sh;
        const int per_row = flat_row_bytes / 4;  // one dword of the flat row per step
        const uint32_t zp = qt.zp4 & 0xffu;
        for (int i = t; i < (own_hi - own_lo) * per_row; i += blockDim.x) {
            const int ro = i / per_row, d = i - ro * per_row;
            const int ih = own_lo + ro;
            const float *src = &rows[(ih - ih_first) * row_floats];
            uint32_t packed = 0;
            int px = (d * 4) / g.C, c = d * 4 - px * g.C;   // pixel and channel of the dword's first byte
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int w = px - pad_left;
                const uint32_t code = (unsigned)w < (unsigned)g.W
                                          ? phys_row(quantize_code(src[w * g.C + c], qt.offset, qt.inv_scale))
                                          : zp;
                packed |= code << (8 * k);
                if (++c == g.C) {
                    c = 0;
                    ++px;
                }
            }
            xq[((int64_t)n * g.H + ih) * per_row + d] = packed;
        }
    } else if (xq) {
        const int own_lo = oh0 * g.sh;           // owned input rows: [own_lo, own_hi)
        const int own_hi = (oh0 + rb >= g.OH) ? g.H : (oh0 + rb) * g.sh;
        const int per_row = g.C4 * g.W;
        for (int i = t; i < (own_hi - own_lo) * per_row; i += blockDim.x) {
            const int ro = i / per_row, rem = i - ro * per_row;
            const int c4 = rem / g.W, w = rem - c4 * g.W;
            const int ih = own_lo + ro;
            const float *src = &rows[(ih - ih_first) * row_floats + w * g.C + c4 * 4];
            uint32_t packed = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
                if (c4 * 4 + k < g.C)
                    packed |= phys_row(quantize_code(src[k], qt.offset, qt.inv_scale)) << (8 * k);
            xq[(((int64_t)n * g.H + ih) * g.C4 + c4) * g.W + w] = packed;
        }
    }
    const int ohl = t / g.OW, ow = t - ohl * g.OW;
    const int oh = oh0 + ohl;
    if (ohl >= rb || oh >= g.OH)
        return;
    const int iw0 = ow * g.sw - g.pw;
    float s = 0.0f;
    if (g.dw == 1) {
        // the taps of a filter row that lie inside the image are one run of floats, in the order of the chain
        const int lo = (iw0 < 0 ? 0 : iw0) * g.C, hi = (iw0 + g.KW < g.W ? iw0 + g.KW : g.W) * g.C;
        for (int kh = 0; kh < g.KH; ++kh) {
            const float *src = &rows[(ohl * g.sh + kh * g.dh) * row_floats];   // rows outside the image hold zeros
#pragma unroll 4
            for (int j = lo; j < hi; ++j)
                s = __fadd_rn(s, src[j]);
        }
        psum[((int64_t)n * g.OH + oh) * g.OW + ow] = s;
        return;
    }
    for (int kh = 0; kh < g.KH; ++kh) {
        const int r = ohl * g.sh + kh * g.dh;        // LDS row of this tap; rows outside the image hold zeros
        for (int kw = 0; kw < g.KW; ++kw) {
            const int iw = iw0 + kw * g.dw;
            if ((unsigned)iw >= (unsigned)g.W)
                continue;
            const float *src = &rows[r * row_floats + iw * g.C];
            for (int c = 0; c < g.C; ++c)
                s = __fadd_rn(s, src[c]);
        }
    }
    psum[((int64_t)n * g.OH + oh) * g.OW + ow] = s;
}

// Same relayout for caller-supplied codes (uint8 NHWC).
__global__ void __launch_bounds__(256) codes_relayout_kernel(const uint8_t *__restrict__ codes, int64_t pixels,
                                                              int W, int C, int C4, uint32_t *__restrict__ xq)
{
    const int64_t pix = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (pix >= pixels)
        return;
    const int w = (int)(pix % W);
    const int64_t nh = pix / W;
    const uint8_t *src = codes + pix * C;
    for (int c4 = 0; c4 < C4; ++c4) {
        uint32_t packed = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = c4 * 4 + i;
            if (c < C)
                packed |= phys_row(src[c]) << (8 * i);
        }
        xq[(nh * C4 + c4) * W + w] = packed;
    }
}

// Filter pre-pass: quantize (tf2/src/approx_nn_conv_kernels.cpp:243, hoisted out of the GEMM loop)
// and pack into the order the LUT-GEMM consumes.
//   wq[ct][fill][slot], fill = (tap * C4 + q) * SUBS + sub, slot = kk * NT + j
//   channel = q*4 + sub*KS + kk, column = ct*NT + j; kNullWeight where channel >= C or column >= Co.
// Element i of the packed filter [column tile][fill][slot]: the code of the filter element the slot stands for, the
// null weight where the slot is padding (i < column tiles x fills x 64).
__device__ __forceinline__ uint16_t filter_code_at(const int64_t i, const float *__restrict__ filter,
                                                   const uint8_t *__restrict__ filter_codes, int taps, int C, int C4,
                                                   int Co, int nt, const TensorQuant &qf)
{
    const int ks = 64 / nt, subs = 4 / ks;
    const int fills = taps * C4 * subs;
    const int slot = (int)(i & 63);
    const int64_t f = i >> 6;
    const int fill = (int)(f % fills);
    const int ct = (int)(f / fills);
    const int sub = fill % subs;
    const int tq = fill / subs;
    const int q = tq % C4;
    const int tap = tq / C4;
    const int kk = slot / nt, j = slot % nt;
    const int c = q * 4 + sub * ks + kk;
    const int col = ct * nt + j;
    uint16_t code = kNullWeight;
    if (c < C && col < Co) {
        const int64_t idx = ((int64_t)tap * C + c) * Co + col;
        code = filter_codes ? (uint16_t)filter_codes[idx]
                            : (uint16_t)quantize_code(fake_quant_value(filter[idx], qf), qf.offset, qf.inv_scale);
    }
    return code;
}

__device__ __forceinline__ void filter_pack_element(const int64_t i, const float *__restrict__ filter,
                                                    const uint8_t *__restrict__ filter_codes, int taps, int C,
                                                    int C4, int Co, int nt, int n_col_tiles, const TensorQuant &qf,
                                                    uint16_t *__restrict__ wq)
{
    const int64_t total = (int64_t)n_col_tiles * (taps * C4 * (nt / 16)) * 64;
    if (i < total)
        wq[i] = filter_code_at(i, filter, filter_codes, taps, C, C4, Co, nt, qf);
}

// Filter sums (tf2/src/approx_nn_conv_kernels.cpp:300-306): one sequential sum per output column, rows (h, w, c)
// ascending.  The chain of K dependent adds sets the time, so everything else is kept off it, and memory latency
// is covered by volume in flight: a block owns only kFsCols columns (64-byte pieces of filter rows), which leaves
// each of its loads a whole row of lead.  It walks the filter rows in passes of kFsRows: all its threads (512 or
// 1024) load a pass kFsAhead passes ahead of its use and store it into one half of an LDS stage; meanwhile the
// first kFsCols lanes extend the sums from the other half.  A lone wavefront issues about one instruction every
// four cycles whatever its kind, so the stage is column-major and a lane fetches four rows per LDS read, one batch
// of 16 rows ahead of the adds: 21 instructions per 16 adds.  One barrier per pass.  Rows beyond K are staged as zeros and summed like the others: the sums start at +0 and
// so are never -0, and x + 0 == x.
constexpr int kFsCols = 16, kFsRows = 256, kFsPitch = kFsRows + 4, kFsAhead = 3, kFsThreads = 1024;
constexpr int kFsLdsBytes = 2 * kFsCols * kFsPitch * 4; // 32.5 KiB: two halves of [column][row], rows padded by 4

extern __shared__ __align__(16) unsigned char fs_lds[];

template <int THREADS>
__device__ __forceinline__ void filter_sums_block(const int block, const float *__restrict__ filter, int K, int Co,
                                                  const TensorQuant &q, float *__restrict__ fsum)
{
    constexpr int kBatch = 16, kStep = THREADS / kFsCols, kPer = kFsRows / kStep; // loads per thread per pass
    float *const stage = reinterpret_cast<float *>(fs_lds);
    const int col0 = block * kFsCols;
    const int t = threadIdx.x;
    const int cl = t % kFsCols, rsub = t / kFsCols;
    const bool col_ok = col0 + cl < Co;
    const float *const src = filter + (col_ok ? col0 + cl : Co - 1);
    const int npass = (K + kFsRows - 1) / kFsRows;
    // Loads and stores below are unconditional (rows beyond K load row K - 1 and are stored as zeros, passes beyond
    // the last likewise), so that the loop body is straight-line code for the compiler's count of loads in flight:
    // a store then waits for its own pass only, not for the passes issued after it.
    float v[kFsAhead][kPer];
    auto issue = [&](float(&dst)[kPer], int pass) {
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int k = pass * kFsRows + rsub + i * kStep;
            dst[i] = src[(int64_t)(k < K ? k : K - 1) * Co];
        }
    };
    auto store = [&](const float(&from)[kPer], int pass) {
        float *const half = stage + (pass & 1) * (kFsCols * kFsPitch);
#pragma unroll
        for (int i = 0; i < kPer; ++i) {
            const int r = rsub + i * kStep;
            float f = from[i];
            if (q.fq)
                f = fake_quant_value(f, q);
            half[cl * kFsPitch + r] = (pass * kFsRows + r < K) ? f : 0.0f;
        }
    };
#pragma unroll
    for (int u = 0; u < kFsAhead; ++u)
        issue(v[u], u);
    store(v[0], 0);
    issue(v[0], kFsAhead);
    __syncthreads();
    float s = 0.0f;
    __builtin_amdgcn_s_setprio(3);   // the chain is the critical path: its wavefront issues ahead of the others on its SIMD
    // one pass: `next` holds pass p + 1 (stored now, then refilled with the loads of pass p + 1 + kFsAhead);
    // pass p lies in its half of the stage
    auto pass_step = [&](const int p, float(&next)[kPer]) {
        store(next, p + 1);
        issue(next, p + 1 + kFsAhead);
        if (t < kFsCols && p < npass) {
            const float4 *const half = reinterpret_cast<const float4 *>(stage + (p & 1) * (kFsCols * kFsPitch) + t * kFsPitch);
            const int left = K - p * kFsRows;
            const int nb = left >= kFsRows ? kFsRows / kBatch : (left + kBatch - 1) / kBatch;
            float4 w0[kBatch / 4], w1[kBatch / 4];
            auto read = [&](float4(&w)[kBatch / 4], int b) {
#pragma unroll
                for (int i = 0; i < kBatch / 4; ++i)
                    w[i] = half[b * (kBatch / 4) + i];
            };
            auto add = [&](const float4(&w)[kBatch / 4]) {
#pragma unroll
                for (int i = 0; i < kBatch / 4; ++i) {
                    s = __fadd_rn(s, w[i].x);
                    s = __fadd_rn(s, w[i].y);
                    s = __fadd_rn(s, w[i].z);
                    s = __fadd_rn(s, w[i].w);
                }
            };
            read(w0, 0);
            for (int b = 0; b < nb; b += 2) { // nb is even or 1; reads beyond the pass's rows stay inside the stage
                read(w1, b + 1);
                chain_fence(s);
                wait_lds_reads<kBatch / 4>();
                add(w0);
                chain_fence(s);
                read(w0, b + 2 < kFsRows / kBatch ? b + 2 : 0);
                chain_fence(s);
                wait_lds_reads<kBatch / 4>();
                if (b + 1 < nb)
                    add(w1);
                chain_fence(s);
            }
        }
        __syncthreads();
    };
    static_assert(kFsAhead == 3, "the pass loop below rotates three register sets");
    for (int p0 = 0; p0 < npass; p0 += kFsAhead) {
        pass_step(p0, v[1]);
        pass_step(p0 + 1, v[2]);
        pass_step(p0 + 2, v[0]);
    }
    if (t < kFsCols && col_ok)
        fsum[col0 + t] = s;
}

// One launch for the whole filter pre-pass: the first sum_blocks workgroups compute the column sums (skipped when
// fsum is null), the others pack the codes.
// One (column tile, pair of fills) of the pre-expanded rows (px_expand.h) by a workgroup of 4 * CB threads that is
// not the one that packs the pair's filter codes: it computes the 128 codes itself, into LDS behind the stage.
template <int CB>
__device__ __forceinline__ void px_expand_own_codes(const int eb, const float *__restrict__ filter,
                                                    const uint8_t *__restrict__ filter_codes, int taps, int C, int C4,
                                                    int Co, const TensorQuant &q, const uint16_t *__restrict__ tableT,
                                                    uint16_t *__restrict__ px_rows)
{
    extern __shared__ __align__(16) unsigned char px_lds[];
    uint32_t *const stage = reinterpret_cast<uint32_t *>(px_lds);
    constexpr int kParts = 256 / CB;
    const int fills = taps * C4, px_fills = fills / 2;   // 16-column tiles: a fill is one channel quad of a tap
    const int part = eb % kParts, cf = eb / kParts;      // cf = ct * px_fills + f
    const int ct = cf / px_fills, f = cf - ct * px_fills;
    uint16_t *const codes = reinterpret_cast<uint16_t *>(stage + px_expand_stage_dwords<CB>());
    if (threadIdx.x < 128)
        codes[threadIdx.x] = filter_code_at(((int64_t)ct * fills + 2 * (int64_t)f) * 64 + threadIdx.x, filter, filter_codes,
                                            taps, C, C4, Co, 16, q);
    __syncthreads();
    px_expand_part<CB>(stage, part, [&](const int sl) { return codes[sl]; }, tableT,
                       reinterpret_cast<uint32_t *>(px_rows + (size_t)cf * (kPxFillBytes / 2)));
}

// One launch for the whole filter pre-pass: the first sum_blocks workgroups compute the column sums (skipped when
// fsum is null), the next pack_blocks pack the codes, any further ones build pre-expanded rows.
__global__ void __launch_bounds__(kFsThreads) filter_prep_kernel(const float *__restrict__ filter,
                                                                  const uint8_t *__restrict__ filter_codes, int taps,
                                                                  int C, int C4, int Co, int nt, int n_col_tiles,
                                                                  const TensorQuant tq,
                                                                  const LayerQuant *__restrict__ lq_dev,
                                                                  uint16_t *__restrict__ wq, int sum_blocks,
                                                                  float *__restrict__ fsum, int pack_blocks,
                                                                  const uint16_t *__restrict__ tableT,
                                                                  uint16_t *__restrict__ px_rows)
{
    const TensorQuant q = lq_dev ? lq_dev->flt : tq;
    if ((int)blockIdx.x < sum_blocks) {
        filter_sums_block<kFsThreads>((int)blockIdx.x, filter, taps * C, Co, q, fsum);
        return;
    }
    const int pb = (int)blockIdx.x - sum_blocks;
    if (pb < pack_blocks) {
        const int64_t i = (int64_t)pb * blockDim.x + threadIdx.x;
        filter_pack_element(i, filter, filter_codes, taps, C, C4, Co, nt, n_col_tiles, q, wq);
        return;
    }
    px_expand_own_codes<kFsThreads / 4>(pb - pack_blocks, filter, filter_codes, taps, C, C4, Co, q, tableT, px_rows);
}

// Patch sums of a 1x1, stride-1, unpadded layer: the patch of an output pixel is the pixel itself, so the pixels
// of the whole batch form one flat list and no window or halo exists.  A workgroup takes up to kFlatPixels consecutive
// pixels and walks their channels in chunks of kFlatChunk: all threads copy a chunk into LDS (and quantize it
// into the code layout on the way, when xq is given), then one thread per pixel extends its sequential sum by the
// chunk's channels.  With many channels this keeps 256 sums going per workgroup where a band of image rows in
// LDS would hold one row's worth.  The loads of the next chunk are in flight while the current one is summed.
constexpr int kFlatPixels = 256, kFlatChunk = 64, kFlatThreads = 512;
constexpr int kFlatPitch = kFlatChunk + 4;                         // floats per pixel in LDS
constexpr int kFlatPer = kFlatPixels * (kFlatChunk / 4) / kFlatThreads; // 16-byte loads per thread and chunk

__device__ __forceinline__ void patch_sums_flat_body(const float *__restrict__ x, const ConvGeom &g,
                                                     const TensorQuant &tq, const LayerQuant *__restrict__ lq_dev,
                                                     float *__restrict__ psum, uint32_t *__restrict__ xq,
                                                     const int bid, const int pixels)
{
    // pixels: pixels per workgroup, 64 / 128 / 256 (fewer when the layer has few pixels, for enough workgroups)
    const TensorQuant qt = lq_dev ? lq_dev->in : tq;
    if (xq && bid == 0)
        for (int i = threadIdx.x; i < g.C4 * g.W; i += blockDim.x)
            xq[(int64_t)g.N * g.H * g.C4 * g.W + i] = qt.zp4;
    extern __shared__ __align__(16) unsigned char pf_lds[];
    float *const rows = reinterpret_cast<float *>(pf_lds);
    const int t = threadIdx.x;
    const int64_t m0 = (int64_t)bid * pixels;
    const int npx = (int)(g.M - m0 < pixels ? g.M - m0 : pixels);
    // thread -> (channel quad of the chunk, pixel) once: quad q of pixels px0, px0 + 32, ...
    constexpr int QUADS = kFlatChunk / 4, PSTEP = kFlatThreads / QUADS;
    const int q = t % QUADS, px0 = t / QUADS;
    const bool copier = t < kFlatThreads;
    int64_t x_idx[kFlatPer];          // float index in x of (pixel, quad q of chunk 0)
#pragma unroll
    for (int k = 0; k < kFlatPer; ++k) {
        const int px = px0 + k * PSTEP;    // k beyond pixels / PSTEP: px >= npx, nothing loaded or stored
        const int64_t m = m0 + (px < npx ? px : 0);
        x_idx[k] = m * g.C + q * 4;
    }
    // ... and thread -> (pixel, first quad) for the codes: pixel t % pixels, quads t / pixels, + kFlatThreads / pixels, ...
    const int code_px = t % pixels, code_q0 = t / pixels, code_qstep = kFlatThreads / pixels;
    uint32_t code_idx = 0;            // dword index in xq of (that pixel, quad 0)
    {
        const int64_t m = m0 + (code_px < npx ? code_px : 0);
        const int64_t nh = m / g.W;
        code_idx = (uint32_t)(nh * g.C4 * g.W + (m - nh * g.W));
    }
    const int chunks = (g.C + kFlatChunk - 1) / kFlatChunk;
    float4 v[kFlatPer];
    auto load_chunk = [&](int c0) {
#pragma unroll
        for (int k = 0; k < kFlatPer; ++k) {
            v[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (copier && px0 + k * PSTEP < npx && c0 + q * 4 < g.C)
                v[k] = *reinterpret_cast<const float4 *>(x + x_idx[k] + c0);
        }
    };
    load_chunk(0);
    float s = 0.0f;
    __builtin_amdgcn_s_setprio(3);   // the chain is the critical path: its wavefront issues ahead of the others on its SIMD
    for (int ch = 0; ch < chunks; ++ch) {
        const int c0 = ch * kFlatChunk;
        if (copier) {
#pragma unroll
            for (int k = 0; k < kFlatPer; ++k) {
                const int px = px0 + k * PSTEP;
                if (px >= pixels)
                    continue;
                *reinterpret_cast<float4 *>(&rows[px * kFlatPitch + q * 4]) = fake_quant_value4(v[k], qt);
            }
        }
        __syncthreads();
        if (ch + 1 < chunks)
            load_chunk(c0 + kFlatChunk);
        if (xq && copier && code_px < npx) {
            // The codes go out of LDS, not out of the registers the floats came in: there a wavefront holds 16 quads
            // of 4 pixels, and a quad's codes lie a row of W dwords apart in xq - 16 runs of 16 bytes per store;
            // here it holds one quad of 64 consecutive pixels: one run of 256 bytes.
            const int nq = (g.C - c0 < kFlatChunk ? g.C - c0 : kFlatChunk) / 4;
            for (int qq = code_q0; qq < nq; qq += code_qstep) {
                const float4 f = *reinterpret_cast<const float4 *>(&rows[code_px * kFlatPitch + qq * 4]);
                xq[code_idx + (uint32_t)(c0 / 4 + qq) * (uint32_t)g.W] =
                    phys_row(quantize_code(f.x, qt.offset, qt.inv_scale)) |
                    (phys_row(quantize_code(f.y, qt.offset, qt.inv_scale)) << 8) |
                    (phys_row(quantize_code(f.z, qt.offset, qt.inv_scale)) << 16) |
                    (phys_row(quantize_code(f.w, qt.offset, qt.inv_scale)) << 24);
            }
        }
        if (t < npx) {
            const int nq = (g.C - c0 < kFlatChunk ? g.C - c0 : kFlatChunk) / 4;
            const float *src = &rows[t * kFlatPitch];
#pragma unroll 8
            for (int qq = 0; qq < nq; ++qq) {
                const float4 f = *reinterpret_cast<const float4 *>(src + qq * 4);
                s = __fadd_rn(s, f.x);
                s = __fadd_rn(s, f.y);
                s = __fadd_rn(s, f.z);
                s = __fadd_rn(s, f.w);
            }
        }
        __syncthreads();
    }
    if (t < npx)
        psum[m0 + t] = s;
}

// The flat pixel list with many channels and few pixels (the deep, small layers of a network): there the chain of
// C dependent adds per pixel is what takes the time, and memory latency has to stay off it.  A workgroup takes
// `pixels` (8 or 16) consecutive pixels, so that even a few thousand pixels spread over all CUs, and walks their
// channels in passes of kDeepChunk: all threads load a pass kDeepAhead passes ahead of its use (16 bytes per lane,
// a wavefront fetches 1 KiB of one pixel), quantize it into the code layout when xq is given and store it into
// one half of an LDS stage [pixel][channel]; meanwhile one lane per pixel extends its sum from the other half,
// its 16-byte LDS reads a batch of 32 channels ahead of the adds.  One barrier per pass.  Loads, stores and LDS
// reads are unconditional (indices clamped, zeros stored beyond C) to keep the loop body straight-line code for
// the compiler's count of loads in flight: a store then waits for its own pass only.
constexpr int kDeepChunk = 256, kDeepPitch = kDeepChunk + 4, kDeepAhead = 3, kDeepThreads = 512;
constexpr int deep_lds_bytes(int pixels) { return 2 * pixels * kDeepPitch * 4; }

template <int PIXELS>
__device__ __forceinline__ void patch_sums_deep_body(const float *__restrict__ x, const ConvGeom &g,
                                                     const TensorQuant &tq, const LayerQuant *__restrict__ lq_dev,
                                                     float *__restrict__ psum, uint32_t *__restrict__ xq,
                                                     const int bid)
{
    constexpr int pixels = PIXELS, kDeepMaxPixels = PIXELS;
    constexpr int kDeepPer = PIXELS * (kDeepChunk / 4) / kDeepThreads; // 16-byte loads per thread and pass
    const TensorQuant qt = lq_dev ? lq_dev->in : tq;
    if (xq && bid == 0)
        for (int i = threadIdx.x; i < g.C4 * g.W; i += blockDim.x)
            xq[(int64_t)g.N * g.H * g.C4 * g.W + i] = qt.zp4;
    extern __shared__ __align__(16) unsigned char pd_lds[];
    float *const stage = reinterpret_cast<float *>(pd_lds);
    const int t = threadIdx.x;
    const int64_t m0 = (int64_t)bid * pixels;
    const int npx = (int)(g.M - m0 < pixels ? g.M - m0 : pixels);
    constexpr int QUADS = kDeepChunk / 4, PSTEP = kDeepThreads / QUADS;
    const int q = t % QUADS, px0 = t / QUADS;
    const bool loader = t < kDeepThreads;
    const int npass = (g.C + kDeepChunk - 1) / kDeepChunk;
    const float *src[kDeepPer];
    uint32_t xq_idx[kDeepPer];
    bool px_ok[kDeepPer];
#pragma unroll
    for (int k = 0; k < kDeepPer; ++k) {
        const int px = px0 + k * PSTEP;
        px_ok[k] = loader && px < npx;
        const int64_t m = m0 + (px < npx ? px : npx - 1);
        const int64_t nh = m / g.W;
        const int w = (int)(m - nh * g.W);
        xq_idx[k] = (uint32_t)((nh * g.C4 + q) * g.W + w);
        src[k] = x + m * g.C;
    }
    float4 v[kDeepAhead][kDeepPer];
    auto issue = [&](float4(&dst)[kDeepPer], int pass) {
        const int c = pass * kDeepChunk + q * 4;
        const int cc = c < g.C ? c : g.C - 4;
#pragma unroll
        for (int k = 0; k < kDeepPer; ++k)
            dst[k] = *reinterpret_cast<const float4 *>(src[k] + cc);
    };
    auto store = [&](const float4(&from)[kDeepPer], int pass) {
        float *const half = stage + (pass & 1) * (kDeepMaxPixels * kDeepPitch);
        const bool c_ok = pass * kDeepChunk + q * 4 < g.C;
#pragma unroll
        for (int k = 0; k < kDeepPer; ++k) {
            const int px = px0 + k * PSTEP;
            float4 f = fake_quant_value4(from[k], qt);
            if (!c_ok)
                f = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (loader && px < kDeepMaxPixels)
                *reinterpret_cast<float4 *>(&half[px * kDeepPitch + q * 4]) = f;
            if (xq && px_ok[k] && c_ok)
                xq[xq_idx[k] + (uint32_t)(pass * (kDeepChunk / 4)) * (uint32_t)g.W] =
                    phys_row(quantize_code(f.x, qt.offset, qt.inv_scale)) |
                    (phys_row(quantize_code(f.y, qt.offset, qt.inv_scale)) << 8) |
                    (phys_row(quantize_code(f.z, qt.offset, qt.inv_scale)) << 16) |
                    (phys_row(quantize_code(f.w, qt.offset, qt.inv_scale)) << 24);
        }
    };
#pragma unroll
    for (int u = 0; u < kDeepAhead; ++u)
        issue(v[u], u);
    store(v[0], 0);
    if (kDeepAhead < npass)
        issue(v[0], kDeepAhead);
    __syncthreads();
    float s = 0.0f;
    __builtin_amdgcn_s_setprio(3);   // the chain is the critical path: its wavefront issues ahead of the others on its SIMD
    constexpr int kBatch = 8, kBatches = QUADS / kBatch; // 16-byte reads per batch; batches per pass
    auto pass_step = [&](const int p, float4(&next)[kDeepPer]) {
        store(next, p + 1);
        if (p + 1 + kDeepAhead < npass)
            issue(next, p + 1 + kDeepAhead);
        if (t < kDeepMaxPixels && p < npass) {
            const float4 *const row =
                reinterpret_cast<const float4 *>(stage + (p & 1) * (kDeepMaxPixels * kDeepPitch) + t * kDeepPitch);
            float4 w0[kBatch], w1[kBatch];
            auto read = [&](float4(&w)[kBatch], int b) {
#pragma unroll
                for (int i = 0; i < kBatch; ++i)
                    w[i] = row[b * kBatch + i];
            };
            auto add = [&](const float4(&w)[kBatch]) {
#pragma unroll
                for (int i = 0; i < kBatch; ++i) {
                    s = __fadd_rn(s, w[i].x);
                    s = __fadd_rn(s, w[i].y);
                    s = __fadd_rn(s, w[i].z);
                    s = __fadd_rn(s, w[i].w);
                }
            };
            read(w0, 0);
#pragma unroll
            for (int b = 0; b < kBatches; b += 2) {
                read(w1, b + 1);
                chain_fence(s);
                wait_lds_reads<kBatch>();
                add(w0);
                chain_fence(s);
                if (b + 2 < kBatches)
                    read(w0, b + 2);
                chain_fence(s);
                if (b + 2 < kBatches)
                    wait_lds_reads<kBatch>();
                else
                    wait_lds_reads<0>();
                add(w1);
                chain_fence(s);
            }
        }
        __syncthreads();
    };
    static_assert(kDeepAhead == 3, "the pass loop below rotates three register sets");
    for (int p0 = 0; p0 < npass; p0 += kDeepAhead) {
        pass_step(p0, v[1]);
        pass_step(p0 + 1, v[2]);
        pass_step(p0 + 2, v[0]);
    }
    if (t < npx)
        psum[m0 + t] = s;
}

// The filter work of a patch-sum launch: true if this workgroup is one of those that do it (and has done it), else
// *bid is its index among the patch-sum workgroups.
__device__ __forceinline__ bool filter_work_block(const FilterWork &fw, const LayerQuant *__restrict__ lq_dev, int *bid)
{
    const int b = (int)blockIdx.x;
    if (b < fw.sum8) {
        if (b < fw.sum_blocks) { // the launcher gives these workgroups 512 or 1024 threads
            const TensorQuant q = lq_dev ? lq_dev->flt : fw.tq;
            if (blockDim.x == 512)
                filter_sums_block<512>(b, fw.filter, fw.taps * fw.C, fw.Co, q, fw.fsum);
            else
                filter_sums_block<1024>(b, fw.filter, fw.taps * fw.C, fw.Co, q, fw.fsum);
        }
        return true;
    }
    *bid = b - fw.sum8;
    if (*bid < fw.work_blocks)
        return false;
    const TensorQuant q = lq_dev ? lq_dev->flt : fw.tq;
    const int pb = *bid - fw.work_blocks;
    if (pb < fw.pack_blocks || fw.expand_blocks == 0) {
        const int64_t i = (int64_t)pb * blockDim.x + threadIdx.x;
        filter_pack_element(i, fw.filter, fw.filter_codes, fw.taps, fw.C, fw.C4, fw.Co, fw.nt, fw.n_col_tiles, q, fw.wq);
        return true;
    }
    // pre-expanded rows: blockDim.x / 4 activation codes of a pair of fills per workgroup
    const int eb = pb - fw.pack_blocks;
    if (blockDim.x == 512)
        px_expand_own_codes<128>(eb, fw.filter, fw.filter_codes, fw.taps, fw.C, fw.C4, fw.Co, q, fw.tableT, fw.px_rows);
    else
        px_expand_own_codes<256>(eb, fw.filter, fw.filter_codes, fw.taps, fw.C, fw.C4, fw.Co, q, fw.tableT, fw.px_rows);
    return true;
}

// Bands cut into column segments: a kernel of its own, so that the common variants below stay as small as they were.
__global__ void __launch_bounds__(1024) patch_sums_segments_kernel(const float *__restrict__ x, const ConvGeom g,
                                                                    int rb, int in_rows, int nthreads, int wseg,
                                                                    const TensorQuant tq,
                                                                    const LayerQuant *__restrict__ lq_dev,
                                                                    float *__restrict__ psum, uint32_t *__restrict__ xq,
                                                                    const FilterWork fw)
{
    int bid;
    if (filter_work_block(fw, lq_dev, &bid))
        return;
    patch_sums_rows_body<true>(x, g, rb, in_rows, wseg, tq, lq_dev, psum, xq, bid, fw.work_blocks, nthreads, fw);
}

__global__ void __launch_bounds__(1024) patch_sums_rows_kernel(const float *__restrict__ x, const ConvGeom g, int rb,
                                                                int in_rows, int nthreads, const TensorQuant tq,
                                                                const LayerQuant *__restrict__ lq_dev,
                                                                float *__restrict__ psum, uint32_t *__restrict__ xq,
                                                                const FilterWork fw)
{
    int bid;
    if (filter_work_block(fw, lq_dev, &bid))
        return;
    if (rb < 0) { // 1x1, stride 1, many channels, few pixels
        if (in_rows == 8)
            patch_sums_deep_body<8>(x, g, tq, lq_dev, psum, xq, bid);
        else
            patch_sums_deep_body<16>(x, g, tq, lq_dev, psum, xq, bid);
        return;
    }
    if (rb == 0) { // 1x1, stride 1: flat pixel list
        patch_sums_flat_body(x, g, tq, lq_dev, psum, xq, bid, in_rows);
        return;
    }
    patch_sums_rows_body<false>(x, g, rb, in_rows, g.OW, tq, lq_dev, psum, xq, bid, fw.work_blocks, nthreads, fw);
}

__global__ void __launch_bounds__(256) quantize_flat_kernel(const float *__restrict__ v, int64_t n, float offset,
                                                             float inv_scale, uint8_t *__restrict__ codes)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        codes[i] = (uint8_t)quantize_code(v[i], offset, inv_scale);
}

// Depthwise filter pre-pass: codes [taps][C] and per-channel sums (taps ascending).
__global__ void __launch_bounds__(256) depthwise_filter_kernel(const float *__restrict__ filter, int taps, int C,
                                                                const TensorQuant tq,
                                                                const LayerQuant *__restrict__ lq_dev,
                                                                uint8_t *__restrict__ wcodes,
                                                                float *__restrict__ fsum)
{
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C)
        return;
    const TensorQuant q = lq_dev ? lq_dev->flt : tq;
    float s = 0.0f;
    for (int t = 0; t < taps; ++t) {
        const float v = fake_quant_value(filter[(int64_t)t * C + c], q);
        s = __fadd_rn(s, v);
        wcodes[(int64_t)t * C + c] = (uint8_t)quantize_code(v, q.offset, q.inv_scale);
    }
    fsum[c] = s;
}

static inline unsigned blocks_for(int64_t n, int threads) { return (unsigned)((n + threads - 1) / threads); }

// The extra [C4][W] row behind xq: every dword is the zero-point code x4.
__global__ void __launch_bounds__(256) fill_u32_kernel(uint32_t *__restrict__ dst, int n, uint32_t value)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n)
        dst[i] = value;
}

// ---- the Keras layer's pre-step: per-tensor min / max and the quantization constants, all on the device ----
// (tf2/python/keras/layers/fake_approx_convolutional.py:233-242: reduce_min / reduce_max of the batch and of
// the kernel, then fake quantization with them.)  Stage 1: one (min, max) pair per workgroup.
// The first blocks_a workgroups reduce tensor a, the others tensor b (one launch for the input and the filter).
__global__ void __launch_bounds__(256) minmax_partial_kernel(const float *__restrict__ a, int64_t na, int blocks_a,
                                                              const float *__restrict__ b, int64_t nb,
                                                              float *__restrict__ partials)
{
    __shared__ float smin[256], smax[256];
    const bool second = (int)blockIdx.x >= blocks_a;
    const float *__restrict__ v = second ? b : a;
    const int64_t n = second ? nb : na;
    const int block = second ? (int)blockIdx.x - blocks_a : (int)blockIdx.x;
    const int nblocks = second ? (int)gridDim.x - blocks_a : blocks_a;
    partials += second ? 2 * kMinMaxBlocks : 0;
    float lo = INFINITY, hi = -INFINITY;
    const int64_t stride = (int64_t)nblocks * blockDim.x;
    const int64_t tid = (int64_t)block * blockDim.x + threadIdx.x;
    int64_t done = 0;
    if (((uintptr_t)v & 15) == 0) { // 16 bytes per lane while they last, the remainder one float at a time
        const float4 *v4 = reinterpret_cast<const float4 *>(v);
        const int64_t n4 = n / 4;
        for (int64_t i = tid; i < n4; i += stride) {
            const float4 x = v4[i];
            lo = fminf(fminf(lo, x.x), fminf(fminf(x.y, x.z), x.w));
            hi = fmaxf(fmaxf(hi, x.x), fmaxf(fmaxf(x.y, x.z), x.w));
        }
        done = n4 * 4;
    }
    for (int64_t i = done + tid; i < n; i += stride) {
        const float x = v[i];
        lo = fminf(lo, x);
        hi = fmaxf(hi, x);
    }
    smin[threadIdx.x] = lo;
    smax[threadIdx.x] = hi;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            smin[threadIdx.x] = fminf(smin[threadIdx.x], smin[threadIdx.x + s]);
            smax[threadIdx.x] = fmaxf(smax[threadIdx.x], smax[threadIdx.x + s]);
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partials[2 * block] = smin[0];
        partials[2 * block + 1] = smax[0];
    }
}

// Nudge + UpdateVarQuantProps (tf2/src/approx_ops_types.h:29-49,135-152) for one tensor, every operation rounded
// on its own like the host code of axc_quant_props_compute.
__device__ void tensor_quant_device(float mn, float mx, TensorQuant *t, int *zero_point)
{
    t->fq = 1u;
    t->zp4 = 0u;
    *zero_point = 0;
    if (mn == 0.0f && mx == 0.0f) {
        t->offset = t->inv_scale = t->scale = t->nudged_max = 0.0f;
        return;
    }
    const float sc = __fdiv_rn(__fsub_rn(mx, mn), 255.0f);
    const float zp_from_min = __fsub_rn(0.0f, __fdiv_rn(mn, sc));
    int zp;
    if (zp_from_min < 0.0f)
        zp = 0;
    else if (zp_from_min > 255.0f)
        zp = 255;
    else
        zp = (int)(uint16_t)roundf(zp_from_min);
    t->scale = sc;
    t->offset = __fmul_rn(__fsub_rn(0.0f, (float)zp), sc);
    t->nudged_max = __fmul_rn(__fsub_rn(255.0f, (float)zp), sc);
    t->inv_scale = __fdiv_rn(1.0f, sc);
    *zero_point = zp;
}

// Stage 2: one workgroup folds the partial pairs of both tensors and writes the layer's constants.
__global__ void __launch_bounds__(256) layer_quant_kernel(const float *__restrict__ partials, int n_in, int n_flt,
                                                           int K, LayerQuant *__restrict__ out)
{
    __shared__ float red[4][256];
    float v[4] = {INFINITY, -INFINITY, INFINITY, -INFINITY};
    for (int i = threadIdx.x; i < n_in; i += 256) {
        v[0] = fminf(v[0], partials[2 * i]);
        v[1] = fmaxf(v[1], partials[2 * i + 1]);
    }
    const float *pf = partials + 2 * kMinMaxBlocks;
    for (int i = threadIdx.x; i < n_flt; i += 256) {
        v[2] = fminf(v[2], pf[2 * i]);
        v[3] = fmaxf(v[3], pf[2 * i + 1]);
    }
    for (int k = 0; k < 4; ++k)
        red[k][threadIdx.x] = v[k];
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s)
            for (int k = 0; k < 4; ++k)
                red[k][threadIdx.x] = (k & 1) ? fmaxf(red[k][threadIdx.x], red[k][threadIdx.x + s])
                                              : fminf(red[k][threadIdx.x], red[k][threadIdx.x + s]);
        __syncthreads();
    }
    if (threadIdx.x != 0)
        return;
    LayerQuant lq;
    int zp_in = 0, zp_f = 0;
    tensor_quant_device(red[0][0], red[1][0], &lq.in, &zp_in);
    tensor_quant_device(red[2][0], red[3][0], &lq.flt, &zp_f);
    // the code the op gives 0.0f (what taps outside the image look up): its own quantize expression
    lq.in.zp4 = phys_row(quantize_code(0.0f, lq.in.offset, lq.in.inv_scale)) * 0x01010101u;
    // approx_ops_types.h:184-187
    lq.s1xs2 = __fmul_rn(lq.in.scale, lq.flt.scale);
    lq.m1 = lq.in.offset;
    lq.m2 = lq.flt.offset;
    lq.k_m1xm2 = __fmul_rn((float)K, __fmul_rn(lq.in.offset, lq.flt.offset));
    *out = lq;
}

hipError_t launch_layer_quant(const float *input, int64_t n_input, const float *filter, int64_t n_filter, int K,
                              float *partials, LayerQuant *lq_dev, hipStream_t stream)
{
    auto blocks = [](int64_t n) {
        const int64_t b = (n + 256 * 32 - 1) / (256 * 32);
        return (int)(b < 1 ? 1 : (b > kMinMaxBlocks ? kMinMaxBlocks : b));
    };
    const int b_in = blocks(n_input), b_f = blocks(n_filter);
    hipLaunchKernelGGL(minmax_partial_kernel, dim3(b_in + b_f), dim3(256), 0, stream, input, n_input, b_in, filter,
                       n_filter, partials);
    hipLaunchKernelGGL(layer_quant_kernel, dim3(1), dim3(256), 0, stream, partials, b_in, b_f, K, lq_dev);
    return hipGetLastError();
}

// ---- integer zero-point correction of the tf1 AxConv2D op (tf1/axqconv/axqconv.cc:228-247) ----
// total = sum(T[a][b] - a*offset_filter - b*offset_input + offset_input*offset_filter) over the patch, where a tap
// outside the image has a = offset_input.  The LUT-GEMM gives sum(T); these kernels give sum(a) per output pixel and
// sum(b) per output column, and the last one combines them.
__global__ void __launch_bounds__(256) code_patch_sums_kernel(const uint8_t *__restrict__ codes, ConvGeom g,
                                                               int offset_input, int32_t *__restrict__ asum)
{
    const int64_t m = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= g.M)
        return;
    const int n = (int)(m / ((int64_t)g.OH * g.OW));
    const int rem = (int)(m - (int64_t)n * g.OH * g.OW);
    const int oh = rem / g.OW, ow = rem - oh * g.OW;
    const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
    int32_t s = 0;
    for (int kh = 0; kh < g.KH; ++kh)
        for (int kw = 0; kw < g.KW; ++kw) {
            const int ih = ih0 + kh * g.dh, iw = iw0 + kw * g.dw;
            if ((unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W) {
                const uint8_t *src = codes + (((int64_t)n * g.H + ih) * g.W + iw) * g.C;
                for (int c = 0; c < g.C; ++c)
                    s += src[c];
            } else {
                s += offset_input * g.C;
            }
        }
    asum[m] = s;
}

__global__ void __launch_bounds__(256) code_filter_sums_kernel(const uint8_t *__restrict__ fcodes, int K, int Co,
                                                                int32_t *__restrict__ bsum)
{
    const int col = blockIdx.x * blockDim.x + threadIdx.x;
    if (col >= Co)
        return;
    int32_t s = 0;
    for (int k = 0; k < K; ++k)
        s += fcodes[(int64_t)k * Co + col];
    bsum[col] = s;
}

__global__ void __launch_bounds__(256) axconv_correct_kernel(int32_t *__restrict__ out, int64_t mc, int Co,
                                                              const int32_t *__restrict__ asum,
                                                              const int32_t *__restrict__ bsum, int offset_input,
                                                              int offset_filter, int K)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= mc)
        return;
    const int64_t m = i / Co;
    const int col = (int)(i - m * Co);
    // wraps like the reference's int32 arithmetic would
    const int64_t t = (int64_t)out[i] - (int64_t)asum[m] * offset_filter - (int64_t)bsum[col] * offset_input +
                      (int64_t)K * offset_input * offset_filter;
    out[i] = (int32_t)t;
}

hipError_t launch_axconv_correction(const uint8_t *codes, const uint8_t *fcodes, const ConvGeom &g, int offset_input,
                                    int offset_filter, int32_t *asum, int32_t *bsum, int32_t *out, hipStream_t stream)
{
    hipLaunchKernelGGL(code_patch_sums_kernel, dim3(blocks_for(g.M, 256)), dim3(256), 0, stream, codes, g, offset_input,
                       asum);
    hipLaunchKernelGGL(code_filter_sums_kernel, dim3(blocks_for(g.Co, 256)), dim3(256), 0, stream, fcodes, g.K, g.Co,
                       bsum);
    const int64_t mc = g.M * g.Co;
    hipLaunchKernelGGL(axconv_correct_kernel, dim3(blocks_for(mc, 256)), dim3(256), 0, stream, out, mc, g.Co, asum, bsum,
                       offset_input, offset_filter, g.K);
    return hipGetLastError();
}

hipError_t launch_fill_u32(uint32_t *dst, int64_t n, uint32_t value, hipStream_t stream)
{
    for (int64_t done = 0; done < n; done += (int64_t)1 << 30) { // int-sized pieces
        const int piece = (int)(n - done < ((int64_t)1 << 30) ? n - done : (int64_t)1 << 30);
        hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks_for(piece, 256)), dim3(256), 0, stream, dst + done, piece, value);
    }
    return hipGetLastError();
}

// Reduction of the K splits' int32 partial sums (exact, so the order does not matter) followed by the op's
// epilogue (approx_nn_conv_kernels.cpp:250-253), four consecutive columns per thread when Co % 4 == 0.
template <int V>
__global__ void __launch_bounds__(256) splitk_epilogue_kernel(const int32_t *__restrict__ part, int ks, int64_t mc,
                                                               int Co, const float *__restrict__ psum,
                                                               const float *__restrict__ fsum, float s1xs2, float m1,
                                                               float m2, float k_m1xm2,
                                                               const LayerQuant *__restrict__ lq_dev,
                                                               const float *__restrict__ bias, int relu,
                                                               float *__restrict__ out_f,
                                                               int32_t *__restrict__ out_i)
{
    if (lq_dev) {
        s1xs2 = lq_dev->s1xs2;
        m1 = lq_dev->m1;
        m2 = lq_dev->m2;
        k_m1xm2 = lq_dev->k_m1xm2;
    }
    const int64_t i = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * V;
    if (i >= mc)
        return;
    int32_t a[V];
#pragma unroll
    for (int e = 0; e < V; ++e)
        a[e] = 0;
    for (int k = 0; k < ks; ++k) {
        if (V == 4) {
            const int4 v = *reinterpret_cast<const int4 *>(part + (int64_t)k * mc + i);
            a[0] += v.x; a[1 % V] += v.y; a[2 % V] += v.z; a[3 % V] += v.w;
        } else {
            a[0] += part[(int64_t)k * mc + i];
        }
    }
    if (out_i) {
#pragma unroll
        for (int e = 0; e < V; ++e)
            out_i[i + e] = a[e];
        return;
    }
    const int64_t m = i / Co;
    const int col = (int)(i - m * Co);
    const float t1 = __fmul_rn(m2, psum[m]);
    float r[V];
#pragma unroll
    for (int e = 0; e < V; ++e) {
        const float t0 = __fmul_rn((float)a[e], s1xs2);
        const float t2 = __fadd_rn(t0, t1);
        const float t3 = __fmul_rn(m1, fsum[col + e]);
        const float t4 = __fadd_rn(t2, t3);
        r[e] = __fsub_rn(t4, k_m1xm2);
        if (bias)
            r[e] = __fadd_rn(r[e], bias[col + e]);
        if (relu)
            r[e] = fmaxf(r[e], 0.0f);
    }
    if (V == 4)
        *reinterpret_cast<float4 *>(out_f + i) = make_float4(r[0], r[1 % V], r[2 % V], r[3 % V]);
    else
        out_f[i] = r[0];
}

hipError_t launch_splitk_epilogue(const DenseParams &p, const int32_t *partials, float *out_f, int32_t *out_i,
                                  hipStream_t stream)
{
    const int64_t mc = p.g.M * p.g.Co;
    if ((p.g.Co & 3) == 0)
        hipLaunchKernelGGL(splitk_epilogue_kernel<4>, dim3(blocks_for(mc / 4, 256)), dim3(256), 0, stream, partials,
                           p.plan.k_splits, mc, p.g.Co, p.psum, p.fsum, p.s1xs2, p.m1, p.m2, p.k_m1xm2, p.lq_dev, p.bias, p.relu,
                           out_f, out_i);
    else
        hipLaunchKernelGGL(splitk_epilogue_kernel<1>, dim3(blocks_for(mc, 256)), dim3(256), 0, stream, partials,
                           p.plan.k_splits, mc, p.g.Co, p.psum, p.fsum, p.s1xs2, p.m1, p.m2, p.k_m1xm2, p.lq_dev, p.bias, p.relu,
                           out_f, out_i);
    return hipGetLastError();
}

static hipError_t launch_zero_point_row(const ConvGeom &g, uint32_t zp4, uint32_t *xq, hipStream_t stream)
{
    const int n = g.C4 * g.W;
    hipLaunchKernelGGL(fill_u32_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, stream,
                       xq + (size_t)g.N * g.H * g.C4 * g.W, n, zp4);
    return hipGetLastError();
}

hipError_t launch_quantize_relayout(const float *x, const ConvGeom &g, const TensorQuant &tq, const LayerQuant *lq_dev,
                                    uint32_t *xq, float *chsum, hipStream_t stream)
{
    const int64_t pixels = (int64_t)g.N * g.H * g.W;
    if ((g.C & 3) == 0 && !chsum && ((uintptr_t)x & 15) == 0) {
        const int64_t quads = pixels * g.C4;
        int64_t blocks = (quads + 256 * 4 - 1) / (256 * 4);
        if (blocks > 65536) blocks = 65536;
        hipLaunchKernelGGL(quantize_relayout_vec4_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                           reinterpret_cast<const float4 *>(x), quads, g.W, g.C4, tq, lq_dev, xq);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(quantize_relayout_kernel, dim3(blocks_for(pixels, 256)), dim3(256), 0, stream, x, pixels,
                       g.H, g.W, g.C, g.C4, tq, lq_dev, xq, chsum);
    return hipGetLastError();
}

// Band height for patch_sums_rows_body: the one with the least estimated time.  A block first copies its input rows
// (all resident blocks of a CU share that CU's part of the memory bandwidth, ~17 bytes/ns with every CU copying), then
// runs its chains: K dependent adds of ~2.75 ns each, one wavefront per 64 pixels, and a SIMD that holds several
// such wavefronts interleaves them at no better than one add per ~1.9 ns, so lanes left idle by a thin band and
// chain wavefronts that share a SIMD are what make deep layers slow.  Blocks beyond what the CUs hold at once
// run as further rounds; the blocks that sum filter columns in the same launch (sum_blocks) count like the others.
// Rows of many channels fit LDS only a few at a time, or not at all: the band is then cut into column segments of
// wseg output columns, each workgroup holding only the input columns under its segment (input_columns_under).
// Measured on the layers of the networks: where whole rows leave room for one workgroup per CU only, segments that
// let two be resident (the copy of one runs under the chains of the other) are 10-20 % faster, the more pixels per
// workgroup the better; with room for two, whole rows stay ahead.
static int input_columns_under(const ConvGeom &g, int wseg)
{
    if (wseg >= g.OW)
        return g.W;
    const int cols = (wseg - 1) * g.sw + (g.KW - 1) * g.dw + 1;
    return cols < g.W ? cols : g.W;
}

// Least estimated time over the band heights of one segment width; returns false if no band fits.
static bool best_band(const ConvGeom &g, int wseg, int sum_blocks, int64_t lds_limit, int *rb_out, int *in_rows_out,
                      double *t_out, int64_t *lds_out)
{
    const int cus = device_cus();
    const double K = (double)g.KH * g.KW * g.C;
    const int64_t lds_max = device_lds_bytes();
    const int nsegs = (g.OW + wseg - 1) / wseg;
    const int64_t row_bytes = (int64_t)input_columns_under(g, wseg) * (g.C + 4) * 4;
    bool found = false;
    for (int cand = 1; cand <= g.OH && cand * wseg <= 1024; ++cand) {
        const int rows_needed = (cand - 1) * g.sh + (g.KH - 1) * g.dh + 1;
        const int64_t lds = rows_needed * row_bytes + (int64_t)(g.C + 4) * 4;
        if (lds > lds_limit)
            break;
        const int chains = cand * wseg;
        const int block_threads = chains <= 512 ? 512 : 1024;
        int64_t per_cu = lds_max / lds;
        if (per_cu > 2048 / block_threads)
            per_cu = 2048 / block_threads;
        const int64_t blocks = (int64_t)g.N * ((g.OH + cand - 1) / cand) * nsegs + sum_blocks; // all of one LDS size
        const int64_t rounds = (blocks + cus * per_cu - 1) / (cus * per_cu);
        int64_t resident = (blocks + cus - 1) / cus;
        if (resident > per_cu)
            resident = per_cu;
        const int64_t chain_waves = resident * ((chains + 63) / 64);
        const double copy_ns = (double)(resident * lds) / 17.0;
        const double chain_ns = K * 2.75 * (double)((chain_waves + 3) / 4);
        const double t = (double)rounds * (copy_ns + chain_ns);
        if (!found || t < *t_out) {
            found = true;
            *t_out = t;
            *rb_out = cand;
            *in_rows_out = rows_needed;
            *lds_out = lds;
        }
    }
    return found;
}

static void choose_band(const ConvGeom &g, int sum_blocks, int *rb_out, int *in_rows_out, int *wseg_out)
{
    const int64_t lds_max = device_lds_bytes(), lds_two = lds_max / 2;
    double t = 0.0;
    int64_t lds = 0;
    *rb_out = 0;
    *wseg_out = g.OW;
    const bool whole = best_band(g, g.OW, sum_blocks, lds_max, rb_out, in_rows_out, &t, &lds);
    // whole rows with room for two workgroups per CU, or with no more workgroups than CUs: nothing to gain
    if (whole && (lds <= lds_two || (int64_t)g.N * ((g.OH + *rb_out - 1) / *rb_out) + sum_blocks <= device_cus()))
        return;
    // segments with room for two workgroups per CU: the most pixels per workgroup, at least eight, and more
    // segments only for 15 % more pixels (thin segments copy more halo and fill their wavefronts worse).  Not under
    // long chains (K above ~3000: 8 us and more), where the largest workgroup that fits is the better one.
    int best_chains = 7, last_wseg = g.OW;
    const bool long_chains = (int64_t)g.KH * g.KW * g.C > 3000;
    for (int segs : {2, 3, 4, 6, 8}) {
        if (long_chains)
            break;
        const int wseg = (g.OW + segs - 1) / segs;
        if (wseg == last_wseg || wseg < 4)
            continue;
        last_wseg = wseg;
        const int64_t row_bytes = (int64_t)input_columns_under(g, wseg) * (g.C + 4) * 4;
        for (int cand = 1; cand <= g.OH && cand * wseg <= 1024; ++cand) {
            const int rows_needed = (cand - 1) * g.sh + (g.KH - 1) * g.dh + 1;
            if (rows_needed * row_bytes + (int64_t)(g.C + 4) * 4 > lds_two)
                break;
            if (cand * wseg > best_chains && (best_chains == 7 || cand * wseg * 100 > best_chains * 115 ||
                                              wseg == *wseg_out)) {
                best_chains = cand * wseg;
                *rb_out = cand;
                *in_rows_out = rows_needed;
                *wseg_out = wseg;
            }
        }
    }
    if (best_chains > 7 || whole)
        return;
    // whole rows do not fit and neither does a pair of segments: one workgroup per CU, by the estimate
    last_wseg = g.OW;
    bool any = false;
    for (int segs : {2, 3, 4, 6, 8}) {
        const int wseg = (g.OW + segs - 1) / segs;
        if (wseg == last_wseg || wseg < 4)
            continue;
        last_wseg = wseg;
        int rb = 0, in_rows = 0;
        double ts = 0.0;
        if (best_band(g, wseg, sum_blocks, lds_max, &rb, &in_rows, &ts, &lds) && (!any || ts < t)) {
            any = true;
            t = ts;
            *rb_out = rb;
            *in_rows_out = in_rows;
            *wseg_out = wseg;
        }
    }
}

hipError_t launch_patch_sums(const float *x, const ConvGeom &g, const TensorQuant &tq, const LayerQuant *lq_dev,
                             float *psum, hipStream_t stream, uint32_t *xq_fused, bool *fused,
                             const FilterJob *filter_job, bool *filter_done, int flat_row_bytes, bool *px_done)
{
    if (fused)
        *fused = false;
    if (filter_done)
        *filter_done = false;
    if (px_done)
        *px_done = false;
    const bool vec = (g.C & 3) == 0 && ((uintptr_t)x & 15) == 0;
    if (flat_row_bytes && vec)   // the flat layout belongs to channel counts that are no multiple of four
        return hipErrorInvalidValue;
    if (vec && g.OW <= 1024) {
        // largest band of output rows whose input rows fit in 96 KiB of LDS and whose pixels fit in one block,
        // but no larger than what still leaves every CU a few blocks
        const int64_t row_bytes = (int64_t)g.W * (g.C + 4) * 4;
        int rb = 0, in_rows = 0;
        for (int cand = 1; cand <= g.OH && cand * g.OW <= 1024; ++cand) {
            const int rows_needed = (cand - 1) * g.sh + (g.KH - 1) * g.dh + 1;
            if (rows_needed * row_bytes > 96 * 1024)
                break;
            if (cand > 1 && (int64_t)g.N * ((g.OH + cand - 1) / cand) < 1024)
                break;
            rb = cand;
            in_rows = rows_needed;
        }
        // 1x1, stride 1, no padding, and a band would hold few pixels (many channels): the flat-list variant
        const bool flat = g.KH == 1 && g.KW == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 &&
                          rb * g.OW < 192;
        int wseg = g.OW;   // output columns per workgroup: whole rows unless choose_band cuts them
        if (!flat)
            choose_band(g, (filter_job && filter_job->fsum && filter_job->filter) ? (int)blocks_for(g.Co, kFsCols) : 0,
                        &rb, &in_rows, &wseg);
        // ... and with many channels and too few pixels to give every CU a workgroup of 64, the variant built around
        // the chain of adds
        const bool deep = flat && g.C >= 512 && g.M < (int64_t)64 * device_cus();
        if (flat) { // in_rows carries the pixels per workgroup: at least ~2 workgroups per CU where the layer allows
            rb = 0;
            // measured: 128 pixels from 28x28x64 images on (-13 % against 64), 256 only with few channels
            in_rows = (g.M >= 512 * kFlatPixels && g.C <= 128) ? kFlatPixels : (g.M >= 512 * 64 ? 128 : 64);
        }
        if (deep) {
            rb = -1;
            in_rows = g.M >= (int64_t)2 * 16 * device_cus() ? 16 : 8;
        }
        if (rb > 0 || flat) {
            int threads = ((rb * wseg + 63) / 64) * 64;
            threads = threads < 512 ? 512 : threads;   // the copy into LDS wants more threads than there are pixels
            // Band b owns input rows [b*rb*sh, (b+1)*rb*sh), the last band up to H.  They are quantized by the
            // block that holds them if every band's window (rows b*rb*sh - ph onwards, in_rows of them) contains
            // its owned rows, the last window reaches the last image row, and the fast copy loop is in use.  The
            // same along the row where a band is cut into column segments (segment s owns input columns
            // [s*wseg*sw, (s+1)*wseg*sw), the last one up to W).
            const bool segmented = !flat && wseg < g.OW;
            const bool fuse = xq_fused && fused &&
                              (flat || (g.sh - 1 + g.ph <= (g.KH - 1) * g.dh &&
                                        (g.OH - 1) * g.sh - g.ph + (g.KH - 1) * g.dh >= g.H - 1 && threads % g.C4 == 0 &&
                                        (!segmented || (g.sw - 1 + g.pw <= (g.KW - 1) * g.dw &&
                                                        (g.OW - 1) * g.sw - g.pw + (g.KW - 1) * g.dw >= g.W - 1))));
            if (fuse)
                *fused = true;
            const size_t band_row_bytes = (size_t)input_columns_under(g, wseg) * (g.C + 4) * 4;
            size_t lds = deep ? (size_t)deep_lds_bytes(in_rows)
                              : flat ? (size_t)in_rows * kFlatPitch * 4
                                     : (size_t)in_rows * band_row_bytes + (size_t)(g.C + 4) * 4; // + the pixel of zeros
            const int bands = flat ? 0 : (g.OH + rb - 1) / rb;
            const int64_t work_blocks =
                flat ? (g.M + in_rows - 1) / in_rows : (int64_t)g.N * bands * ((g.OW + wseg - 1) / wseg);
            // the filter pre-pass rides along in the same launch (its workgroups want 512 or 1024 threads, so
            // every workgroup gets that many; only `threads` of them take part in the patch sums)
            FilterWork fw = {};
            int block_threads = threads;
            if (filter_job && filter_done) {
                const DensePlan &plan = *filter_job->plan;
                const int64_t total = (int64_t)plan.n_col_tiles * plan.fills * 64;
                fw.filter = filter_job->filter;
                fw.filter_codes = filter_job->filter_codes;
                fw.taps = g.KH * g.KW;
                fw.C = g.C;
                fw.C4 = g.C4;
                fw.Co = g.Co;
                fw.nt = plan.nt;
                fw.n_col_tiles = plan.n_col_tiles;
                fw.tq = filter_job->tq;
                fw.wq = filter_job->wq;
                fw.sum_blocks = (filter_job->fsum && filter_job->filter) ? (int)blocks_for(g.Co, kFsCols) : 0;
                fw.fsum = filter_job->fsum;
                block_threads = threads <= 512 ? 512 : 1024;
                // A block of pack work would hold a patch-sum block's worth of LDS for nothing: with bands of rows
                // (large LDS, most threads idle while the chains run) idle wavefronts of the patch-sum blocks pack,
                // those on SIMDs that hold no chain, so at most three chain wavefronts per block.
                if (!flat && rb * wseg <= 3 * 64)
                    fw.pack_total = total;
                fw.sum8 = (fw.sum_blocks + 7) & ~7;
                fw.pack_blocks = fw.pack_total > 0 ? 0 : (int)blocks_for(total, block_threads);
                if (fw.sum_blocks && lds < (size_t)kFsLdsBytes)
                    lds = kFsLdsBytes;
                *filter_done = true;
                // ... and so do the pre-expanded rows where the layer runs out of them: blockDim.x / 4 activation
                // codes of a pair of fills per workgroup, the stage and the pair's 128 filter codes in LDS
                if (px_done && filter_job->px_rows && plan.nt == 16 && plan.fills == fw.taps * fw.C4 &&
                    (plan.fills & 1) == 0) {
                    const int64_t eb = (int64_t)plan.n_col_tiles * (plan.fills / 2) * (1024 / block_threads);
                    const size_t need = (size_t)(block_threads / 4) * kPxExpandPitch * 4 + 256;
                    // Every workgroup of a launch takes the same LDS.  Where the patch sums take so much that a CU
                    // holds fewer of these workgroups than its wavefront slots allow (2048 threads), the rows are
                    // written more slowly; that still beats a launch of their own (north star -1.8 %, 3x3 128->128
                    // @28x28 -3.1 %) until the rows are many (1.2 GB: 0.26 -> 0.33 ms, +2.3 % on the layer).
                    const size_t lds_with = lds < need ? need : lds;
                    const bool slow = lds_with * (size_t)(2048 / block_threads) > (size_t)device_lds_bytes();
                    const size_t row_bytes = (size_t)plan.n_col_tiles * (size_t)(plan.fills / 2) * kPxFillBytes;
                    if (eb + fw.sum8 + work_blocks + fw.pack_blocks < ((int64_t)1 << 31) &&
                        lds_with <= (size_t)device_lds_bytes() && !(slow && row_bytes > ((size_t)512 << 20))) {
                        fw.expand_blocks = (int)eb;
                        fw.tableT = filter_job->tableT;
                        fw.px_rows = filter_job->px_rows;
                        lds = lds < need ? need : lds;
                        *px_done = true;
                    }
                }
            }
            fw.work_blocks = (int)work_blocks;
            const unsigned grid = (unsigned)(fw.sum8 + work_blocks + fw.pack_blocks + fw.expand_blocks);
            if (segmented) {
                const hipError_t e =
                    set_max_dynamic_lds_once(reinterpret_cast<const void *>(patch_sums_segments_kernel), device_lds_bytes());
                if (e != hipSuccess)
                    return e;
                hipLaunchKernelGGL(patch_sums_segments_kernel, dim3(grid), dim3(block_threads), lds, stream, x, g, rb, in_rows, threads, wseg, tq, lq_dev, psum,
                                   fuse ? xq_fused : nullptr, fw);
                return hipGetLastError();
            }
            const hipError_t e = set_max_dynamic_lds_once(reinterpret_cast<const void *>(patch_sums_rows_kernel), device_lds_bytes());
            if (e != hipSuccess)
                return e;
            hipLaunchKernelGGL(patch_sums_rows_kernel, dim3(grid), dim3(block_threads),
                               lds, stream, x, g, rb, in_rows, threads, tq, lq_dev, psum, fuse ? xq_fused : nullptr, fw);
            return hipGetLastError();
        }
    }
    if (!vec && g.OW <= 1024 && g.C < 64) {
        // few channels that are not a multiple of four: bands of output rows with their input rows in LDS
        const int64_t row_bytes = (int64_t)g.W * g.C * 4;
        int rb = 0, in_rows = 0;
        for (int cand = 1; cand <= g.OH && cand * g.OW <= 1024; ++cand) {
            const int rows_needed = (cand - 1) * g.sh + (g.KH - 1) * g.dh + 1;
            if (rows_needed * row_bytes > 96 * 1024)
                break;
            if (cand > 1 && (int64_t)g.N * ((g.OH + cand - 1) / cand) < 1024)
                break;
            rb = cand;
            in_rows = rows_needed;
        }
        if (rb > 0) {
            int threads = ((rb * g.OW + 63) / 64) * 64;
            threads = threads < 256 ? 256 : threads;
            const bool fuse = xq_fused && fused && g.sh - 1 + g.ph <= (g.KH - 1) * g.dh &&
                              (g.OH - 1) * g.sh - g.ph + (g.KH - 1) * g.dh >= g.H - 1;
            if (fuse)
                *fused = true;
            const hipError_t e = set_max_dynamic_lds_once(reinterpret_cast<const void *>(patch_sums_smallc_kernel), 96 * 1024);
            if (e != hipSuccess)
                return e;
            const int bands = (g.OH + rb - 1) / rb;
            hipLaunchKernelGGL(patch_sums_smallc_kernel, dim3((unsigned)((int64_t)g.N * bands)), dim3(threads),
                               (size_t)in_rows * row_bytes, stream, x, g, rb, in_rows, tq, lq_dev, psum,
                               fuse ? xq_fused : nullptr, flat_row_bytes, g.pw);
            return hipGetLastError();
        }
    }
    if (vec)
        hipLaunchKernelGGL(patch_sums_tiled_kernel, dim3(blocks_for(g.M, kPsTile)), dim3(kPsTile), 0, stream, x, g,
                           tq, lq_dev, psum);
    else
        hipLaunchKernelGGL(patch_sums_kernel, dim3(blocks_for(g.M, 256)), dim3(256), 0, stream, x, g, tq, lq_dev, psum);
    return hipGetLastError();
}

// Gathers the pixels a strided 1x1 filter reads into a dense tensor: VEC bytes per thread and step, pixel_bytes
// (a multiple of VEC) per pixel.
template <typename V>
__global__ void __launch_bounds__(256) subsample_kernel(const V *__restrict__ in, V *__restrict__ out, int64_t total,
                                                         int per_pixel, int H, int W, int sh, int sw, int OH, int OW)
{
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        const int64_t pix = i / per_pixel;
        const int e = (int)(i - pix * per_pixel);
        const int ow = (int)(pix % OW);
        const int64_t r = pix / OW;
        const int oh = (int)(r % OH);
        const int64_t n = r / OH;
        out[i] = in[((n * H + (int64_t)oh * sh) * W + (int64_t)ow * sw) * per_pixel + e];
    }
}

hipError_t launch_subsample(const void *in, int element_bytes, int N, int H, int W, int C, int sh, int sw, int OH, int OW,
                            void *out, hipStream_t stream)
{
    const int64_t pixel_bytes = (int64_t)C * element_bytes;
    const int64_t pixels = (int64_t)N * OH * OW;
    const bool wide = (pixel_bytes & 15) == 0 && ((uintptr_t)in & 15) == 0 && ((uintptr_t)out & 15) == 0;
    const int vec = wide ? 16 : (((pixel_bytes & 3) == 0 && ((uintptr_t)in & 3) == 0) ? 4 : 1);
    const int64_t total = pixels * (pixel_bytes / vec);
    int64_t blocks = (total + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > 16384 ? 16384 : blocks);
    const int per_pixel = (int)(pixel_bytes / vec);
    if (vec == 16)
        hipLaunchKernelGGL(subsample_kernel<float4>, dim3((unsigned)blocks), dim3(256), 0, stream,
                           static_cast<const float4 *>(in), static_cast<float4 *>(out), total, per_pixel, H, W, sh, sw, OH, OW);
    else if (vec == 4)
        hipLaunchKernelGGL(subsample_kernel<uint32_t>, dim3((unsigned)blocks), dim3(256), 0, stream,
                           static_cast<const uint32_t *>(in), static_cast<uint32_t *>(out), total, per_pixel, H, W, sh, sw, OH, OW);
    else
        hipLaunchKernelGGL(subsample_kernel<uint8_t>, dim3((unsigned)blocks), dim3(256), 0, stream,
                           static_cast<const uint8_t *>(in), static_cast<uint8_t *>(out), total, per_pixel, H, W, sh, sw, OH, OW);
    return hipGetLastError();
}

hipError_t launch_codes_relayout(const uint8_t *codes, const ConvGeom &g, uint32_t zp4, uint32_t *xq,
                                 hipStream_t stream)
{
    hipError_t ez = launch_zero_point_row(g, zp4, xq, stream);
    if (ez != hipSuccess)
        return ez;
    const int64_t pixels = (int64_t)g.N * g.H * g.W;
    hipLaunchKernelGGL(codes_relayout_kernel, dim3(blocks_for(pixels, 256)), dim3(256), 0, stream, codes, pixels,
                       g.W, g.C, g.C4, xq);
    return hipGetLastError();
}

hipError_t launch_filter_pack(const float *filter, const uint8_t *filter_codes, const ConvGeom &g,
                              const DensePlan &plan, const TensorQuant &tq, const LayerQuant *lq_dev, uint16_t *wq,
                              float *fsum, hipStream_t stream, const uint16_t *tableT, uint16_t *px_rows, bool *px_done)
{
    if (px_done)
        *px_done = false;
    const int64_t total = (int64_t)plan.n_col_tiles * plan.fills * 64;
    const int sum_blocks = (fsum && filter) ? (int)blocks_for(g.Co, kFsCols) : 0;
    const int pack_blocks = (int)blocks_for(total, kFsThreads);
    size_t lds = sum_blocks ? kFsLdsBytes : 0;
    // the pre-expanded rows ride along as in launch_patch_sums: a whole pair of fills per workgroup of 1024
    int64_t expand_blocks = 0;
    const size_t row_bytes = (size_t)plan.n_col_tiles * (size_t)(plan.fills / 2) * kPxFillBytes;
    if (px_done && px_rows && plan.nt == 16 && plan.fills == g.KH * g.KW * g.C4 && (plan.fills & 1) == 0 &&
        row_bytes <= ((size_t)512 << 20)) {
        expand_blocks = (int64_t)plan.n_col_tiles * (plan.fills / 2);
        const size_t need = (size_t)(kFsThreads / 4) * kPxExpandPitch * 4 + 256;
        lds = lds < need ? need : lds;
        *px_done = true;
    }
    if (lds) {
        const hipError_t ea = set_max_dynamic_lds_once(reinterpret_cast<const void *>(filter_prep_kernel),
                                                       (int)(lds > (size_t)kFsLdsBytes ? lds : (size_t)kFsLdsBytes));
        if (ea != hipSuccess)
            return ea;
    }
    hipLaunchKernelGGL(filter_prep_kernel, dim3((unsigned)(sum_blocks + pack_blocks + expand_blocks)), dim3(kFsThreads), lds,
                       stream, filter, filter_codes, g.KH * g.KW, g.C, g.C4, g.Co, plan.nt, plan.n_col_tiles, tq, lq_dev,
                       wq, sum_blocks, fsum, pack_blocks, tableT, px_rows);
    return hipGetLastError();
}

// Flat layout of the quantized input for channel counts that are no multiple of four: one thread per dword of xq.
// Byte b of row r (r = image * H + input row; row N * H is the zero-point row that taps outside the image read)
// is the code of channel b % C of pixel b / C - pad_left, the zero-point code where that pixel lies outside the
// image or b lies behind the last pixel.
__global__ void __launch_bounds__(256) quantize_flat_rows_kernel(const float *__restrict__ x,
                                                                 const uint8_t *__restrict__ codes, int64_t rows,
                                                                 int W, int C, int pad_left, int row_bytes,
                                                                 const TensorQuant tq,
                                                                 const LayerQuant *__restrict__ lq_dev,
                                                                 uint32_t *__restrict__ xq)
{
    const TensorQuant qt = lq_dev ? lq_dev->in : tq;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // dword index
    const int dwords_per_row = row_bytes / 4;
    if (i >= (rows + 1) * dwords_per_row)
        return;
    const int64_t r = i / dwords_per_row;
    const int b0 = (int)(i - r * dwords_per_row) * 4;
    const uint32_t zp = qt.zp4 & 0xffu;
    uint32_t word = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int b = b0 + k;
        const int px = b / C, c = b - px * C, w = px - pad_left;
        uint32_t code = zp;
        if (r < rows && (unsigned)w < (unsigned)W) {
            const int64_t src = (r * W + w) * C + c;
            code = codes ? phys_row(codes[src])
                         : phys_row(quantize_code(fake_quant_value(x[src], qt), qt.offset, qt.inv_scale));
        }
        word |= code << (8 * k);
    }
    xq[i] = word;
}

hipError_t launch_quantize_flat_rows(const float *x, const uint8_t *codes, const ConvGeom &g, int pad_left,
                                     int row_bytes, const TensorQuant &tq, const LayerQuant *lq_dev, uint8_t *xq,
                                     hipStream_t stream)
{
    const int64_t rows = (int64_t)g.N * g.H;
    const int64_t dwords = (rows + 1) * (row_bytes / 4);
    hipLaunchKernelGGL(quantize_flat_rows_kernel, dim3(blocks_for(dwords, 256)), dim3(256), 0, stream, x, codes, rows,
                       g.W, g.C, pad_left, row_bytes, tq, lq_dev, reinterpret_cast<uint32_t *>(xq));
    return hipGetLastError();
}

hipError_t launch_quantize_flat(const float *v, int64_t n, float offset, float inv_scale, uint8_t *codes,
                                hipStream_t stream)
{
    if (n == 0)
        return hipSuccess;
    hipLaunchKernelGGL(quantize_flat_kernel, dim3(blocks_for(n, 256)), dim3(256), 0, stream, v, n, offset,
                       inv_scale, codes);
    return hipGetLastError();
}

hipError_t launch_depthwise_filter(const float *filter, int taps, int C, const TensorQuant &tq,
                                   const LayerQuant *lq_dev, uint8_t *wcodes, float *fsum, hipStream_t stream)
{
    hipLaunchKernelGGL(depthwise_filter_kernel, dim3(blocks_for(C, 256)), dim3(256), 0, stream, filter, taps, C,
                       tq, lq_dev, wcodes, fsum);
    return hipGetLastError();
}

} // namespace axc
