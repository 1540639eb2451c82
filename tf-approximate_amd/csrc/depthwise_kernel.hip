// Depthwise LUT convolution (channel multiplier 1) and the LDS / VALU rate probes.
#include "axconv_internal.h"

#include <type_traits>

namespace axc {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

extern __shared__ __align__(16) unsigned char lds_dw[];

// Quantization of the input as this launch sees it: by value for the op, from the device for the layer entry point.
__device__ __forceinline__ TensorQuant dw_input_quant(const DepthwiseParams &p) { return p.lq_dev ? p.lq_dev->in : p.in_q; }

struct DwEpilogue {
    float s1xs2, m1, m2, k_m1xm2;
};
__device__ __forceinline__ DwEpilogue dw_epilogue_consts(const DepthwiseParams &p)
{
    if (p.lq_dev)   // K of the layer's constants is the dense patch length; depthwise has K = taps
        return {p.lq_dev->s1xs2, p.lq_dev->m1, p.lq_dev->m2,
                __fmul_rn((float)(p.KH * p.KW), __fmul_rn(p.lq_dev->m1, p.lq_dev->m2))};
    return {p.s1xs2, p.m1, p.m2, p.k_m1xm2};
}

// Every output (pixel, channel) is its own dot product over the KH*KW taps, so there is no weight
// reuse across lanes to expand: lanes look single entries up in the LDS-resident table,
// T[b][a] at byte b*512 + a*2.  Lanes walk consecutive channels (NHWC: coalesced loads and stores).
// Per-channel semantics: out[p][c] = dense op on channel c alone (K = KH*KW), so the patch sum is the
// sequential fp32 sum of the taps of that channel, in tap order, zeros included outside the image.
template <bool OUT_I32>
__global__ void __launch_bounds__(kBlockThreads) depthwise_lut_kernel(const DepthwiseParams p)
{
    const int tid = threadIdx.x;
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(p.tableT);
        u32x4 *dst = reinterpret_cast<u32x4 *>(lds_dw);
#pragma unroll
        for (int i = 0; i < kTableBytes / 16 / kBlockThreads; ++i)
            dst[tid + i * kBlockThreads] = src[tid + i * kBlockThreads];
    }
    __syncthreads();
    const uint16_t *table = reinterpret_cast<const uint16_t *>(lds_dw);
    const TensorQuant q = dw_input_quant(p);
    const DwEpilogue ep = dw_epilogue_consts(p);

    const int64_t total = p.M * p.C;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + tid; idx < total; idx += stride) {
        const int c = (int)(idx % p.C);
        const int64_t m = idx / p.C;
        const int n = (int)(m / ((int64_t)p.OH * p.OW));
        const int rem = (int)(m - (int64_t)n * p.OH * p.OW);
        const int oh = rem / p.OW, ow = rem - oh * p.OW;
        const int ih0 = oh * p.sh - p.ph, iw0 = ow * p.sw - p.pw;
        int32_t acc = 0;
        float psum = 0.0f;
        int tap = 0;
        for (int kh = 0; kh < p.KH; ++kh)
            for (int kw = 0; kw < p.KW; ++kw, ++tap) {
                const int ih = ih0 + kh * p.dh, iw = iw0 + kw * p.dw;
                float v = 0.0f;
                if ((unsigned)ih < (unsigned)p.H && (unsigned)iw < (unsigned)p.W)
                    v = fake_quant_value(p.x[(((int64_t)n * p.H + ih) * p.W + iw) * p.C + c], q);
                psum = __fadd_rn(psum, v);
                const uint32_t a = quantize_code(v, q.offset, q.inv_scale);
                const uint32_t b = p.wcodes[(int64_t)tap * p.C + c];
                acc += (int32_t)table[b * 256u + a];
            }
        if (OUT_I32) {
            p.out_i[idx] = acc;
        } else {
            const float t0 = __fmul_rn((float)acc, ep.s1xs2);
            const float t1 = __fmul_rn(ep.m2, psum);
            const float t2 = __fadd_rn(t0, t1);
            const float t3 = __fmul_rn(ep.m1, p.fsum[c]);
            const float t4 = __fadd_rn(t2, t3);
            float v = __fsub_rn(t4, ep.k_m1xm2);
            if (p.bias)
                v = __fadd_rn(v, p.bias[c]);
            p.out_f[idx] = p.relu ? fmaxf(v, 0.0f) : v;
        }
    }
}

// ---- 3x3 filters, dilation 1, strides 1 or 2 -------------------------------------------------------------------
// A workgroup serves kDwChannels consecutive channels.  For them it keeps, in LDS, the table row of every one of the
// 9 x kDwChannels filter codes, transposed to activation-code major, two taps to a dword:
//     entry a of (tap t, channel c) at byte  a * kDwCodeStride + (t >> 1) * 128 + c * 4 + (t & 1) * 2
// with kDwCodeStride = 5 * 128 (the tenth tap slot is unused), 160 KiB in all.  A lane is one channel (two bands of
// output rows per wavefront: lanes 0-31 and 32-63), and a two-byte read serves 32 lanes per pass over 32 banks:
// channel c only ever touches bank c, whatever the activation codes are.  The byte offset of an activation code is
// one multiply-add and the tap is an immediate offset of the read.
//
// A lane produces a block of R output rows by `len` output columns: it slides a window of (R-1)*S+3 input rows by 3
// columns along the row, so an input value is loaded, fake-quantized (layer entry point) and turned into its LDS
// offset once per block instead of once per output row and tap, and rows shared by the R outputs of a column are
// fetched once.  Both halves of a wavefront walk the same columns, so column offsets are scalars.  Rows outside the
// image are buffer offsets past the end, which read 0.0f (the value the reference pads with; it quantizes to the
// zero-point code) and drop stores, without a branch; so are columns outside the image (a wave-uniform case).
// Results are those of depthwise_lut_kernel: taps in (kh, kw) order, the patch sum sequential in that order.
constexpr int kDwChannels = 32;
// output columns by which the window's loads run ahead of its lookups (2 and 3 measured no faster than 1)
#ifndef AXC_DW_AHEAD
#define AXC_DW_AHEAD 1
#endif

// f(integral_constant<int, I>) for I = A .. B-1
template <int A, int B, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    if constexpr (A < B) {
        f(std::integral_constant<int, A>());
        static_for<A + 1, B>(f);
    }
}
constexpr int kDwCodeStride = 5 * kDwChannels * 4;    // bytes between activation codes: five pairs of taps
constexpr int kDwLdsBytes = 256 * kDwCodeStride;      // 163840

typedef __amdgpu_buffer_rsrc_t dw_rsrc_t;
__device__ __forceinline__ dw_rsrc_t dw_make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

template <int S, int R, bool OUT_I32, bool FQ, bool EPI>
__global__ void __launch_bounds__(kBlockThreads) depthwise_lut3x3_kernel(const DepthwiseParams p, const int seg_len,
                                                                          const int nseg, const int wgs_per_group,
                                                                          const int group_slots)
{
    constexpr int RIN = (R - 1) * S + 3;               // input rows under R output rows
    constexpr int AHEAD = AXC_DW_AHEAD;                // output columns by which the loads run ahead of the lookups
    constexpr int SLOTS = 3 + S * AHEAD;               // window columns held at a time: the 3 in use and those on their way
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int cl = lane & (kDwChannels - 1), half = lane >> 5;
    const int slot = (int)blockIdx.x / wgs_per_group, member = (int)blockIdx.x - slot * wgs_per_group;
    if (slot >= group_slots)
        return;
    TensorQuant q = dw_input_quant(p);
    q.fq = FQ ? 1u : 0u;                                // known at compile time: no branch per value
    const DwEpilogue ep = dw_epilogue_consts(p);
    const uint32_t x_bytes = (uint32_t)((int64_t)p.N * p.H * p.W * p.C * 4);
    const uint32_t o_bytes = (uint32_t)(p.M * p.C * 4);
    const dw_rsrc_t x_rsrc = dw_make_rsrc(p.x, x_bytes);
    const dw_rsrc_t o_rsrc = dw_make_rsrc(OUT_I32 ? static_cast<const void *>(p.out_i) : static_cast<const void *>(p.out_f), o_bytes);
    const dw_rsrc_t t_rsrc = dw_make_rsrc(p.tableT, (uint32_t)kTableAllocBytes);
    const uint32_t col_bytes = (uint32_t)p.C * 4u;
    const int band_pairs = (p.OH + 2 * R - 1) / (2 * R);
    // a task = (image, pair of bands of R output rows, column segment), segment fastest; the halves of a wavefront
    // take the two bands of a pair
    const int tasks = p.N * band_pairs * nseg;
    const int ngroups = (p.C + kDwChannels - 1) / kDwChannels;
    // the members of a group take contiguous runs of its tasks: neighbouring bands, which share input rows, stay in
    // one workgroup (and so in one L2)
    const int run_first = (int)((int64_t)tasks * member / wgs_per_group);
    const int run_end = (int)((int64_t)tasks * (member + 1) / wgs_per_group);

    for (int group = slot; group < ngroups; group += group_slots) {
        const int chan = group * kDwChannels + cl;
        const bool live = chan < p.C;
        __syncthreads();                                // every wavefront is done with the previous group's rows
        // ---- stage the 9 x 32 table rows, transposed: a lane takes 8 activation codes (16 bytes of a row) of one
        // channel for a pair of taps and writes one dword (both taps' entries) per code
        for (int item = tid; item < 5 * kDwChannels * 32; item += kBlockThreads) {
            const int c = item & 31, piece = (item >> 5) & 31, tp = item >> 10;
            const int ch = group * kDwChannels + c;
            const uint32_t code0 = ch < p.C ? p.wcodes[(2 * tp) * p.C + ch] : kNullWeight;
            const uint32_t code1 = (ch < p.C && 2 * tp + 1 < 9) ? p.wcodes[(2 * tp + 1) * p.C + ch] : kNullWeight;
            const u32x4 v0 = __builtin_amdgcn_raw_buffer_load_b128(t_rsrc, (int)(code0 * 512u + (uint32_t)piece * 16u), 0, 0);
            const u32x4 v1 = __builtin_amdgcn_raw_buffer_load_b128(t_rsrc, (int)(code1 * 512u + (uint32_t)piece * 16u), 0, 0);
            unsigned char *dst = lds_dw + (8 * piece) * kDwCodeStride + tp * 128 + c * 4;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                *reinterpret_cast<uint32_t *>(dst + (2 * e) * kDwCodeStride) = (v0[e] & 0xffffu) | (v1[e] << 16);
                *reinterpret_cast<uint32_t *>(dst + (2 * e + 1) * kDwCodeStride) = (v0[e] >> 16) | (v1[e] & 0xffff0000u);
            }
        }
        __syncthreads();

        const float t3 = (!OUT_I32 && live) ? __fmul_rn(ep.m1, p.fsum[chan]) : 0.0f;
        // EPI: the call has a bias or a ReLU (a template parameter: the plain op pays for neither).  Without a bias
        // the kernel adds -0.0f, which changes no value, the sign of a zero included.
        const bool has_relu = EPI && p.relu;
        const float bias = (EPI && !OUT_I32 && p.bias && live) ? p.bias[chan] : -0.0f;
        // LDS address of this lane's entries of activation code 0: the tap is an immediate offset of the read
        const uint32_t lane_base = (uint32_t)reinterpret_cast<uintptr_t>(lds_dw) + (uint32_t)cl * 4u;
        typedef const __attribute__((address_space(3))) uint16_t *lds_entry_ptr;
        // value -> (fake-quantized value, LDS address of its code's entries); the code is below 2^24
        auto convert = [&](float &val, uint32_t &off) {
            val = fake_quant_value(val, q);
            off = __umul24(quantize_code(val, q.offset, q.inv_scale), (uint32_t)kDwCodeStride) + lane_base;
        };

        for (int task = run_first + wave; task < run_end; task += kWaves) {
            const int seg = task % nseg, nb = task / nseg;
            const int bp = nb % band_pairs, n = nb / band_pairs;
            const int oh0 = (2 * bp + half) * R, ow0 = seg * seg_len;
            const int len = (ow0 + seg_len < p.OW ? ow0 + seg_len : p.OW) - ow0;   // wave-uniform
            const int ih0 = oh0 * S - p.ph, iw0 = ow0 * S - p.pw;
            uint32_t rowoff[RIN];
#pragma unroll
            for (int r = 0; r < RIN; ++r) {
                const int ih = ih0 + r;
                rowoff[r] = (live && (unsigned)ih < (unsigned)p.H)
                                ? (uint32_t)((((int64_t)n * p.H + ih) * p.W * p.C + chan) * 4)
                                : 0x80000000u;
            }
            uint32_t ooff[R];                           // byte offset of (n, oh0 + rr, 0, chan) in the output
#pragma unroll
            for (int rr = 0; rr < R; ++rr)
                ooff[rr] = (live && oh0 + rr < p.OH)
                               ? (uint32_t)((((int64_t)(n * p.OH + oh0 + rr) * p.OW) * p.C + chan) * 4)
                               : 0x80000000u;

            // The window: input column j of the block (j = 0 is column iw0) lives in slot j % SLOTS for as long as an
            // output column needs it.  SLOTS = 3 + S * AHEAD: the S columns that enter with output column k + AHEAD are
            // loaded into the slots that column k - 1 left, while column k is computed, and those of column k + 1 are
            // converted in place afterwards - no value is ever copied from one register to another.  (AHEAD = 2 and 3
            // measured no faster than 1: the kernel is bound by the memory system, not by a wavefront's latency.)
            float val[RIN][SLOTS];
            uint32_t off[RIN][SLOTS];
            // Column iw of every window row into a slot; zeros when the column is outside the image or not wanted (both
            // wave-uniform).  No branch: the offset of such a column is past the end of the buffer, like a row outside
            // the image.  With a branch around the loads the compiler no longer knows, where the paths meet, which
            // loads have returned, and waits in every output column for loads - and with them for the stores issued
            // after them - that have long been waited for.
            auto load_col = [&](int iw, auto slot_tag, bool wanted) {
                constexpr int SL = decltype(slot_tag)::value;
                const bool inside = wanted && (unsigned)iw < (unsigned)p.W;
                const uint32_t past = inside ? 0u : 0x80000000u;
                const uint32_t coff = inside ? (uint32_t)iw * col_bytes : 0u;
#pragma unroll
                for (int r = 0; r < RIN; ++r)
                    val[r][SL] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(x_rsrc, (int)(rowoff[r] | past), (int)coff, 0));
            };
            auto convert_col = [&](auto slot_tag) {
                constexpr int SL = decltype(slot_tag)::value;
#pragma unroll
                for (int r = 0; r < RIN; ++r)
                    convert(val[r][SL], off[r][SL]);
            };
            // the columns of the first AHEAD output columns
            static_for<0, 3 + S * (AHEAD - 1)>([&](auto j) { load_col(iw0 + decltype(j)::value, j, true); });
            static_for<0, 3>([&](auto j) { convert_col(j); });

            auto step = [&](const int k, auto phase_tag) {
                constexpr int PH = decltype(phase_tag)::value;   // k % SLOTS
                // slots of the columns that enter with output column k + AHEAD (loaded now) and with k + 1 (converted
                // when this column is done)
                constexpr int LD0 = (S * (PH + AHEAD) + 3 - S) % SLOTS, LD1 = (LD0 + 1) % SLOTS;
                constexpr int CV0 = (S * PH + 3) % SLOTS, CV1 = (CV0 + 1) % SLOTS;
                load_col(iw0 + (k + AHEAD) * S + 3 - S, std::integral_constant<int, LD0>(), k + AHEAD < len);
                if (S == 2)
                    load_col(iw0 + (k + AHEAD) * S + 2, std::integral_constant<int, LD1>(), k + AHEAD < len);
                const uint32_t ocol = (uint32_t)(ow0 + k) * col_bytes;
#pragma unroll
                for (int rr = 0; rr < R; ++rr) {
                    uint32_t e[9];
                    float psum = 0.0f;
#pragma unroll
                    for (int kh = 0; kh < 3; ++kh)
#pragma unroll
                        for (int kw = 0; kw < 3; ++kw) {
                            const int ps = (S * PH + kw) % SLOTS;
                            const int tap = kh * 3 + kw;
                            psum = __fadd_rn(psum, val[rr * S + kh][ps]);
                            e[tap] = reinterpret_cast<lds_entry_ptr>(off[rr * S + kh][ps])[(tap >> 1) * 64 + (tap & 1)];
                        }
                    const uint32_t acc = ((e[0] + e[1] + e[2]) + (e[3] + e[4] + e[5])) + (e[6] + e[7] + e[8]);
                    uint32_t outw;
                    if (OUT_I32) {
                        outw = acc;
                    } else {
                        const float t0 = __fmul_rn((float)(int32_t)acc, ep.s1xs2);
                        const float t1 = __fmul_rn(ep.m2, psum);
                        const float t2 = __fadd_rn(t0, t1);
                        const float t4 = __fadd_rn(t2, t3);
                        float v = __fsub_rn(t4, ep.k_m1xm2);
                        if (EPI)
                            v = __fadd_rn(v, bias);
                        outw = __float_as_uint(has_relu ? fmaxf(v, 0.0f) : v);
                    }
                    // streamed past the caches, which the input rows neighbouring bands share need
                    __builtin_amdgcn_raw_buffer_store_b32(outw, o_rsrc, (int)ooff[rr], (int)ocol, 2);
                }
                convert_col(std::integral_constant<int, CV0>());   // behind the last column: zeros, never used
                if (S == 2)
                    convert_col(std::integral_constant<int, CV1>());
            };
            for (int k = 0; k < len; k += SLOTS)
                static_for<0, SLOTS>([&](auto ph) {
                    if (k + decltype(ph)::value < len)
                        step(k + decltype(ph)::value, ph);
                });
        }
    }
}

template <typename Kernel, typename... Args>
static hipError_t launch_with_lds(Kernel kernel, int grid, int lds_bytes, hipStream_t stream, Args... args)
{
    const hipError_t e = set_max_dynamic_lds_once(reinterpret_cast<const void *>(kernel), lds_bytes);
    if (e != hipSuccess)
        return e;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kBlockThreads), lds_bytes, stream, args...);
    return hipGetLastError();
}

hipError_t launch_depthwise(const DepthwiseParams &p, bool out_i32, int grid, hipStream_t stream)
{
    // the 3x3 kernel addresses input and output with 32-bit byte offsets and keeps the top of that range free
    const bool banked = p.KH == 3 && p.KW == 3 && p.dh == 1 && p.dw == 1 && p.sh == p.sw && (p.sw == 1 || p.sw == 2) &&
                        (int64_t)p.N * p.H * p.W * p.C * 4 < 0x7fffffffll && p.M * p.C * 4 < 0x7fffffffll;
    if (banked) {
        const int cus = device_cus();
        const int R = p.sw == 1 ? 4 : 2;
        const int ngroups = (p.C + kDwChannels - 1) / kDwChannels;
        // Workgroups per channel group, and channel groups served at a time: every group gets the same number of
        // workgroups so that all finish together.
        int wgs_per_group = cus / ngroups;
        int group_slots = ngroups;
        if (wgs_per_group < 1) {
            wgs_per_group = 1;
            group_slots = cus;
        }
        const int band_pairs = (p.OH + 2 * R - 1) / (2 * R);
        // Column segments.  A workgroup deals its run of tasks to its wavefronts in rounds, and a wavefront without a
        // task in the last round idles while the others work: the number of rounds times the columns a task loads
        // (its segment and the window's restart) is what a workgroup takes.  The segment count with the smallest such
        // product among segments of 8 to 24 columns: shorter ones restart the window too often.
        int nseg = 1, seg_len = p.OW;
        int64_t best = -1;
        for (int ns = 1; ns <= p.OW; ++ns) {
            const int sl = (p.OW + ns - 1) / ns;
            if (ns > 1 && sl < 8)
                break;
            if (sl > 24 && (p.OW + ns) / (ns + 1) >= 8)
                continue;       // long segments let the wavefronts that share halo rows drift apart (measured: 1 % slower)
            const int ns_eff = (p.OW + sl - 1) / sl;
            const int64_t tasks = (int64_t)p.N * band_pairs * ns_eff;
            const int64_t per_wg = (tasks + wgs_per_group - 1) / wgs_per_group;
            const int64_t cost = ((per_wg + kWaves - 1) / kWaves) * (sl + 3);
            if (best < 0 || cost < best) {
                best = cost;
                nseg = ns_eff;
                seg_len = sl;
            }
        }
        const int g3 = wgs_per_group * group_slots;
#define AXC_DW_LAUNCH_AS(S_, R_, I32_, FQ_, EPI_)                                                                     \
    launch_with_lds(depthwise_lut3x3_kernel<S_, R_, I32_, FQ_, EPI_>, g3, kDwLdsBytes, stream, p, seg_len, nseg,         \
                    wgs_per_group, group_slots)
#define AXC_DW_LAUNCH(S_, R_)                                                                                        \
    (out_i32    ? AXC_DW_LAUNCH_AS(S_, R_, true, false, false)                                                           \
     : p.lq_dev ? AXC_DW_LAUNCH_AS(S_, R_, false, true, true)                                                            \
     : epi      ? AXC_DW_LAUNCH_AS(S_, R_, false, false, true)                                                           \
                : AXC_DW_LAUNCH_AS(S_, R_, false, false, false))
        const bool epi = p.bias != nullptr || p.relu != 0;
        return p.sw == 1 ? AXC_DW_LAUNCH(1, 4) : AXC_DW_LAUNCH(2, 2);
#undef AXC_DW_LAUNCH
#undef AXC_DW_LAUNCH_AS
    }
    return out_i32 ? launch_with_lds(depthwise_lut_kernel<true>, grid, kTableBytes, stream, p)
                   : launch_with_lds(depthwise_lut_kernel<false>, grid, kTableBytes, stream, p);
}

// ---- LDS gather-rate probe: conflict-free ds_read_u16, 16 wavefronts per CU ------------------
// Each lane reads its own dword-aligned uint16 (64 consecutive dwords per wavefront), 16 independent
// reads in flight per iteration.  The sum is written out so nothing is optimized away.
__global__ void __launch_bounds__(kBlockThreads) lds_gather_probe_kernel(uint32_t *out, int iters)
{
    uint32_t *l32 = reinterpret_cast<uint32_t *>(lds_dw);
    for (int i = threadIdx.x; i < kTableBytes / 4; i += blockDim.x)
        l32[i] = (uint32_t)i * 2654435761u;
    __syncthreads();
    const uint32_t base = (uint32_t)(threadIdx.x & 63) * 4u + (uint32_t)(threadIdx.x >> 6) * 256u;
    uint32_t acc = 0;
    for (int it = 0; it < iters; ++it) {
        uint32_t v[16];
#pragma unroll
        for (int r = 0; r < 16; ++r)
            asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(v[r]) : "v"(base), "n"(r * 4096));
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]),
                       "+v"(v[7]), "+v"(v[8]), "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]),
                       "+v"(v[14]), "+v"(v[15]));
#pragma unroll
        for (int r = 0; r < 16; ++r)
            acc += v[r];
    }
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

// Streaming ds_read_b128: every lane reads its own 16 bytes of a contiguous 1 KiB per wavefront, no bank
// conflicts.  The byte rate is the ceiling of the LDS read port for the access width the LUT-GEMM uses.
__global__ void __launch_bounds__(kBlockThreads) lds_stream_probe_kernel(uint32_t *out, int iters)
{
    uint32_t *l32 = reinterpret_cast<uint32_t *>(lds_dw);
    for (int i = threadIdx.x; i < kTableBytes / 4; i += blockDim.x)
        l32[i] = (uint32_t)i * 2654435761u;
    __syncthreads();
    // a wavefront walks 8 x 1 KiB per iteration inside its own 16 KiB window
    const uint32_t base = (uint32_t)(threadIdx.x & 63) * 16u + ((uint32_t)(threadIdx.x >> 6) & 7u) * 16384u;
    uint32_t acc = 0;
    for (int it = 0; it < iters; ++it) {
        u32x4 v[8];
#pragma unroll
        for (int r = 0; r < 8; ++r)
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v[r]) : "v"(base), "n"(r * 1024));
        asm volatile("s_waitcnt lgkmcnt(0)"
                     : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]));
#pragma unroll
        for (int r = 0; r < 8; ++r)
            acc += v[r].x ^ v[r].w;
    }
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = acc;
}

// VALU issue-rate probe: the accumulate instructions of the dense kernel and nothing else, in its own occupancy (one
// workgroup of 8 wavefronts per CU, two per SIMD).  MIX 0: v_add_u32 / v_add_u32_sdwa alternating (one per
// table entry); MIX 1: v_add3_u32, v_add_u32_sdwa, v_add_u32_sdwa (three per four entries).  32 independent
// accumulators, so no instruction waits for the one before it.
template <int MIX>
__global__ void __launch_bounds__(kDenseThreads) valu_issue_probe_kernel(uint32_t *out, int iters)
{
    uint32_t acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i)
        acc[i] = threadIdx.x + i;
    uint32_t s0 = threadIdx.x * 2654435761u, s1 = s0 ^ 0x9e3779b9u;
    for (int it = 0; it < iters; ++it) {
        // 512 instructions between two branches: the loop overhead stays below half a percent
#pragma unroll
        for (int u = 0; u < 16; ++u)
#pragma unroll
        for (int i = 0; i < 32; i += 4) {
            if (MIX == 0)
                asm volatile("v_add_u32 %0, %0, %4\n\t"
                             "v_add_u32_sdwa %1, %1, %4 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add_u32 %2, %2, %5\n\t"
                             "v_add_u32_sdwa %3, %3, %5 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1"
                             : "+v"(acc[i]), "+v"(acc[i + 1]), "+v"(acc[i + 2]), "+v"(acc[i + 3])
                             : "v"(s0), "v"(s1));
            else
                asm volatile("v_add3_u32 %0, %0, %4, %5\n\t"
                             "v_add_u32_sdwa %1, %1, %4 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add_u32_sdwa %2, %2, %5 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add3_u32 %3, %3, %5, %4"
                             : "+v"(acc[i]), "+v"(acc[i + 1]), "+v"(acc[i + 2]), "+v"(acc[i + 3])
                             : "v"(s0), "v"(s1));
        }
    }
    uint32_t sum = 0;
#pragma unroll
    for (int i = 0; i < 32; ++i)
        sum += acc[i];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = sum;
}

hipError_t run_valu_issue_peak(double *lane_ops_per_second, int mix, hipStream_t stream)
{
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    uint32_t *out = nullptr;
    e = hipMalloc(&out, (size_t)cus * kDenseThreads * sizeof(uint32_t));
    if (e != hipSuccess) return e;
    auto probe = mix == 0 ? valu_issue_probe_kernel<0> : valu_issue_probe_kernel<1>;
    // the dense kernel's LDS size: one workgroup per CU
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(probe), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kDenseLdsBytes);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const int iters = 1500;
    if (e == hipSuccess) {
        hipLaunchKernelGGL(probe, dim3(cus), dim3(kDenseThreads), kDenseLdsBytes, stream, out, 20);
        e = hipEventRecord(e0, stream);
    }
    if (e == hipSuccess) {
        hipLaunchKernelGGL(probe, dim3(cus), dim3(kDenseThreads), kDenseLdsBytes, stream, out, iters);
        e = hipEventRecord(e1, stream);
    }
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e == hipSuccess && ms > 0.0f)
        *lane_ops_per_second = (double)cus * kDenseThreads * (double)iters * 512.0 / (ms * 1e-3);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(out);
    return e;
}

// The whole instruction mix of a LUT-GEMM lookup instruction, and nothing else: one v_perm_b32 (address), one
// ds_read_b128 through a rolling window of eight (16 different 16-byte chunks of 256-byte rows per LDS pass: no bank
// conflict), and the six accumulate instructions of its eight table entries (v_add3_u32 on whole dwords of two
// lookups, v_add_u32_sdwa on their high halves), in the LUT-GEMM's occupancy (one workgroup of 8 wavefronts and all of
// the LDS per CU).  Neither the LDS read port nor the vector ALUs alone say what a SIMD can do when a wavefront pair
// has to issue both kinds: this is the rate a kernel built of exactly these instructions, without fills, activations,
// barriers, prologue or epilogue, reaches.
extern __shared__ __align__(16) unsigned char mix_lds[];
__global__ void __launch_bounds__(kDenseThreads) lookup_mix_probe_kernel(uint32_t *out, int iters)
{
    typedef uint32_t u32x4p __attribute__((ext_vector_type(4)));
    uint32_t *const l32 = reinterpret_cast<uint32_t *>(mix_lds);
    for (int i = threadIdx.x; i < 32768; i += blockDim.x)
        l32[i] = (uint32_t)i * 2654435761u;
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63u;
    // a row per lane (any of 256), the lane's own chunk of it: byte 1 of the address comes out of `rows`, byte 0
    // out of `chunks`, as in the kernels
    const uint32_t rows = ((lane * 37u) & 255u) * 0x01010101u;
    const uint32_t chunks = ((lane & 15u) << 4) * 0x01010101u;
    const uint32_t sel = 0x0c0c0400u;   // byte 0 <- chunks byte 0, byte 1 <- rows byte 0
    uint32_t acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
        acc[i] = threadIdx.x + i;
    u32x4p v[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        uint32_t a;
        asm volatile("v_perm_b32 %0, %2, %3, %4\n\tds_read_b128 %1, %0 offset:%5"
                     : "=&v"(a), "=v"(v[s]) : "v"(rows), "v"(chunks), "v"(sel), "n"(s * 4096));
    }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int rep = 0; rep < 4; ++rep)
#pragma unroll
            for (int s = 0; s < 8; s += 2) {   // two lookup instructions at a time, as the phase bodies do
                // few, long asm statements: the compiler puts an s_nop between two of them
                uint32_t *const a = &acc[(s & 2) * 4];
                const uint32_t x0 = v[s][0], x1 = v[s][1], x2 = v[s][2], x3 = v[s][3];
                const uint32_t y0 = v[s + 1][0], y1 = v[s + 1][1], y2 = v[s + 1][2], y3 = v[s + 1][3];
                asm volatile("s_waitcnt lgkmcnt(6)\n\t"
                             "v_add3_u32 %0, %0, %8, %12\n\t"
                             "v_add_u32_sdwa %1, %1, %8 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add_u32_sdwa %1, %1, %12 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add3_u32 %2, %2, %9, %13\n\t"
                             "v_add_u32_sdwa %3, %3, %9 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add_u32_sdwa %3, %3, %13 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add3_u32 %4, %4, %10, %14\n\t"
                             "v_add_u32_sdwa %5, %5, %10 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add_u32_sdwa %5, %5, %14 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add3_u32 %6, %6, %11, %15\n\t"
                             "v_add_u32_sdwa %7, %7, %11 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1\n\t"
                             "v_add_u32_sdwa %7, %7, %15 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:WORD_1"
                             : "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7])
                             : "v"(x0), "v"(x1), "v"(x2), "v"(x3), "v"(y0), "v"(y1), "v"(y2), "v"(y3));
                uint32_t a0, a1;
                asm volatile("v_perm_b32 %0, %4, %5, %6\n\tds_read_b128 %2, %0 offset:%7\n\t"
                             "v_perm_b32 %1, %4, %5, %6\n\tds_read_b128 %3, %1 offset:%8"
                             : "=&v"(a0), "=&v"(a1), "=&v"(v[s]), "=&v"(v[s + 1])
                             : "v"(rows), "v"(chunks), "v"(sel), "n"(s * 4096), "n"(s * 4096 + 4096));
            }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]),
                 "+v"(v[6]), "+v"(v[7]));
    uint32_t sum = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i)
        sum += acc[i];
#pragma unroll
    for (int s = 0; s < 8; ++s)
        sum += v[s][0] ^ v[s][3];
    out[(size_t)blockIdx.x * blockDim.x + threadIdx.x] = sum;
}

hipError_t run_lookup_mix_peak(double *lookups_per_second, hipStream_t stream)
{
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    uint32_t *out = nullptr;
    e = hipMalloc(&out, (size_t)cus * kDenseThreads * sizeof(uint32_t));
    if (e != hipSuccess) return e;
    const int lds_bytes = kDenseLdsBytes + kDenseParkBytes;   // what a LUT-GEMM workgroup takes: one workgroup per CU
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(lookup_mix_probe_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const int iters = 3000;
    if (e == hipSuccess) {
        hipLaunchKernelGGL(lookup_mix_probe_kernel, dim3(cus), dim3(kDenseThreads), lds_bytes, stream, out, 100);
        e = hipEventRecord(e0, stream);
    }
    if (e == hipSuccess) {
        hipLaunchKernelGGL(lookup_mix_probe_kernel, dim3(cus), dim3(kDenseThreads), lds_bytes, stream, out, iters);
        e = hipEventRecord(e1, stream);
    }
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    // 32 lookup instructions per iteration and wavefront, 64 lanes x 8 table entries each
    if (e == hipSuccess && ms > 0.0f)
        *lookups_per_second = (double)cus * (kDenseThreads / 64) * (double)iters * 32.0 * 512.0 / (ms * 1e-3);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(out);
    return e;
}

hipError_t run_lds_gather_peak(double *lookups_per_second, hipStream_t stream, bool stream_b128)
{
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    uint32_t *out = nullptr;
    e = hipMalloc(&out, (size_t)cus * kBlockThreads * sizeof(uint32_t));
    if (e != hipSuccess) return e;
    auto probe = stream_b128 ? lds_stream_probe_kernel : lds_gather_probe_kernel;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(probe), hipFuncAttributeMaxDynamicSharedMemorySize,
                            kTableBytes);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const int iters = 8000;
    if (e == hipSuccess) {
        hipLaunchKernelGGL(probe, dim3(cus), dim3(kBlockThreads), kTableBytes, stream, out, 100);
        e = hipEventRecord(e0, stream);
    }
    if (e == hipSuccess) {
        hipLaunchKernelGGL(probe, dim3(cus), dim3(kBlockThreads), kTableBytes, stream, out, iters);
        e = hipEventRecord(e1, stream);
    }
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e == hipSuccess && ms > 0.0f)
        // gather mode: 16 two-byte lookups per lane and iteration; stream mode: 8 x 16 bytes (the result is bytes/s)
        *lookups_per_second = (double)cus * kBlockThreads * (double)iters * (stream_b128 ? 128.0 : 16.0) / (ms * 1e-3);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(out);
    return e;
}

} // namespace axc
