// Depthwise LUT convolution (channel multiplier 1) and the LDS gather-rate probe.
#include "axconv_internal.h"

namespace axc {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

extern __shared__ __align__(16) unsigned char lds_dw[];

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
                    v = p.x[(((int64_t)n * p.H + ih) * p.W + iw) * p.C + c];
                psum = __fadd_rn(psum, v);
                const uint32_t a = quantize_code(v, p.in_offset, p.in_inv_scale);
                const uint32_t b = p.wcodes[(int64_t)tap * p.C + c];
                acc += (int32_t)table[b * 256u + a];
            }
        if (OUT_I32) {
            p.out_i[idx] = acc;
        } else {
            const float t0 = __fmul_rn((float)acc, p.s1xs2);
            const float t1 = __fmul_rn(p.m2, psum);
            const float t2 = __fadd_rn(t0, t1);
            const float t3 = __fmul_rn(p.m1, p.fsum[c]);
            const float t4 = __fadd_rn(t2, t3);
            p.out_f[idx] = __fsub_rn(t4, p.k_m1xm2);
        }
    }
}

// 3x3 filters, dilation 1, column stride SW in {1, 2}: a thread owns one channel of a run of consecutive output
// pixels of one output row and slides the 3x3 window along it.  Every input value is loaded and quantized once
// per window row instead of once per tap, and the nine filter codes of the channel live in registers as table row
// offsets.  Loads and stores go through buffer descriptors with 32-bit offsets: a column or row outside the image
// gets an offset past the end of the buffer and reads 0.0f without a branch, and 0.0f quantizes to the zero-point
// code, which is what a tap outside the image looks up.  Same results as depthwise_lut_kernel: taps in (kh, kw)
// order, zeros (code = zero point) outside the image.
typedef __amdgpu_buffer_rsrc_t dw_rsrc_t;
__device__ __forceinline__ dw_rsrc_t dw_make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

template <int SW, bool OUT_I32>
__global__ void __launch_bounds__(kBlockThreads) depthwise_lut3x3_kernel(const DepthwiseParams p, const int seg_len,
                                                                          const int nseg)
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

    // the launcher has checked that input and output are below 2 GiB, so offsets from 0x70000000 up are outside
    constexpr uint32_t kOutside = 0x70000000u;
    const uint32_t x_bytes = (uint32_t)((int64_t)p.N * p.H * p.W * p.C * 4);
    const uint32_t o_bytes = (uint32_t)(p.M * p.C * 4);
    const dw_rsrc_t x_rsrc = dw_make_rsrc(p.x, x_bytes);
    const dw_rsrc_t o_rsrc = dw_make_rsrc(OUT_I32 ? static_cast<const void *>(p.out_i) : static_cast<const void *>(p.out_f), o_bytes);
    const uint32_t col_bytes = (uint32_t)p.C * 4u;           // bytes between neighbouring pixels of a row

    const int64_t items = (int64_t)p.N * p.OH * nseg * p.C;   // (output row segment, channel), channel fastest
    // Neighbouring output rows read the same input rows.  Workgroups go to the 8 XCDs round-robin and every XCD
    // has its own L2, so each XCD gets one contiguous band of output rows (whole rows): an input row is then
    // fetched from memory by one L2 instead of by up to three.
    const int64_t per_row = (int64_t)nseg * p.C;
    const int64_t rows_total = (int64_t)p.N * p.OH;
    int64_t last = items, stride = (int64_t)gridDim.x * blockDim.x;
    int64_t start = (int64_t)blockIdx.x * blockDim.x + tid;
    if ((gridDim.x & 7) == 0) {
        const int xcd = blockIdx.x & 7;
        const int64_t rows_per_xcd = (rows_total + 7) / 8;
        const int64_t first = rows_per_xcd * xcd * per_row;
        last = rows_per_xcd * (xcd + 1) * per_row;
        last = last < items ? last : items;
        stride = (int64_t)(gridDim.x >> 3) * blockDim.x;
        start = first + (int64_t)(blockIdx.x >> 3) * blockDim.x + tid;
    }
    constexpr int U = 4;                 // outputs per group
    constexpr int NEW = U * SW;          // columns that enter the window per group
    constexpr int CARRY = 3 - SW;        // columns the next group shares with this one
    for (int64_t item = start; item < last; item += stride) {
        // items < 2^31 here (the output is below 2 GiB): 32-bit divisions, a fraction of the cost of 64-bit ones
        const uint32_t it32 = (uint32_t)item;
        const uint32_t rs = it32 / (uint32_t)p.C;
        const int c = (int)(it32 - rs * (uint32_t)p.C);
        const uint32_t row = rs / (uint32_t)nseg;              // n * OH + oh
        const int seg = (int)(rs - row * (uint32_t)nseg);
        const int n = (int)(row / (uint32_t)p.OH);
        const int oh = (int)(row - (uint32_t)n * (uint32_t)p.OH);
        const int ow0 = seg * seg_len;
        const int len = (ow0 + seg_len < p.OW ? ow0 + seg_len : p.OW) - ow0;
        const int ih0 = oh * p.sh - p.ph;

        uint32_t wrow[9];                                      // byte offset of the table row of each tap's filter code
#pragma unroll
        for (int t = 0; t < 9; ++t)
            wrow[t] = (uint32_t)p.wcodes[t * p.C + c] * 512u;
        const float t3 = OUT_I32 ? 0.0f : __fmul_rn(p.m1, p.fsum[c]);
        uint32_t rowbase[3];                                   // byte offset of (n, ih, 0, c); outside for a row that is
#pragma unroll
        for (int kh = 0; kh < 3; ++kh) {
            const int ih = ih0 + kh;
            rowbase[kh] = (unsigned)ih < (unsigned)p.H
                              ? (uint32_t)((((int64_t)n * p.H + ih) * p.W * p.C + c) * 4)
                              : 0x80000000u;
        }
        const int iw0 = ow0 * SW - p.pw;                       // input column under tap kw = 0 of the first output
        auto col_off = [&](int iw) {                           // byte offset of column iw inside a row; outside if none
            return (unsigned)iw < (unsigned)p.W ? (uint32_t)iw * col_bytes : kOutside;
        };
        auto load = [&](int kh, uint32_t coff) {
            return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(x_rsrc, (int)(rowbase[kh] + coff), 0, 0));
        };
        float cv[3][CARRY + NEW];                              // window columns of the group: values ...
        uint32_t ca[3][CARRY + NEW];                           // ... and activation codes * 2 (byte offset in a table row)
#pragma unroll
        for (int t = 0; t < CARRY; ++t) {
            const uint32_t coff = col_off(iw0 + t);
#pragma unroll
            for (int kh = 0; kh < 3; ++kh) {
                cv[kh][t] = load(kh, coff);
                ca[kh][t] = quantize_code(cv[kh][t], p.in_offset, p.in_inv_scale) * 2u;
            }
        }
        // the columns that enter the window with the next group are loaded one group ahead
        float pf[3][NEW];
        auto prefetch = [&](int jfirst) {                      // new columns of outputs jfirst .. jfirst + U - 1
#pragma unroll
            for (int t = 0; t < NEW; ++t) {
                const uint32_t coff = col_off(iw0 + jfirst * SW + CARRY + t);
#pragma unroll
                for (int kh = 0; kh < 3; ++kh)
                    pf[kh][t] = load(kh, coff);
            }
        };
        prefetch(0);
        uint32_t o_off = (uint32_t)((((int64_t)row * p.OW + ow0) * p.C + c) * 4);
        for (int j0 = 0; j0 < len; j0 += U) {
#pragma unroll
            for (int kh = 0; kh < 3; ++kh)
#pragma unroll
                for (int t = 0; t < NEW; ++t) {
                    cv[kh][CARRY + t] = pf[kh][t];
                    ca[kh][CARRY + t] = quantize_code(pf[kh][t], p.in_offset, p.in_inv_scale) * 2u;
                }
            if (j0 + U < len)
                prefetch(j0 + U);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (j0 + u >= len)
                    break;
                int32_t acc = 0;
                float psum = 0.0f;
#pragma unroll
                for (int kh = 0; kh < 3; ++kh)
#pragma unroll
                    for (int kw = 0; kw < 3; ++kw) {
                        psum = __fadd_rn(psum, cv[kh][u * SW + kw]);
                        acc += (int32_t)*reinterpret_cast<const uint16_t *>(lds_dw + wrow[kh * 3 + kw] + ca[kh][u * SW + kw]);
                    }
                uint32_t outw;
                if (OUT_I32) {
                    outw = (uint32_t)acc;
                } else {
                    const float t0 = __fmul_rn((float)acc, p.s1xs2);
                    const float t1 = __fmul_rn(p.m2, psum);
                    const float t2 = __fadd_rn(t0, t1);
                    const float t4 = __fadd_rn(t2, t3);
                    outw = __float_as_uint(__fsub_rn(t4, p.k_m1xm2));
                }
                __builtin_amdgcn_raw_buffer_store_b32(outw, o_rsrc, (int)o_off, 0, 2); // nt: streamed past the caches, which
                                                                                    // the input rows three output rows share need
                o_off += col_bytes;
            }
#pragma unroll
            for (int kh = 0; kh < 3; ++kh)
#pragma unroll
                for (int t = 0; t < CARRY; ++t) {
                    cv[kh][t] = cv[kh][NEW + t];
                    ca[kh][t] = ca[kh][NEW + t];
                }
        }
    }
}

template <typename Kernel, typename... Args>
static hipError_t launch_with_table_lds(Kernel kernel, int grid, hipStream_t stream, Args... args)
{
    const hipError_t e = set_max_dynamic_lds_once(reinterpret_cast<const void *>(kernel), kTableBytes);
    if (e != hipSuccess)
        return e;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(kBlockThreads), kTableBytes, stream, args...);
    return hipGetLastError();
}

hipError_t launch_depthwise(const DepthwiseParams &p, bool out_i32, int grid, hipStream_t stream)
{
    // the sliding kernel addresses input and output with 32-bit byte offsets and keeps the top of that range free
    const bool sliding = p.KH == 3 && p.KW == 3 && p.dh == 1 && p.dw == 1 && (p.sw == 1 || p.sw == 2) &&
                         (int64_t)p.N * p.H * p.W * p.C * 4 < 0x70000000ll && p.M * p.C * 4 < 0x70000000ll;
    if (sliding) {
        // runs of at most 32 (stride 2: 16) output pixels per thread: enough items to balance the CUs, few window
        // restarts, and the rows in flight on an XCD at one time still fit its L2
        const int run = p.sw == 1 ? 32 : 16;
        const int nseg = (p.OW + run - 1) / run;
        const int seg_len = (p.OW + nseg - 1) / nseg;
        const int cus = device_cus();
        const int64_t items = (int64_t)p.N * p.OH * nseg * p.C;
        const int64_t blocks = (items + kBlockThreads - 1) / kBlockThreads;
        int g3 = (int)(blocks < cus ? blocks : cus);
        if (g3 >= 64)
            g3 &= ~7;   // a multiple of 8 workgroups: the kernel then keeps bands of output rows on one XCD each
        if (p.sw == 1)
            return out_i32 ? launch_with_table_lds(depthwise_lut3x3_kernel<1, true>, g3, stream, p, seg_len, nseg)
                           : launch_with_table_lds(depthwise_lut3x3_kernel<1, false>, g3, stream, p, seg_len, nseg);
        return out_i32 ? launch_with_table_lds(depthwise_lut3x3_kernel<2, true>, g3, stream, p, seg_len, nseg)
                       : launch_with_table_lds(depthwise_lut3x3_kernel<2, false>, g3, stream, p, seg_len, nseg);
    }
    return out_i32 ? launch_with_table_lds(depthwise_lut_kernel<true>, grid, stream, p)
                   : launch_with_table_lds(depthwise_lut_kernel<false>, grid, stream, p);
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
