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

hipError_t launch_depthwise(const DepthwiseParams &p, bool out_i32, int grid, hipStream_t stream)
{
    hipError_t e;
    if (out_i32) {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(depthwise_lut_kernel<true>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kTableBytes);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(depthwise_lut_kernel<true>, dim3(grid), dim3(kBlockThreads), kTableBytes, stream, p);
    } else {
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(depthwise_lut_kernel<false>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, kTableBytes);
        if (e != hipSuccess) return e;
        hipLaunchKernelGGL(depthwise_lut_kernel<false>, dim3(grid), dim3(kBlockThreads), kTableBytes, stream, p);
    }
    return hipGetLastError();
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

hipError_t run_lds_gather_peak(double *lookups_per_second, hipStream_t stream)
{
    int dev = 0, cus = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return e;
    uint32_t *out = nullptr;
    e = hipMalloc(&out, (size_t)cus * kBlockThreads * sizeof(uint32_t));
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void *>(lds_gather_probe_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, kTableBytes);
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (e == hipSuccess) e = hipEventCreate(&e0);
    if (e == hipSuccess) e = hipEventCreate(&e1);
    const int iters = 8000;
    if (e == hipSuccess) {
        hipLaunchKernelGGL(lds_gather_probe_kernel, dim3(cus), dim3(kBlockThreads), kTableBytes, stream, out, 100);
        e = hipEventRecord(e0, stream);
    }
    if (e == hipSuccess) {
        hipLaunchKernelGGL(lds_gather_probe_kernel, dim3(cus), dim3(kBlockThreads), kTableBytes, stream, out, iters);
        e = hipEventRecord(e1, stream);
    }
    if (e == hipSuccess) e = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e == hipSuccess && ms > 0.0f)
        *lookups_per_second = (double)cus * kBlockThreads * (double)iters * 16.0 / (ms * 1e-3);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    (void)hipFree(out);
    return e;
}

} // namespace axc
