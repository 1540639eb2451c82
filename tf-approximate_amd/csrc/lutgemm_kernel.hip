// Dense LUT-GEMM for gfx950: implicit-GEMM gather + table lookups out of LDS + fused epilogue.
//
// One workgroup (16 wavefronts) owns a CU and its 160 KiB of LDS:
//   [0, 128 KiB)        the whole truth table, weight-code major: row b holds T[a][b] for a = 0..255
//   [128 KiB, 160 KiB)  the "expanded rows": for the 64 weight slots of the current fill,
//                       E[phys_row(a)][slot] = T[a][code(slot)], 128 bytes per activation code
//
// A fill takes 64 filter entries (KS consecutive input channels x NT output columns, KS * NT = 64),
// copies the table row of each entry into the expanded area transposed (derive phase), then every
// lane looks up, for each of its R = 64 / NT output pixels, the expanded row of its activation code
// with ds_read_b128: eight table entries per LDS access instead of one, and the 16-byte chunks the
// lanes of a wavefront touch in one instruction are rotated by lane so they fall into different
// banks whatever the activation codes are.  Sums are exact int32.
//
// Restates, as one fused kernel, what the reference does in ApproxConvIm2ColKernel +
// ApproxConvGEMMKernel (tf2/src/approx_nn_conv_kernels.cpp:215-296) per chunk.
#include "axconv_internal.h"
#include "lookup_asm.inc"

namespace axc {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

extern __shared__ __align__(16) unsigned char lds[];

// Four table-row reads in flight, then one wait: the compiler would serialize them.
__device__ __forceinline__ void lds_read4_b64(uint64_t (&v)[4], const uint32_t (&addr)[4])
{
    asm volatile("ds_read_b64 %0, %4\n\t"
                 "ds_read_b64 %1, %5\n\t"
                 "ds_read_b64 %2, %6\n\t"
                 "ds_read_b64 %3, %7\n\t"
                 "s_waitcnt lgkmcnt(0)"
                 : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3])
                 : "v"(addr[0]), "v"(addr[1]), "v"(addr[2]), "v"(addr[3])
                 : "memory");
}

template <int NT, bool OUT_I32>
__global__ void __launch_bounds__(kBlockThreads) lutgemm_expand_kernel(const DenseParams p)
{
    constexpr int R = 64 / NT;        // output pixels per lane
    constexpr int KS = 64 / NT;       // input channels per fill
    constexpr int SETS = NT / 8;      // 8-column groups per pixel
    constexpr int SUBS = 4 / KS;      // fills per channel quad
    constexpr int LOG_SETS = (SETS == 8) ? 3 : (SETS == 4) ? 2 : 1;

    const ConvGeom &g = p.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: row activity branches on SGPRs

    // ---- stage the truth table (once per workgroup; the workgroup is persistent) ----
    {
        const u32x4 *src = reinterpret_cast<const u32x4 *>(p.tableT);
        u32x4 *dst = reinterpret_cast<u32x4 *>(lds);
#pragma unroll
        for (int i = 0; i < kTableBytes / 16 / kBlockThreads; ++i)
            dst[tid + i * kBlockThreads] = src[tid + i * kBlockThreads];
    }

    // ---- lane constants ----
    const int c0 = lane & 7;
    uint32_t choff[8];   // byte offset of the chunk this lane reads at step s
#pragma unroll
    for (int s = 0; s < 8; ++s)
        choff[s] = (uint32_t)kTableBytes + ((uint32_t)((c0 + s) & 7) << 4);
    // The chunk of step s belongs to input channel kk_s = ((c0 + s) & 7) >> LOG_SETS of the fill.
    // KS == 4: kk_s = (kk0 + ((p0 + s) >> 1)) & 3 with kk0 = c0 >> 1, p0 = c0 & 1, so after rotating the
    //          activation dword right by kk0 bytes (and by p0 more for odd s) the byte index is the
    //          compile-time constant s >> 1.
    // KS == 2: kk_s is one bit; it is kept as a per-step lane mask.
    const uint32_t rot_kk0 = (uint32_t)(c0 >> 1) << 3;
    const uint32_t rot_p0 = (uint32_t)(c0 & 1) << 3;
    bool kk_hi[8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
        kk_hi[s] = ((((c0 + s) & 7) >> LOG_SETS) & 1) != 0;
    // derive phase: lane transposes activation codes 4*lane .. 4*lane+3 for slots 4*jq .. 4*jq+3
    const int jq = (lane + wave) & 15;
    const uint32_t rd_off = (uint32_t)lane * 8u;
    const uint32_t wr_off = (uint32_t)kTableBytes + (uint32_t)lane * 128u + (uint32_t)jq * 8u;

    const int taps = g.KH * g.KW;
    const int ntiles = p.plan.n_row_tiles * p.plan.n_col_tiles;
    const int fills = p.plan.fills;
    const int rowstep = g.C4 * g.W; // dwords between input rows in xq

    for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int ct = tile % p.plan.n_col_tiles;
        const int rt = tile / p.plan.n_col_tiles;
        const int64_t row0 = (int64_t)rt * p.plan.rows_per_tile;
        const int64_t row_end = (row0 + p.plan.rows_per_tile < g.M) ? row0 + p.plan.rows_per_tile : g.M;

        // ---- per-pixel geometry ----
        int32_t pbase[R];  // dword index in xq of tap (0, 0), channel quad 0 (may point outside the image)
        int hw0[R];        // (ih0 << 16) | (iw0 & 0xffff): input coordinates of tap (0, 0)
        bool rvalid[R];    // this lane's pixel exists
        bool ractive[R];   // some lane of this wavefront has a pixel (wave-uniform)
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t wrow = row0 + (int64_t)(r * kWaves + wave) * 64;
            ractive[r] = wrow < row_end;
            const int64_t m = wrow + lane;
            rvalid[r] = m < row_end;
            const int64_t mm = rvalid[r] ? m : row0;
            const int n = (int)(mm / ((int64_t)g.OH * g.OW));
            const int rem = (int)(mm - (int64_t)n * g.OH * g.OW);
            const int oh = rem / g.OW;
            const int ow = rem - oh * g.OW;
            const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
            pbase[r] = (n * g.H + ih0) * rowstep + iw0;
            hw0[r] = (ih0 << 16) | (iw0 & 0xffff);
        }

        int32_t acc[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                acc[r][j] = 0;

        const uint16_t *wq_tile = p.wq + (size_t)ct * fills * 64 + jq * 4;

        // ---- load cursor: (tap, quad) of the activation dwords to fetch next ----
        int tap_n = 0, q_n = 0, kh_n = 0, kw_n = 0;
        bool inb_n[R];
        int32_t idx_n[R];
        auto tap_setup = [&]() {
            const int dh = kh_n * g.dh, dw = kw_n * g.dw;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int ih = (hw0[r] >> 16) + dh;
                const int iw = (int)(int16_t)(hw0[r] & 0xffff) + dw;
                inb_n[r] = rvalid[r] && (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
                idx_n[r] = inb_n[r] ? pbase[r] + dh * rowstep + dw : 0;
            }
        };
        uint32_t a4n[R];
        auto issue_act_loads = [&]() {
            // unconditional loads (index 0 when outside the image) keep the number of outstanding
            // loads static, so waits on older loads do not have to drain these
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const uint32_t v = p.xq[idx_n[r] + (inb_n[r] ? q_n * g.W : 0)];
                a4n[r] = inb_n[r] ? v : p.zp4;
            }
        };
        auto advance_cursor = [&]() {
            if (++q_n == g.C4) {
                q_n = 0;
                ++tap_n;
                if (++kw_n == g.KW) { kw_n = 0; ++kh_n; }
                if (tap_n < taps)
                    tap_setup();
            }
        };

        // derive phase, split so the table-row reads can run before the barrier that frees the
        // expanded area and only the four writes sit between the two barriers
        u32x2 o[4];
        auto derive_read = [&](const u32x2 wc) {
            const uint32_t code[4] = {wc.x & 0xffffu, wc.x >> 16, wc.y & 0xffffu, wc.y >> 16};
            uint32_t addr[4];
            bool none[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                none[i] = code[i] == kNullWeight;
                addr[i] = (none[i] ? 0u : code[i]) * 512u + rd_off;
            }
            uint64_t v[4];
            lds_read4_b64(v, addr);
            uint32_t x[4], y[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                x[i] = none[i] ? 0u : (uint32_t)v[i];
                y[i] = none[i] ? 0u : (uint32_t)(v[i] >> 32);
            }
            o[0].x = __builtin_amdgcn_perm(x[1], x[0], 0x05040100u);
            o[0].y = __builtin_amdgcn_perm(x[3], x[2], 0x05040100u);
            o[1].x = __builtin_amdgcn_perm(x[1], x[0], 0x07060302u);
            o[1].y = __builtin_amdgcn_perm(x[3], x[2], 0x07060302u);
            o[2].x = __builtin_amdgcn_perm(y[1], y[0], 0x05040100u);
            o[2].y = __builtin_amdgcn_perm(y[3], y[2], 0x05040100u);
            o[3].x = __builtin_amdgcn_perm(y[1], y[0], 0x07060302u);
            o[3].y = __builtin_amdgcn_perm(y[3], y[2], 0x07060302u);
        };
        auto derive_write = [&]() {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                *reinterpret_cast<u32x2 *>(lds + wr_off + (uint32_t)i * (64u * 128u)) = o[i];
        };

        // ---- prologue: activations of quad 0, weights of fill 0 -> expanded rows of fill 0 ----
        uint32_t a4[R];
        tap_setup();
        issue_act_loads();
        u32x2 wn = *reinterpret_cast<const u32x2 *>(wq_tile);
        __syncthreads(); // table staged / previous tile's lookups done
        derive_read(wn);
        derive_write();
        __syncthreads();
#pragma unroll
        for (int r = 0; r < R; ++r)
            a4[r] = a4n[r];
        advance_cursor();
        if (tap_n < taps)
            issue_act_loads();
        if (fills > 1)
            wn = *reinterpret_cast<const u32x2 *>(wq_tile + 64);

        int sub = 0;
        for (int fill = 0; fill < fills; ++fill) {
            // ---- lookups of this fill ----
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (!ractive[r])
                    continue;
                // row offsets (128 B per activation code) of the channels of this fill
                uint32_t ax = 0, ay = 0;
                if (KS == 1) {
                    ax = ((a4[r] >> (8 * sub)) & 0xffu) << 7;
                } else if (KS == 2) {
                    ax = ((a4[r] >> (16 * sub)) & 0xffu) << 7;
                    ay = ((a4[r] >> (16 * sub + 8)) & 0xffu) << 7;
                } else {
                    ax = __builtin_amdgcn_alignbit(a4[r], a4[r], rot_kk0);
                    ay = __builtin_amdgcn_alignbit(ax, ax, rot_p0);
                }
                uint32_t ad[8];
#pragma unroll
                for (int s = 0; s < 8; ++s) {
                    uint32_t aoff;
                    if (KS == 1)
                        aoff = ax;
                    else if (KS == 2)
                        aoff = kk_hi[s] ? ay : ax;
                    else
                        aoff = ((((s & 1) ? ay : ax) >> (8 * (s >> 1))) & 0xffu) << 7;
                    ad[s] = aoff + choff[s];
                }
                if constexpr (NT == 16) {
                    LOOKUP_ROW_NT16(acc[r], ad);
                } else if constexpr (NT == 32) {
                    LOOKUP_ROW_NT32(acc[r], ad);
                } else {
                    LOOKUP_ROW_NT64(acc[r], ad);
                }
            }
            if (fill + 1 == fills)
                break;

            // ---- expanded rows of the next fill ----
            derive_read(wn);   // table-row reads + transposes overlap other wavefronts' lookups
            __syncthreads();   // every wavefront is done reading the expanded rows of this fill
            derive_write();
            __syncthreads();

            // ---- roll the pipeline: consume the prefetched registers, then issue the next loads ----
            if (++sub == SUBS) {
                sub = 0;
#pragma unroll
                for (int r = 0; r < R; ++r)
                    a4[r] = a4n[r];
                advance_cursor();
                if (tap_n < taps)
                    issue_act_loads();
            }
            if (fill + 2 < fills)
                wn = *reinterpret_cast<const u32x2 *>(wq_tile + (size_t)(fill + 2) * 64);
        }

        // ---- epilogue: zero-point correction + dequantize (approx_nn_conv_kernels.cpp:250-253) ----
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!rvalid[r])
                continue;
            const int64_t m = row0 + (int64_t)(r * kWaves + wave) * 64 + lane;
            // patch sum of the raw input in the reference's order (tap-major, channels ascending)
            const float psum = OUT_I32 ? 0.0f : p.psum[m];
            const float t1 = __fmul_rn(p.m2, psum);
#pragma unroll
            for (int set = 0; set < SETS; ++set) {
                const int h = (c0 + set) & (SETS - 1);
                const int col0 = ct * NT + h * 8;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int col = col0 + e;
                    if (col >= g.Co)
                        continue;
                    const int32_t a = acc[r][set * 8 + e];
                    if (OUT_I32) {
                        p.out_i[m * g.Co + col] = a;
                    } else {
                        const float t0 = __fmul_rn((float)a, p.s1xs2);
                        const float t2 = __fadd_rn(t0, t1);
                        const float t3 = __fmul_rn(p.m1, p.fsum[col]);
                        const float t4 = __fadd_rn(t2, t3);
                        p.out_f[m * g.Co + col] = __fsub_rn(t4, p.k_m1xm2);
                    }
                }
            }
        }
    }
}

template <int NT, bool OUT_I32>
static hipError_t launch_one(const DenseParams &p, hipStream_t stream)
{
    auto kernel = lutgemm_expand_kernel<NT, OUT_I32>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
    if (e != hipSuccess)
        return e;
    hipLaunchKernelGGL(kernel, dim3(p.plan.grid), dim3(kBlockThreads), kLdsBytes, stream, p);
    return hipGetLastError();
}

hipError_t launch_dense(const DenseParams &p, bool out_i32, hipStream_t stream)
{
    switch (p.plan.nt) {
    case 16: return out_i32 ? launch_one<16, true>(p, stream) : launch_one<16, false>(p, stream);
    case 32: return out_i32 ? launch_one<32, true>(p, stream) : launch_one<32, false>(p, stream);
    case 64: return out_i32 ? launch_one<64, true>(p, stream) : launch_one<64, false>(p, stream);
    default: return hipErrorInvalidValue;
    }
}

} // namespace axc
