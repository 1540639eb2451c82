// Pieces of a dense LUT-GEMM tile that do not depend on how the table entries reach LDS: which wavefront-rows a
// wavefront owns, the per-pixel geometry it parks in LDS, and the epilogue (zero-point correction, dequantize,
// bias / ReLU, store).  Included by the kernels' translation units only.
#pragma once

#include "axconv_internal.h"

#include <type_traits>

namespace axc {

// Global loads go through raw buffer descriptors: address = SGPR base + SGPR offset + one 32-bit VGPR
// offset, so no load needs a 64-bit VGPR address, and reads past the end return 0 instead of faulting.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
__device__ __forceinline__ rsrc_t make_rsrc(const void *base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint32_t ld_u32(rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0);
}

constexpr int kOldShare = 11; // sixteenths of a tile's wavefront-rows owned by the older four wavefronts
constexpr int kOwnSplitFrom = 29, kOwnSplitTo = 48; // tiles of this many wavefront-rows: tile_rows_of's OWN_SPLIT differs from kOldShare

// The rows of a tile and this wavefront's share of them.  A wavefront-row is 64 consecutive output pixels (one per
// lane); a wavefront owns wavefront-rows wr_base, wr_base + 4, ... below its half's end.  The SIMD issues the older
// of its two wavefronts first, so the first four wavefronts get through their lookups faster: they own
// kOldShare/16 of the tile, and both halves reach the barrier together.
struct TileRows {
    int64_t row0, row_end;  // output pixels [row0, row_end) of the tile
    int64_t wr_end;         // end of the pixels owned by this wavefront's half
    int wr_base;
};
// ROUND_ROBIN: wavefront-row i goes to SIMD i & 3 whichever half owns it (wavefront w sits on SIMD w & 3), so the
// SIMDs' loads differ by one row at most however the rows divide between the halves.
template <int R, bool EVEN_SMALL = false, bool ROUND_ROBIN = false, bool OWN_SPLIT = false>
__device__ __forceinline__ TileRows tile_rows_of(const DenseParams &p, int rt, int wave)
{
    TileRows t;
    t.row0 = (int64_t)rt * p.plan.rows_per_tile;
    t.row_end = (t.row0 + p.plan.rows_per_tile < p.g.M) ? t.row0 + p.plan.rows_per_tile : p.g.M;
    const int wrows = (int)((t.row_end - t.row0 + 63) / 64);
    int wr_old = (wrows * kOldShare + 8) / 16;
    // OWN_SPLIT (the kernel without barriers, whose wavefronts are not held to a common pace fill by fill: a tile
    // takes as long as its longest wavefront).  Measured over tiles of 32-60 wavefront-rows at 72 fills, an older
    // wavefront with o rows takes 57 + 25.5 o microseconds, a younger one with y rows 13 + 45 y: whole rows per older
    // wavefront, as many as make the larger of the two smallest.  From 49 rows on that is the rule above.
    if (OWN_SPLIT && wrows >= kOwnSplitFrom)
        wr_old = wrows <= 36 ? 20 : wrows <= 40 ? 24 : wrows <= kOwnSplitTo ? 28 : 32;
    // EVEN_SMALL: with up to one wavefront-row per wavefront, one each (for a kernel whose phase then lasts as long
    // as the lookups of its slowest wavefront)
    if (EVEN_SMALL && wrows <= kDenseWaves)
        wr_old = wrows < kDenseWaves / 2 ? wrows : kDenseWaves / 2;
    wr_old = wr_old > 4 * R ? 4 * R : wr_old;
    wr_old = wr_old < wrows - 4 * R ? wrows - 4 * R : wr_old;
    const bool old_half = wave < kDenseWaves / 2;
    t.wr_base = old_half ? wave : wr_old + (ROUND_ROBIN ? ((wave - wr_old) & 3) : wave - kDenseWaves / 2);
    t.wr_end = t.row0 + (int64_t)(old_half ? wr_old : wrows) * 64;
    return t;
}

// Per-pixel geometry of this lane's R pixels, parked in LDS in slots private to the thread (park[slot *
// kDenseThreads]) and read back only when the tap changes: slot 2r = dword index in xq of tap (0, 0), channel
// quad 0 in address units (may point outside the image), slot 2r+1 = input coordinates of tap (0, 0) as (ih0 << 16) | (iw0 & 0xffff),
// 0x80000000 for a pixel that does not exist.  Returns the number of this lane's pixels whose wavefront-row exists
// (a prefix of the R; the same in every lane of the wavefront).
// STRIDE: dwords between a thread's slots (kDenseThreads: slot-major over the workgroup; 64: every wavefront owns a
// contiguous piece).  skip_row: a pixel slot that is not written (its place in LDS belongs to something else).
template <int R, int STRIDE = kDenseThreads>
__device__ __forceinline__ uint32_t park_geometry(const DenseParams &p, const TileRows &t, int lane, uint32_t *park,
                                                  const int skip_row = -1)
{
    const ConvGeom &g = p.g;
    const int rowstep = p.row_step;
    uint32_t nr = 0;
    // (n, oh, ow) of this lane's first pixel by division; its further pixels lie a fixed number of output
    // pixels apart (four wavefront-rows), so they follow by adding that step's (n, oh, ow) with carries
    int n = 0, oh = 0, ow = 0;
    {
        const int64_t m0 = t.row0 + (int64_t)t.wr_base * 64 + lane;
        const int64_t mm = m0 < g.M ? m0 : 0;
        int rem;
        if (g.M <= 0x7fffffff) { // the usual case: 32-bit divisions (a 64-bit one costs several times more)
            const uint32_t ohow = (uint32_t)(g.OH * g.OW);
            n = (int)((uint32_t)mm / ohow);
            rem = (int)((uint32_t)mm - (uint32_t)n * ohow);
        } else {
            n = (int)(mm / ((int64_t)g.OH * g.OW));
            rem = (int)(mm - (int64_t)n * g.OH * g.OW);
        }
        oh = (int)((uint32_t)rem / (uint32_t)g.OW);
        ow = rem - oh * g.OW;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t wrow = t.row0 + (int64_t)(t.wr_base + r * (kDenseWaves / 2)) * 64;
        nr += (wrow < t.row_end && wrow < t.wr_end) ? 1u : 0u;
        const bool valid = wrow + lane < t.row_end && wrow < t.wr_end;
        // flat layout: the horizontal padding is part of the row, so the column of tap (0, 0) is ow * sw pixels in
        // and never outside (stored as column 0)
        const int ih0 = oh * g.sh - g.ph, iw0 = p.flat_col_bytes ? 0 : ow * g.sw - g.pw;
        const int col = p.flat_col_bytes ? ow * p.flat_col_bytes : iw0;
        if (r != skip_row) {
            park[(2 * r) * STRIDE] = valid ? (uint32_t)((n * g.H + ih0) * rowstep + col) : 0u;
            park[(2 * r + 1) * STRIDE] = valid ? (uint32_t)((ih0 << 16) | (iw0 & 0xffff)) : 0x80000000u;
        }
        // the next pixel of this lane: p.step_* = (n, oh, ow) of 64 * kDenseWaves / 2 output pixels
        ow += p.step_ow;
        const int c1 = ow >= g.OW ? 1 : 0;
        ow -= c1 ? g.OW : 0;
        oh += p.step_oh + c1;
        const int c2 = oh >= g.OH ? 1 : 0;
        oh -= c2 ? g.OH : 0;
        n += p.step_n + c2;
    }
    return nr;
}

// byte offset in xq of quad 0 of tap (kh, kw) for each of the lane's pixels; the zero-point row outside the image.
// live (the same for the whole wavefront): only the first `live` pixels are recomputed, the others keep what they hold.
template <int R, int STRIDE = kDenseThreads>
__device__ __forceinline__ void tap_offsets(const DenseParams &p, const uint32_t *park, int kh, int kw, uint32_t zp_row,
                                            uint32_t (&idx_tap)[R], uint32_t live = R)
{
    const ConvGeom &g = p.g;
    const int dh = kh * g.dh, dw = kw * g.dw;
    const int tap_off = dh * p.row_step + dw;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if ((uint32_t)r >= live)
            break;
        const int32_t pb = (int32_t)park[(2 * r) * STRIDE];
        const int32_t hw = (int32_t)park[(2 * r + 1) * STRIDE];
        const int ih = (hw >> 16) + dh;
        const int iw = (int)(int16_t)(hw & 0xffff) + dw;
        const bool inb = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
        idx_tap[r] = inb ? (uint32_t)((pb + tap_off) * p.addr_unit) : zp_row;
    }
}

// The phases add whole dwords (two 16-bit table entries) into the accumulator of the even column and the high entry
// alone into that of the odd column: even = sum(lo) + 65536 * sum(hi) modulo 2^32.  Subtracting a multiple of
// 65536 changes the high half only: one 16-bit subtract (high half of the even accumulator minus low half of the
// odd one, written back into the high half, low half kept).
template <int R, int NT>
__device__ __forceinline__ void fix_even_columns(int32_t (&acc)[R][NT])
{
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
        for (int j = 0; j < NT; j += 2)
            __asm__("v_sub_u16_sdwa %0, %0, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1 src1_sel:WORD_0"
                    : "+v"(acc[r][j])
                    : "v"(acc[r][j + 1]));
}

// Epilogue of one tile: zero-point correction + dequantize (approx_nn_conv_kernels.cpp:250-253), then what the Keras
// layer does behind the op (bias_add, activation), then the store.  acc[r][set * 8 + e] is column e of column group
// (c0 + set) & (SETS - 1), c0 = lane & 7, of the lane's pixel r.
//
// A lane holds NT consecutive columns of its pixel: stored as they are, one instruction would touch 64 different
// 64-byte pieces of memory.  With NT <= 32 and Co % 4 == 0 the wavefront therefore turns each of its wavefront-rows
// through a private piece of LDS (turn + wave * 64 * (NT * 4 + 16) bytes; the caller guarantees that nothing else
// uses it) so that NT/4 neighbouring lanes write one pixel's NT columns: 16 or 8 contiguous runs per store.
//
// HALF_TURN: `turn` is the wavefront's own piece already, and only 32 * (NT * 4 + 16) bytes of it: a wavefront-row
// goes through it as two halves of 32 pixels.
template <int NT, bool OUT_I32, bool HALF_TURN = false>
__device__ __forceinline__ void store_tile(const DenseParams &p, int32_t (&acc)[2 * (64 / NT)][NT], const TileRows &t,
                                           const int ct, const int ksi, const uint32_t nr_s, const int lane,
                                           const int wave, unsigned char *const turn)
{
    constexpr int R = 2 * (64 / NT), SETS = NT / 8;
    const ConvGeom &g = p.g;
    const int c0 = lane & 7;
    const float e_s1xs2 = p.lq_dev ? p.lq_dev->s1xs2 : p.s1xs2, e_m1 = p.lq_dev ? p.lq_dev->m1 : p.m1;
    const float e_m2 = p.lq_dev ? p.lq_dev->m2 : p.m2, e_km = p.lq_dev ? p.lq_dev->k_m1xm2 : p.k_m1xm2;
    auto finish = [&](float v, int col) __attribute__((always_inline)) {
        if (p.bias)
            v = __fadd_rn(v, p.bias[col]);
        return p.relu ? fmaxf(v, 0.0f) : v;
    };
    // a lane's pixel r exists if its wavefront-row does (a prefix of nr_s rows) and it lies inside the tile
    auto rvalid = [&](const int r) __attribute__((always_inline)) {
        return r < (int)nr_s && t.row0 + (int64_t)(t.wr_base + r * (kDenseWaves / 2)) * 64 + lane < t.row_end;
    };
    constexpr bool kTransposed = NT <= 32;
    // Every global load of the epilogue is issued here, ahead of the first store: loads and stores complete in
    // issue order, so a load behind a store would wait until that store has reached memory.
    float ps[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int64_t m = t.row0 + (int64_t)(t.wr_base + r * (kDenseWaves / 2)) * 64 + lane;
        ps[r] = (!OUT_I32 && rvalid(r)) ? p.psum[m] : 0.0f;
    }
    if (kTransposed && (g.Co & 3) == 0) {
        constexpr int Q = NT / 4;                 // 16-byte quads (lanes) per pixel
        constexpr int PITCH = NT * 4 + 16;        // bytes per pixel in LDS: the +16 spreads pixels over the banks
        unsigned char *const wl = HALF_TURN ? turn : turn + (size_t)wave * 64 * PITCH;
        typedef uint32_t u32x4s __attribute__((ext_vector_type(4)));
        // Behind the transposition a lane stores the same four columns of every pixel it handles: the terms
        // that depend on the column (filter sum, bias) are applied there, from four registers each.
        const int quad = lane % Q, colq = ct * NT + quad * 4;
        float t3q[4], biasq[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = colq + j < g.Co ? colq + j : g.Co - 1;
            t3q[j] = OUT_I32 ? 0.0f : __fmul_rn(e_m1, p.fsum[c]);
            biasq[j] = (!OUT_I32 && p.bias) ? p.bias[c] : 0.0f;
        }
        // bias and ReLU are wave-uniform run-time switches: one copy of the store loop per combination, chosen
        // once, instead of two selects per output element
        auto store_rows = [&](auto has_bias_t, auto has_relu_t) __attribute__((always_inline)) {
            constexpr bool kBias = decltype(has_bias_t)::value, kRelu = decltype(has_relu_t)::value;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r >= (int)nr_s)
                    break;
                const int64_t m0 = t.row0 + (int64_t)(t.wr_base + r * (kDenseWaves / 2)) * 64;
                const int nvalid = (int)(t.row_end - m0 < 64 ? t.row_end - m0 : 64);
                const float t1 = __fmul_rn(e_m2, ps[r]);
                uint32_t *const out = OUT_I32 ? reinterpret_cast<uint32_t *>(p.out_i) + (int64_t)ksi * g.M * g.Co
                                              : reinterpret_cast<uint32_t *>(p.out_f);
                constexpr int PASSES = HALF_TURN ? 2 : 1, PIX = 64 / PASSES;   // pixels per pass through LDS
#pragma unroll
                for (int pass = 0; pass < PASSES; ++pass) {
                    if (!HALF_TURN || (lane >> 5) == pass) {
#pragma unroll
                        for (int set = 0; set < SETS; ++set) {
                            const int h = (c0 + set) & (SETS - 1);
                            uint32_t w[8];
#pragma unroll
                            for (int e = 0; e < 8; ++e) {
                                if (OUT_I32)
                                    w[e] = (uint32_t)acc[r][set * 8 + e];
                                else
                                    w[e] = __float_as_uint(__fadd_rn(__fmul_rn((float)acc[r][set * 8 + e], e_s1xs2), t1));
                            }
                            u32x4s lo = {w[0], w[1], w[2], w[3]}, hi = {w[4], w[5], w[6], w[7]};
                            *reinterpret_cast<u32x4s *>(wl + (lane & (PIX - 1)) * PITCH + h * 32) = lo;
                            *reinterpret_cast<u32x4s *>(wl + (lane & (PIX - 1)) * PITCH + h * 32 + 16) = hi;
                        }
                    }
#pragma unroll
                    for (int i = 0; i < Q / PASSES; ++i) {
                        const int pl = i * (64 / Q) + lane / Q;      // pixel within the pass
                        const int pix = pass * PIX + pl;
                        u32x4s d = *reinterpret_cast<const u32x4s *>(wl + pl * PITCH + quad * 16);
                        if (!OUT_I32) {
#pragma unroll
                            for (int j = 0; j < 4; ++j) {
                                float v = __fsub_rn(__fadd_rn(__uint_as_float(d[j]), t3q[j]), e_km);
                                if (kBias)
                                    v = __fadd_rn(v, biasq[j]);
                                d[j] = __float_as_uint(kRelu ? fmaxf(v, 0.0f) : v);
                            }
                        }
                        if (pix < nvalid && colq < g.Co) {
                            // the float output is not read again by this op: streamed past the caches, which keeps
                            // them for the activations; split-K partial sums are read back at once and stay cached
                            if (OUT_I32)
                                *reinterpret_cast<u32x4s *>(out + (m0 + pix) * g.Co + colq) = d;
                            else
                                __builtin_nontemporal_store(d, reinterpret_cast<u32x4s *>(out + (m0 + pix) * g.Co + colq));
                        }
                    }
                }
            }
        };
        using yes = std::true_type;
        using no = std::false_type;
        if (OUT_I32 || (!p.bias && !p.relu))
            store_rows(no(), no());
        else if (p.bias && p.relu)
            store_rows(yes(), yes());
        else if (p.bias)
            store_rows(yes(), no());
        else
            store_rows(no(), yes());
        return;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (!rvalid(r))
            continue;
        const int64_t m = t.row0 + (int64_t)(t.wr_base + r * (kDenseWaves / 2)) * 64 + lane;
        // patch sum of the raw input in the reference's order (tap-major, channels ascending)
        const float t1 = __fmul_rn(e_m2, ps[r]);
#pragma unroll
        for (int set = 0; set < SETS; ++set) {
            const int h = (c0 + set) & (SETS - 1);
            const int col0 = ct * NT + h * 8;
            if (col0 >= g.Co)
                continue;
            const int64_t o = m * g.Co + col0;
            const bool vec = (g.Co & 3) == 0 && col0 + 8 <= g.Co; // 32 contiguous, 16-byte aligned bytes
            if (OUT_I32) {
                if (vec) {
                    typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
                    i32x4 lo = {acc[r][set * 8 + 0], acc[r][set * 8 + 1], acc[r][set * 8 + 2], acc[r][set * 8 + 3]};
                    i32x4 hi = {acc[r][set * 8 + 4], acc[r][set * 8 + 5], acc[r][set * 8 + 6], acc[r][set * 8 + 7]};
                    *reinterpret_cast<i32x4 *>(p.out_i + (int64_t)ksi * g.M * g.Co + o) = lo;
                    *reinterpret_cast<i32x4 *>(p.out_i + (int64_t)ksi * g.M * g.Co + o + 4) = hi;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (col0 + e < g.Co)
                            p.out_i[(int64_t)ksi * g.M * g.Co + o + e] = acc[r][set * 8 + e];
                }
            } else {
                float v[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int col = col0 + e < g.Co ? col0 + e : g.Co - 1;
                    const float t0 = __fmul_rn((float)acc[r][set * 8 + e], e_s1xs2);
                    const float t2 = __fadd_rn(t0, t1);
                    const float t3 = __fmul_rn(e_m1, p.fsum[col]);
                    const float t4 = __fadd_rn(t2, t3);
                    v[e] = finish(__fsub_rn(t4, e_km), col);
                }
                if (vec) {
                    *reinterpret_cast<float4 *>(p.out_f + o) = make_float4(v[0], v[1], v[2], v[3]);
                    *reinterpret_cast<float4 *>(p.out_f + o + 4) = make_float4(v[4], v[5], v[6], v[7]);
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (col0 + e < g.Co)
                            p.out_f[o + e] = v[e];
                }
            }
        }
    }
}

} // namespace axc
