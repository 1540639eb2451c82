// Dense LUT-GEMM for gfx950: implicit-GEMM gather + table lookups out of LDS + fused epilogue.
//
// A "fill" takes 64 filter entries (KS consecutive input channels x NT output columns, KS * NT = 64) and
// builds their expanded rows in LDS: E[phys_row(a)][slot] = T[a][code(slot)], 128 bytes per activation
// code a, 32 KiB per fill.  Every lane then looks up, for each of its R output pixels, the expanded row of
// its activation code with ds_read_b128: eight table entries per LDS access instead of one, and the
// 16-byte chunks the lanes of a wavefront touch in one instruction are rotated by lane so they fall into
// different banks whatever the activation codes are.  Sums are exact int32.
//
// Everything is double-buffered in LDS so that one barrier per fill is all the synchronization there is:
//   expanded rows   2 x 32 KiB  wavefronts look up fill p out of one buffer while they transpose the
//                               table rows of fill p + 1 into the other
//   staged rows     2 x 32 KiB  the 64 table rows (512 contiguous bytes per filter code) of fill p + 1,
//                               read bank-conflict free by the transposing lanes, while the rows of fill
//                               p + 2 land in the other buffer
// The table itself (128 KiB, resident in L2) is read with fully coalesced 16-byte loads that land in the staged
// rows directly (buffer loads into LDS: no register, no LDS write instruction), half a wavefront per row, two
// fills ahead of the lookups; the filter codes that select the rows three fills ahead.
//
// One workgroup of 8 wavefronts per CU, 256 VGPRs per wavefront: 128 int32 accumulators per lane
// (R = 8 pixels x 16 columns, 4 x 32 or 2 x 64), eight 16-byte lookups in flight per wavefront.
//
// Restates, as one fused kernel, what the reference does in ApproxConvIm2ColKernel +
// ApproxConvGEMMKernel (tf2/src/approx_nn_conv_kernels.cpp:215-296) per chunk.
#include "axconv_internal.h"
#include "lookup_asm.inc"

#include <type_traits>

namespace axc {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

extern __shared__ __align__(16) unsigned char lds[];

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
__device__ __forceinline__ u32x2 ld_u32x2(rsrc_t r, uint32_t voff, uint32_t soff)
{
    return __builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, (int)soff, 0);
}

constexpr int kOldShare = 11; // sixteenths of a tile's wavefront-rows owned by the older four wavefronts

template <int NT>
struct DenseCfg {
    static constexpr int R = 2 * (64 / NT);   // output pixels per lane
    static constexpr int KS = 64 / NT;        // input channels per fill
    static constexpr int SETS = NT / 8;       // 8-column groups per pixel
    static constexpr int SUBS = 4 / KS;       // fills per channel quad
};

// Lane constants of the phase body.
struct PhaseConsts {
    uint32_t sel[8];   // v_perm_b32 selectors that build the lookup address of step s
    uint32_t cha, chb; // packed chunk offsets of steps 0-3 / 4-7
    uint32_t stm;      // LDS address of this wavefront's two staged rows (1 KiB) of buffer 0, load 0 (wave-uniform)
    uint32_t sto;      // byte offset of this thread's 16 bytes inside a 512-byte table row
    uint32_t cvo;      // byte offset of filter code (thread / 32) inside the 64 codes of a fill
    uint32_t rd[2];    // LDS address (buffer 0) of the staged-row bytes derive item i reads
    uint32_t wr[2];    // LDS address (buffer 0) of the expanded-row bytes derive item i writes
};

// One phase (see gen_lookup_asm.py): lookups of fill p out of expanded-row buffer BUF, interleaved with loading
// the rows of fill p+2 into the staged rows, codes / activations of later fills, and expanding fill p+1.
template <int NT, int BUF>
__device__ __forceinline__ void phase_body(int32_t (&acc)[DenseCfg<NT>::R][NT], const uint32_t (&acur)[DenseCfg<NT>::R],
                                           uint32_t (&anext)[DenseCfg<NT>::R], const uint32_t (&tapoff)[DenseCfg<NT>::R],
                                           uint32_t (&codes)[4], const PhaseConsts &k,
                                           const uint32_t nr, const uint32_t shift, const rsrc_t tab, const rsrc_t wq,
                                           const rsrc_t xq, const uint32_t cso, const uint32_t qoff)
{
    const uint32_t stm = __builtin_amdgcn_readfirstlane(k.stm);
    if constexpr (NT == 16) {
        if constexpr (BUF == 0) PHASE_NT16_B0(acc, acur, anext, tapoff, codes, k.sel, k.cha, k.chb, nr, shift, stm, k.sto, k.cvo, k.rd, k.wr, tab, wq, xq, cso, qoff);
        else PHASE_NT16_B1(acc, acur, anext, tapoff, codes, k.sel, k.cha, k.chb, nr, shift, stm, k.sto, k.cvo, k.rd, k.wr, tab, wq, xq, cso, qoff);
    } else if constexpr (NT == 32) {
        if constexpr (BUF == 0) PHASE_NT32_B0(acc, acur, anext, tapoff, codes, k.sel, k.cha, k.chb, nr, shift, stm, k.sto, k.cvo, k.rd, k.wr, tab, wq, xq, cso, qoff);
        else PHASE_NT32_B1(acc, acur, anext, tapoff, codes, k.sel, k.cha, k.chb, nr, shift, stm, k.sto, k.cvo, k.rd, k.wr, tab, wq, xq, cso, qoff);
    } else {
        if constexpr (BUF == 0) PHASE_NT64_B0(acc, acur, anext, tapoff, codes, k.sel, k.cha, k.chb, nr, shift, stm, k.sto, k.cvo, k.rd, k.wr, tab, wq, xq, cso, qoff);
        else PHASE_NT64_B1(acc, acur, anext, tapoff, codes, k.sel, k.cha, k.chb, nr, shift, stm, k.sto, k.cvo, k.rd, k.wr, tab, wq, xq, cso, qoff);
    }
}

template <int NT, bool OUT_I32>
__global__ void __launch_bounds__(kDenseThreads) lutgemm_expand_kernel(const DenseParams p)
{
    constexpr int R = DenseCfg<NT>::R, SETS = DenseCfg<NT>::SETS, SUBS = DenseCfg<NT>::SUBS;
    constexpr int LOG_SETS = (SETS == 8) ? 3 : (SETS == 4) ? 2 : 1;
    constexpr int ITEMS = 16 / kDenseWaves; // derive items (4 activation codes x 4 slots) per thread per fill

    const ConvGeom &g = p.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: row activity branches on SGPRs

    // ---- lane constants ----
    const int c0 = lane & 7;
    // Step s of a pixel reads chunk c_s = (c0 + s) & 7 of the expanded row of one activation code: the lanes
    // of a wavefront touch eight different chunks per instruction whatever the codes are.  The chunk holds
    // slots 8*c_s .. 8*c_s+7, i.e. input channel kk_s = c_s >> LOG_SETS of the fill, column group
    // c_s & (SETS - 1).  The address (row << 8 | buffer << 7 | c_s << 4) is one v_perm_b32 of the
    // activation dword and the packed chunk offsets: byte 1 <- activation byte kk_s, byte 0 <- offset byte.
    uint32_t sel[8];
    uint32_t cha = 0;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const uint32_t c = (uint32_t)(c0 + s) & 7u;
        sel[s] = 0x0c0c0000u | ((4u + (c >> LOG_SETS)) << 8) | (uint32_t)(s & 3);
        if (s < 4)
            cha |= (c << 4) << (8 * s);
    }
    const uint32_t chb = cha ^ 0x40404040u; // (c0 + s + 4) & 7 == ((c0 + s) & 7) ^ 4
    // derive: item i of this lane transposes activation codes 4*lane .. 4*lane+3 of the staged table rows of
    // slots 4*jq_i .. 4*jq_i+3; the row permutation phys_row() and the rotation of jq by wavefront make
    // both the staged-row reads and the expanded-row writes bank-conflict free
    uint32_t jq8[ITEMS];
#pragma unroll
    for (int i = 0; i < ITEMS; ++i)
        jq8[i] = (uint32_t)((lane + wave + i * kDenseWaves) & 15) * 8u; // byte offset of 4 slots in a row
    const uint32_t rd_lane = (uint32_t)lane * 8u;    // this lane's 8 bytes inside a staged 512-byte row
    const uint32_t wr_row = (uint32_t)lane * 256u;   // expanded rows of the two buffers interleave: 256 bytes apart
    // staging: load j of this thread fetches 16 bytes of the table row of slot 16*j + tid/32
    const uint32_t st_slot = (uint32_t)tid >> 5;
    const uint32_t st_off = ((uint32_t)tid & 31u) * 16u;
    // per-thread geometry is parked in LDS behind the four buffers: [slot][thread]
    uint32_t *const park = reinterpret_cast<uint32_t *>(lds + kDenseLdsBytes) + tid;
    unsigned char *const stage = lds + 2 * kExpandBytes;

    const int taps = g.KH * g.KW;
    // a tile = (row tile, column tile, K split); the K splits of a column tile count as further column tiles
    const int nct_v = p.plan.n_col_tiles * p.plan.k_splits;
    const int ntiles = p.plan.n_row_tiles * nct_v;
    const int fills_all = p.plan.fills;
    const int rowstep = g.C4 * g.W; // dwords between input rows in xq
    // xq ends with one extra input row filled with the zero-point code: taps outside the image read it
    const uint32_t zp_row = p.xq_bytes;
    const rsrc_t xq_rsrc = make_rsrc(p.xq, p.xq_bytes + (uint32_t)rowstep * 4u);
    const rsrc_t wq_rsrc = make_rsrc(p.wq, p.wq_bytes);
    const rsrc_t tab_rsrc = make_rsrc(p.tableT, (uint32_t)kTableAllocBytes);
    (void)taps;

    // Tiles in the order (row tile, column tile incl. K split), column tile fastest, dealt round-robin: at any time
    // the workgroups work on neighbouring tiles, i.e. on the column tiles of a few row tiles.  Workgroups are handed
    // to the 8 XCDs round-robin, and each XCD has its own L2: the deal goes by a workgroup index in which neighbours
    // sit on one XCD, so the column tiles of a row tile (same activations; outputs in the same memory lines, written
    // at about the same time) meet in one L2.
    const int G = (int)gridDim.x;
    const int wg = (G & 7) == 0 ? ((int)blockIdx.x & 7) * (G >> 3) + ((int)blockIdx.x >> 3) : (int)blockIdx.x;
    if (p.stagger_sleeps && ((wg / nct_v) & 1)) // every second group of workgroups (one row tile's column tiles) starts late
        for (int i = 0; i < p.stagger_sleeps; ++i)
            __builtin_amdgcn_s_sleep(127);
    int prev_rt = -1;
    bool rvalid[DenseCfg<NT>::R];    // this lane's pixel exists
    uint32_t nr = 0;                 // pixels of this lane whose wavefront row exists (a prefix; wave-uniform)
    for (int tile = wg; tile < ntiles; tile += G) {
        const int rt = tile / nct_v;
        int ct = tile - rt * nct_v;
        const int ksi = ct / p.plan.n_col_tiles;           // K split of this tile
        ct -= ksi * p.plan.n_col_tiles;
        const int f0 = ksi * p.plan.fills_per_split;        // its fills: [f0, f0 + fills)
        const int fills = fills_all - f0 < p.plan.fills_per_split ? fills_all - f0 : p.plan.fills_per_split;
        const int64_t row0 = (int64_t)rt * p.plan.rows_per_tile;
        const int64_t row_end = (row0 + p.plan.rows_per_tile < g.M) ? row0 + p.plan.rows_per_tile : g.M;

        // ---- which wavefront-rows (64 consecutive output pixels) of the tile this wavefront owns ----
        // The SIMD issues the older of its two wavefronts first, so the first four wavefronts get through
        // their lookups faster; they own kOldShare/16 of the tile, and both halves reach the barrier together.
        const int wrows = (int)((row_end - row0 + 63) / 64);
        int wr_old = (wrows * kOldShare + 8) / 16;
        wr_old = wr_old > 4 * R ? 4 * R : wr_old;
        wr_old = wr_old < wrows - 4 * R ? wrows - 4 * R : wr_old;
        const bool old_half = wave < kDenseWaves / 2;
        const int wr_base = old_half ? wave : wr_old + wave - kDenseWaves / 2; // then every fourth wavefront-row
        const int64_t wr_end = row0 + (int64_t)(old_half ? wr_old : wrows) * 64;

        // ---- per-pixel geometry (parked in LDS, in slots private to the thread; only read back when the tap
        // changes).  It depends on the row tile alone: kept from the previous tile when that had the same one.
        if (rt != prev_rt) {
            prev_rt = rt;
            nr = 0;
            // (n, oh, ow) of this lane's first pixel by division; its further pixels lie a fixed number of output
            // pixels apart (four wavefront-rows), so they follow by adding that step's (n, oh, ow) with carries
            int n = 0, oh = 0, ow = 0;
            {
                const int64_t m0 = row0 + (int64_t)wr_base * 64 + lane;
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
                const int64_t wrow = row0 + (int64_t)(wr_base + r * (kDenseWaves / 2)) * 64;
                nr += (wrow < row_end && wrow < wr_end) ? 1u : 0u;
                const int64_t m = wrow + lane;
                rvalid[r] = m < row_end && wrow < wr_end;
                const int ih0 = oh * g.sh - g.ph, iw0 = ow * g.sw - g.pw;
                // dword index in xq of tap (0, 0), channel quad 0 (may point outside the image)
                park[(2 * r) * kDenseThreads] = rvalid[r] ? (uint32_t)((n * g.H + ih0) * rowstep + iw0) : 0u;
                // input coordinates of tap (0, 0); ih0 = -32768 marks a pixel that does not exist
                park[(2 * r + 1) * kDenseThreads] = rvalid[r] ? (uint32_t)((ih0 << 16) | (iw0 & 0xffff)) : 0x80000000u;
                // the next pixel of this lane: p.step_* = (n, oh, ow) of 64 * kDenseWaves / 2 output pixels
                ow += p.step_ow;
                const int c1 = ow >= g.OW ? 1 : 0;
                ow -= c1 ? g.OW : 0;
                oh += p.step_oh + c1;
                const int c2 = oh >= g.OH ? 1 : 0;
                oh -= c2 ? g.OH : 0;
                n += p.step_n + c2;
            }
        }

        const uint32_t wq_tile = ((uint32_t)ct * (uint32_t)fills_all + (uint32_t)f0) * 128u; // this tile's first codes
        const int fills_left = fills_all - f0;              // codes may be prefetched past the split, not past the end

        // ---- activation cursor: position (tap, quad) of the fill whose activations are fetched next ----
        int cur_fill = 0, cur_sub = f0 % SUBS;
        int cur_q = (f0 / SUBS) % g.C4, cur_kh = (f0 / SUBS / g.C4) / g.KW, cur_kw = (f0 / SUBS / g.C4) % g.KW;
        uint32_t idx_tap[R];   // byte offset in xq of quad 0 of the current tap (the zero-point row outside)
        auto tap_setup = [&]() {
            const int dh = cur_kh * g.dh, dw = cur_kw * g.dw;
            const int tap_off = dh * rowstep + dw;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int32_t pb = (int32_t)park[(2 * r) * kDenseThreads];
                const int32_t hw = (int32_t)park[(2 * r + 1) * kDenseThreads];
                const int ih = (hw >> 16) + dh;
                const int iw = (int)(int16_t)(hw & 0xffff) + dw;
                const bool inb = (unsigned)ih < (unsigned)g.H && (unsigned)iw < (unsigned)g.W;
                idx_tap[r] = inb ? (uint32_t)((pb + tap_off) * 4) : zp_row;
            }
        };
        auto load_acts = [&](uint32_t (&dst)[R]) {
            const uint32_t qoff = (uint32_t)(cur_q * g.W * 4); // scalar: channel quad inside the pixel row
#pragma unroll
            for (int r = 0; r < R; ++r)
                dst[r] = ld_u32(xq_rsrc, idx_tap[r], qoff);
        };
        auto advance_cursor = [&]() { // to the next fill
            ++cur_fill;
            if (++cur_sub == SUBS) {
                cur_sub = 0;
                if (++cur_q == g.C4) {
                    cur_q = 0;
                    if (++cur_kw == g.KW) { cur_kw = 0; ++cur_kh; }
                    if (cur_fill < fills_left)
                        tap_setup();
                }
            }
        };

        // ---- table rows of one fill: global -> registers -> staged rows -> expanded rows ----
        auto load_codes = [&](int fill, uint32_t (&codes)[4]) {
            const uint32_t f = (uint32_t)(fill < fills_left ? fill : fills_left - 1);
#pragma unroll
            for (int j = 0; j < 4; ++j)
                codes[j] = __builtin_amdgcn_raw_buffer_load_b16(wq_rsrc, (int)((st_slot + 16u * j) * 2u),
                                                                (int)(wq_tile + f * 128u), 0);
        };
        // table rows of one fill -> staged rows [buf], straight from memory into LDS: the wavefront's 64 lanes
        // fill 1 KiB (two rows) per load, lane l the 16 bytes at l * 16
        auto load_rows_to_stage = [&](const uint32_t (&codes)[4], const uint32_t buf) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(
                    tab_rsrc,
                    (__attribute__((address_space(3))) void *)(stage + buf * kExpandBytes + 16u * j * 512u + (uint32_t)wave * 1024u),
                    16, (int)((codes[j] & 0xffffu) * 512u + st_off), 0, 0, 0);
        };
        auto derive = [&](const uint32_t buf) { // staged rows [buf] -> expanded rows [buf]
#pragma unroll
            for (int i = 0; i < ITEMS; ++i) {
                u32x2 v[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) // slot 4*jq + k = byte offset jq8/2 + k in units of rows
                    v[k] = *reinterpret_cast<const u32x2 *>(stage + buf * kExpandBytes + (jq8[i] / 2u + k) * 512u + rd_lane);
                u32x2 o[4];
                o[0].x = __builtin_amdgcn_perm(v[1].x, v[0].x, 0x05040100u);
                o[0].y = __builtin_amdgcn_perm(v[3].x, v[2].x, 0x05040100u);
                o[1].x = __builtin_amdgcn_perm(v[1].x, v[0].x, 0x07060302u);
                o[1].y = __builtin_amdgcn_perm(v[3].x, v[2].x, 0x07060302u);
                o[2].x = __builtin_amdgcn_perm(v[1].y, v[0].y, 0x05040100u);
                o[2].y = __builtin_amdgcn_perm(v[3].y, v[2].y, 0x05040100u);
                o[3].x = __builtin_amdgcn_perm(v[1].y, v[0].y, 0x07060302u);
                o[3].y = __builtin_amdgcn_perm(v[3].y, v[2].y, 0x07060302u);
#pragma unroll
                for (int k = 0; k < 4; ++k)
                    *reinterpret_cast<u32x2 *>(lds + buf * 128u + wr_row + jq8[i] + (uint32_t)k * (64u * 256u)) = o[k];
            }
        };

        // ---- prologue ----
        // state entering phase p: expanded rows of fill p in D[p & 1]; staged rows of fill p+1 in S[(p+1) & 1];
        // codes = filter codes of fill p+2 (in flight); acts[p & 1] = activations of fill p
        uint32_t actA[R], actB[R];
        uint32_t codes[4];
        tap_setup();
        load_acts(actA);
        {
            // two rounds of loads, each in flight together: the filter codes of fills 0-2, then the table rows
            // of fills 0 and 1, which go straight into the two staged-row buffers
            uint32_t codes0[4], codes1[4];
            load_codes(0, codes0);
            load_codes(1, codes1);
            load_codes(2, codes);
            __syncthreads();          // the previous tile's last phase and epilogue are done with every buffer
            load_rows_to_stage(codes0, 0);
            load_rows_to_stage(codes1, 1);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        __syncthreads();
        derive(0);
        __syncthreads();

        int32_t acc[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                acc[r][j] = 0;

        // One phase per fill, one barrier per phase.
        PhaseConsts k;
#pragma unroll
        for (int i = 0; i < 8; ++i)
            k.sel[i] = sel[i];
        k.cha = cha;
        k.chb = chb;
        k.stm = 2u * kExpandBytes + (uint32_t)wave * 1024u;
        k.sto = st_off;
        k.cvo = st_slot * 2u;
#pragma unroll
        for (int i = 0; i < ITEMS; ++i) {
            k.rd[i] = 2u * kExpandBytes + (jq8[i] / 2u) * 512u + rd_lane;
            k.wr[i] = wr_row + jq8[i];
        }
        const uint32_t nr_s = __builtin_amdgcn_readfirstlane(nr);
        // Entering phase p the activation cursor stands on fill p+1 and shift_cur belongs to fill p; the cursor
        // is moved on behind the phase body, where most wavefronts would otherwise only wait for the barrier.
        uint32_t shift_cur = (uint32_t)cur_sub * (32u / SUBS);
        if (fills > 1)
            advance_cursor();
        auto phase = [&](const int pcur, uint32_t (&act_cur)[R], uint32_t (&act_next)[R], auto buf_tag) {
            constexpr int BUF = decltype(buf_tag)::value;
            const int fcodes = pcur + 3 < fills_left ? pcur + 3 : fills_left - 1;
            const uint32_t cso = wq_tile + (uint32_t)fcodes * 128u;
            const uint32_t qoff = (uint32_t)(cur_q * g.W * 4);
            phase_body<NT, BUF>(acc, act_cur, act_next, idx_tap, codes, k, nr_s,
                                __builtin_amdgcn_readfirstlane(shift_cur), tab_rsrc, wq_rsrc, xq_rsrc,
                                __builtin_amdgcn_readfirstlane(cso), __builtin_amdgcn_readfirstlane(qoff));
            shift_cur = (uint32_t)cur_sub * (32u / SUBS); // bits to rotate the channels of fill pcur+1 down
            if (pcur + 2 < fills)
                advance_cursor();             // -> fill pcur+2 (re-reads the parked geometry on a new tap)
            __syncthreads();
        };
        for (int pcur = 0; pcur < fills; pcur += 2) {
            phase(pcur, actA, actB, std::integral_constant<int, 0>());
            if (pcur + 1 < fills)
                phase(pcur + 1, actB, actA, std::integral_constant<int, 1>());
        }

        // The phases add whole dwords (two 16-bit table entries) into the accumulator of the even column and the
        // high entry alone into that of the odd column: even = sum(lo) + 65536 * sum(hi) modulo 2^32.
        // Subtracting a multiple of 65536 changes the high half only: one 16-bit subtract (high half of the even
        // accumulator minus low half of the odd one, written back into the high half, low half kept).
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < NT; j += 2)
                __asm__("v_sub_u16_sdwa %0, %0, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_1 src1_sel:WORD_0"
                        : "+v"(acc[r][j])
                        : "v"(acc[r][j + 1]));

        // ---- epilogue: zero-point correction + dequantize (approx_nn_conv_kernels.cpp:250-253) ----
        // A lane holds NT consecutive columns of its pixel: stored as they are, one instruction would touch 64
        // different 64-byte pieces of memory.  The wavefront therefore turns each of its wavefront-rows
        // through a private piece of LDS (every buffer is free after the last phase) so that NT/4 neighbouring
        // lanes write one pixel's NT columns: 16 or 8 contiguous runs per store instruction.
        const float e_s1xs2 = p.lq_dev ? p.lq_dev->s1xs2 : p.s1xs2, e_m1 = p.lq_dev ? p.lq_dev->m1 : p.m1;
        const float e_m2 = p.lq_dev ? p.lq_dev->m2 : p.m2, e_km = p.lq_dev ? p.lq_dev->k_m1xm2 : p.k_m1xm2;
        // what the Keras layer does behind the op (bias_add, then the activation): fused into the store
        auto finish = [&](float v, int col) {
            if (p.bias)
                v = __fadd_rn(v, p.bias[col]);
            return p.relu ? fmaxf(v, 0.0f) : v;
        };
        constexpr bool kTransposed = NT <= 32;
        // Every global load of the epilogue is issued here, ahead of the first store: loads and stores complete in
        // issue order, so a load behind a store would wait until that store has reached memory.
        float ps[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int64_t m = row0 + (int64_t)(wr_base + r * (kDenseWaves / 2)) * 64 + lane;
            ps[r] = (!OUT_I32 && rvalid[r]) ? p.psum[m] : 0.0f;
        }
        if (kTransposed && (g.Co & 3) == 0) {
            constexpr int Q = NT / 4;                 // 16-byte quads (lanes) per pixel
            constexpr int PITCH = NT * 4 + 16;        // bytes per pixel in LDS: the +16 spreads pixels over the banks
            unsigned char *const wl = lds + (size_t)wave * 64 * PITCH;
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
            auto store_rows = [&](auto has_bias_t, auto has_relu_t) {
            constexpr bool kBias = decltype(has_bias_t)::value, kRelu = decltype(has_relu_t)::value;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r >= (int)nr_s)
                    break;
                const int64_t m0 = row0 + (int64_t)(wr_base + r * (kDenseWaves / 2)) * 64;
                const int nvalid = (int)(row_end - m0 < 64 ? row_end - m0 : 64);
                const float t1 = __fmul_rn(e_m2, ps[r]);
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
                    *reinterpret_cast<u32x4s *>(wl + lane * PITCH + h * 32) = lo;
                    *reinterpret_cast<u32x4s *>(wl + lane * PITCH + h * 32 + 16) = hi;
                }
                uint32_t *const out = OUT_I32 ? reinterpret_cast<uint32_t *>(p.out_i) + (int64_t)ksi * g.M * g.Co
                                              : reinterpret_cast<uint32_t *>(p.out_f);
#pragma unroll
                for (int i = 0; i < Q; ++i) {
                    const int pix = i * (64 / Q) + lane / Q;
                    u32x4s d = *reinterpret_cast<const u32x4s *>(wl + pix * PITCH + quad * 16);
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
            continue;
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (!rvalid[r])
                continue;
            const int64_t m = row0 + (int64_t)(wr_base + r * (kDenseWaves / 2)) * 64 + lane;
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
}

template <int NT, bool OUT_I32>
static hipError_t launch_one(const DenseParams &p, hipStream_t stream)
{
    auto kernel = lutgemm_expand_kernel<NT, OUT_I32>;
    // The generated assembly addresses LDS from offset 0: that holds as long as the kernel has no static LDS in
    // front of its dynamic allocation (checked when the attribute is set, once per device).
    const hipError_t e = set_max_dynamic_lds_once(reinterpret_cast<const void *>(kernel),
                                                  kDenseLdsBytes + kDenseParkBytes, true);
    if (e != hipSuccess)
        return e;
    hipLaunchKernelGGL(kernel, dim3(p.plan.grid), dim3(kDenseThreads), kDenseLdsBytes + kDenseParkBytes, stream, p);
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
