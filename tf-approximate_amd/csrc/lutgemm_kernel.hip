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
#include "lutgemm_tile.h"
#include "lookup_asm.inc"

namespace axc {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

extern __shared__ __align__(16) unsigned char lds[];

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
    // xq ends with one extra input row filled with the zero-point code: taps outside the image read it
    const uint32_t zp_row = p.xq_bytes;
    const rsrc_t xq_rsrc = make_rsrc(p.xq, p.xq_bytes + p.zp_tail_bytes);
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
    uint32_t nr = 0;                 // pixels of this lane whose wavefront row exists (a prefix; wave-uniform)
    for (int tile = wg; tile < ntiles; tile += G) {
        const int rt = tile / nct_v;
        int ct = tile - rt * nct_v;
        const int ksi = ct / p.plan.n_col_tiles;           // K split of this tile
        ct -= ksi * p.plan.n_col_tiles;
        const int f0 = ksi * p.plan.fills_per_split;        // its fills: [f0, f0 + fills)
        const int fills = fills_all - f0 < p.plan.fills_per_split ? fills_all - f0 : p.plan.fills_per_split;
        // ---- which wavefront-rows (64 consecutive output pixels) of the tile this wavefront owns, and the
        // per-pixel geometry (parked in LDS, in slots private to the thread; only read back when the tap changes).
        // The geometry depends on the row tile alone: kept from the previous tile when that had the same one.
        const TileRows t = tile_rows_of<R>(p, rt, wave);
        if (rt != prev_rt) {
            prev_rt = rt;
            nr = park_geometry<R>(p, t, lane, park);
        }

        const uint32_t wq_tile = ((uint32_t)ct * (uint32_t)fills_all + (uint32_t)f0) * 128u; // this tile's first codes
        const int fills_left = fills_all - f0;              // codes may be prefetched past the split, not past the end

        // ---- activation cursor: position (tap, quad) of the fill whose activations are fetched next ----
        int cur_fill = 0, cur_sub = f0 % SUBS;
        int cur_q = (f0 / SUBS) % g.C4, cur_kh = (f0 / SUBS / g.C4) / g.KW, cur_kw = (f0 / SUBS / g.C4) % g.KW;
        uint32_t idx_tap[R];   // byte offset in xq of quad 0 of the current tap (the zero-point row outside)
        auto tap_setup = [&]() { tap_offsets<R>(p, park, cur_kh, cur_kw, zp_row, idx_tap); };
        auto load_acts = [&](uint32_t (&dst)[R]) {
            const uint32_t qoff = (uint32_t)cur_q * p.quad_bytes; // scalar: channel quad inside the pixel row
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
            const uint32_t qoff = (uint32_t)cur_q * p.quad_bytes;
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

        fix_even_columns<R, NT>(acc);
        // every buffer is free after the last phase: the epilogue turns its outputs through the expanded rows
        store_tile<NT, OUT_I32>(p, acc, t, ct, ksi, nr_s, lane, wave, lds);
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
