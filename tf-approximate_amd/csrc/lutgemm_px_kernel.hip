// Dense LUT-GEMM out of PRE-EXPANDED rows (gfx950), for layers with many output pixels and a small filter.
//
// lutgemm_kernel.hip builds the expanded rows of every fill inside every workgroup: table rows are staged in LDS
// and transposed, once per (tile, fill).  Here px_expand_rows_kernel builds them once per layer in memory:
//
//   E[column tile][fill][phys_row(a)][slot]  = T[a][filter code of slot],   256 rows x 128 slots x uint16 = 64 KiB
//
// where a fill is a PAIR of the other kernel's fills: 8 input channels (two channel quads of one tap) x 16 columns,
// slot = quad-in-pair * 64 + channel-in-quad * 16 + column.  The lookup kernel then only copies fills from memory
// (L2: the workgroups of an XCD walk the same few column tiles at the same time) straight into LDS with buffer
// loads that carry the lds modifier - no staged table rows, no transposition, half as many barriers - and, because
// an expanded row is now 256 bytes, a 64-lane ds_read_b128 spreads over all 64 banks.
//
// LDS: two fill buffers of 64 KiB, then the parked pixel geometry (32 KiB).  While fill p is looked up out of one
// buffer, fill p + 1 lands in the other; a tile starts in buffer 0, which receives the first fill of the
// workgroup's next tile as soon as the last fill that used it is done, and the epilogue turns its outputs through
// buffer 1.
//
// Restates ApproxConvIm2ColKernel + ApproxConvGEMMKernel (tf2/src/approx_nn_conv_kernels.cpp:215-296) like the
// other kernel; results are bit-identical to it (same int32 sums, same epilogue).
#include "lutgemm_tile.h"
#include "px_expand.h"
#include "lookup_asm.inc"

namespace axc {

extern __shared__ __align__(16) unsigned char lds_px[];

constexpr int kPxBlockCols = 4;         // column tiles that the workgroups of an XCD walk side by side

// One workgroup per (column tile, fill, part): see px_expand.h.
constexpr int kPxExpandParts = 2;
constexpr int kPxExpandCodes = 256 / kPxExpandParts;
__global__ void __launch_bounds__(4 * kPxExpandCodes) px_expand_rows_kernel(const uint16_t *__restrict__ wq,
                                                                            const uint16_t *__restrict__ tableT,
                                                                            const int fills, uint16_t *__restrict__ rows)
{
    __shared__ uint32_t stage[px_expand_stage_dwords<kPxExpandCodes>()];
    const int px_fills = fills / 2;
    const int part = (int)blockIdx.x % kPxExpandParts, cf = (int)blockIdx.x / kPxExpandParts;   // cf = ct * px_fills + f
    const int ct = cf / px_fills, f = cf - ct * px_fills;
    // the codes of the two ordinary fills of this pair lie side by side: 128 uint16
    const uint16_t *codes = wq + ((size_t)ct * fills + 2 * (size_t)f) * 64;
    px_expand_part<kPxExpandCodes>(stage, part, [&](const int s) { return codes[s]; }, tableT,
                                   reinterpret_cast<uint32_t *>(rows + (size_t)cf * (kPxFillBytes / 2)));
}

hipError_t launch_px_expand_rows(const uint16_t *wq, const uint16_t *tableT, const DensePlan &plan, uint16_t *rows,
                                 hipStream_t stream)
{
    const int blocks = plan.n_col_tiles * (plan.fills / 2) * kPxExpandParts;
    hipLaunchKernelGGL(px_expand_rows_kernel, dim3(blocks), dim3(4 * kPxExpandCodes), 0, stream, wq, tableT, plan.fills,
                       rows);
    return hipGetLastError();
}

template <bool OUT_I32>
__global__ void __launch_bounds__(kDenseThreads) lutgemm_px_kernel(const DenseParams p)
{
    constexpr int NT = 16, R = 8;
    const ConvGeom &g = p.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- lane constants ----
    // A pixel is looked up in two units of eight steps, one per activation dword.  Step s of a unit reads chunk
    // (c0 + s) & 7 of one half of the 256-byte row; lanes with bit 3 set keep their two dwords swapped and read the
    // upper half first, so the 16 lanes of an LDS pass touch 16 different chunks whatever their codes are.
    // Chunk c of a half holds input channel c >> 1 of its quad, column group c & 1.  The address
    // (row << 8 | half << 7 | c << 4) is one v_perm_b32: byte 1 <- activation byte c >> 1, byte 0 <- the chunk byte.
    const int c0 = lane & 7;
    const uint32_t upper = ((uint32_t)lane >> 3) & 1u;
    uint32_t sel[8];
    uint32_t ch[2][4] = {{0, 0, 0, 0}, {0, 0, 0, 0}};   // [buffer][unit * 2 + (step >> 2)]: four chunk bytes each
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const uint32_t c = (uint32_t)(c0 + s) & 7u;
        sel[s] = 0x0c0c0000u | ((4u + (c >> 1)) << 8) | (uint32_t)(s & 3);
#pragma unroll
        for (int unit = 0; unit < 2; ++unit) {
            const uint32_t half = (uint32_t)unit ^ upper;
            const uint32_t byte = ((half << 3) | c) << 4;
            ch[0][unit * 2 + (s >> 2)] |= byte << (8 * (s & 3));
            // buffer 1 starts 65536 bytes in, one more than an instruction offset holds: +15 here, +65521 there
            ch[1][unit * 2 + (s >> 2)] |= (byte | 15u) << (8 * (s & 3));
        }
    }
    const uint32_t l16 = (uint32_t)lane * 16u;
    uint32_t *const park = reinterpret_cast<uint32_t *>(lds_px + 2 * kPxFillBytes) + tid;

    // a tile = (row tile, column tile, K split); the K splits of a column tile count as further column tiles
    const int n_col = p.plan.n_col_tiles * p.plan.k_splits, n_row = p.plan.n_row_tiles;
    const int ntiles = n_row * n_col;
    const int F = p.plan.fills / 2;                 // pre-expanded fills over K
    const int Fs = p.plan.k_splits > 1 ? p.plan.fills_per_split / 2 : F;   // ... and per K split
    const int qpairs = g.C4 / 2;                    // fills per tap
    const uint32_t quad_bytes = p.quad_bytes;        // between the channel quads of a pixel in xq
    const uint32_t dlf = upper ? quad_bytes : 0u;   // this lane's FIRST dword is the pair's second quad if swapped
    const uint32_t dls = upper ? 0u : quad_bytes;
    const uint32_t zp_row = p.xq_bytes;             // one extra input row of the zero-point code behind xq
    const rsrc_t xq_rsrc = make_rsrc(p.xq, p.xq_bytes + p.zp_tail_bytes);
    const rsrc_t e_rsrc = make_rsrc(p.px_rows, p.px_bytes);

    // Tiles in blocks of kPxBlockCols column tiles: inside a block row tile after row tile, the column tile fastest.
    // The workgroups of an XCD (own L2) work on neighbouring tiles at the same time: the same few column tiles (same
    // pre-expanded rows) of a few row tiles (same activations).
    auto decode = [&](const int tile, int &rt, int &ct) __attribute__((always_inline)) {
        const int per_block = n_row * kPxBlockCols;
        const int cb = tile / per_block;
        const int in_block = tile - cb * per_block;
        const int left = n_col - cb * kPxBlockCols;
        const int w = left < kPxBlockCols ? left : kPxBlockCols;
        rt = in_block / w;
        ct = cb * kPxBlockCols + in_block - rt * w;
    };
    // Workgroups are handed to the 8 XCDs round-robin.  Each XCD gets one contiguous eighth of the tiles and its
    // workgroups walk it side by side (workgroup i of the XCD takes its tiles i, i + 32, ...): an XCD stays with the
    // same few column blocks for the whole launch, so their rows are fetched into its L2 once.
    const int G = (int)gridDim.x;
    int tile_first, tile_end, tile_step;
    if ((G & 7) == 0) {
        const int xcd = (int)blockIdx.x & 7, i = (int)blockIdx.x >> 3;
        tile_first = (int)((int64_t)ntiles * xcd / 8) + i;
        tile_end = (int)((int64_t)ntiles * (xcd + 1) / 8);
        tile_step = G >> 3;
    } else {
        tile_first = (int)blockIdx.x;
        tile_end = ntiles;
        tile_step = G;
    }
    if (p.stagger_sleeps) {
        const int late = p.stagger_sleeps * ((tile_first / (n_col < kPxBlockCols ? n_col : kPxBlockCols)) % p.stagger_groups);
        for (int i = 0; i < late; ++i)
            __builtin_amdgcn_s_sleep(127);
    }

    int prev_rt = -1;
    uint32_t nr = 0;
    const uint32_t edst = (uint32_t)wave * 8192u;   // this wavefront's eighth of a fill, in memory and in LDS
    // the first fill of a tile (column tile incl. K split ctv) -> buffer 0: eight loads of 1 KiB, memory straight
    // into LDS
    auto load_first_fill = [&](const int ctv) __attribute__((always_inline)) {
        const int ksi = ctv / p.plan.n_col_tiles;
        const uint32_t eoff = (uint32_t)((ctv - ksi * p.plan.n_col_tiles) * F + ksi * Fs) * (uint32_t)kPxFillBytes + edst;
#pragma unroll
        for (int j = 0; j < 8; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(
                e_rsrc, (__attribute__((address_space(3))) void *)(lds_px + edst + j * 1024u), 16, (int)l16,
                (int)(eoff + j * 1024u), 0, 0);
    };
    if (tile_first < tile_end) {
        int rt0, ct0;
        decode(tile_first, rt0, ct0);
        load_first_fill(ct0);
    }
    for (int tile = tile_first; tile < tile_end; tile += tile_step) {
        int rt, ctv;
        decode(tile, rt, ctv);
        int ctv_next = ctv;
        const bool has_next = tile + tile_step < tile_end;
        if (has_next) {
            int rt_next;
            decode(tile + tile_step, rt_next, ctv_next);
        }
        const int ksi = ctv / p.plan.n_col_tiles;           // K split of this tile
        const int ct = ctv - ksi * p.plan.n_col_tiles;
        const int f0 = ksi * Fs;                            // its fills: [f0, f0 + Ft)
        const int Ft = F - f0 < Fs ? F - f0 : Fs;
        const int ksi_next = ctv_next / p.plan.n_col_tiles;
        const uint32_t first_fill = (uint32_t)(ct * F + f0);
        const uint32_t first_fill_next = (uint32_t)((ctv_next - ksi_next * p.plan.n_col_tiles) * F + ksi_next * Fs);
        const TileRows t = tile_rows_of<R, true>(p, rt, wave);
        if (rt != prev_rt) {
            prev_rt = rt;
            nr = park_geometry<R>(p, t, lane, park);
        }
        const uint32_t nr_s = __builtin_amdgcn_readfirstlane(nr);

        // ---- activation cursor: (tap, quad pair) of the fill whose activations are fetched next ----
        int cur_fill = 0, cur_qp = 0, cur_kh = 0, cur_kw = 0;   // cur_fill counts from the tile's first fill
        if (f0) {
            const int tap = f0 / qpairs;
            cur_qp = f0 - tap * qpairs;
            cur_kh = tap / g.KW;
            cur_kw = tap - cur_kh * g.KW;
        }
        uint32_t idx_tap[R];
        tap_offsets<R>(p, park, cur_kh, cur_kw, zp_row, idx_tap);
        auto advance_cursor = [&]() __attribute__((always_inline)) {
            ++cur_fill;
            if (++cur_qp == qpairs) {
                cur_qp = 0;
                if (++cur_kw == g.KW) { cur_kw = 0; ++cur_kh; }
                if (cur_fill < Ft)   // pixel 0's activations are fetched whether the wavefront has a pixel or not
                    tap_offsets<R>(p, park, cur_kh, cur_kw, zp_row, idx_tap, nr_s > 1u ? nr_s : 1u);
            }
        };
        uint32_t fA[R], sA[R], fB[R], sB[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            fA[r] = ld_u32(xq_rsrc, idx_tap[r] + dlf, (uint32_t)cur_qp * 2u * quad_bytes);
            sA[r] = ld_u32(xq_rsrc, idx_tap[r] + dls, (uint32_t)cur_qp * 2u * quad_bytes);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): this wavefront's part of fill 0 and its activations are there
        __syncthreads();                      // ... and everyone's; the previous tile's epilogue is done with LDS

        int32_t acc[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                acc[r][j] = 0;

        if (Ft > 1)
            advance_cursor();   // entering phase p the cursor stands on fill p + 1
        auto phase = [&](const int pcur, uint32_t (&f_cur)[R], uint32_t (&s_cur)[R], uint32_t (&f_next)[R],
                         uint32_t (&s_next)[R], auto buf_tag) __attribute__((always_inline)) {
            constexpr int BUF = decltype(buf_tag)::value;
            // What lands in the other buffer during this phase: the next fill of this tile.  Behind the last fill of
            // an even count the other buffer is buffer 0, and it gets the first fill of the workgroup's next tile;
            // otherwise the last fill once more (never used).
            uint32_t fill_next = first_fill + (uint32_t)(pcur + 1);
            if (pcur + 1 >= Ft)
                fill_next = (BUF == 1 && has_next) ? first_fill_next : first_fill + (uint32_t)(Ft - 1);
            const uint32_t eoff = fill_next * (uint32_t)kPxFillBytes + edst;
            const uint32_t qoff = (uint32_t)cur_qp * 2u * quad_bytes;
            uint32_t stmp;
            if constexpr (BUF == 0)
                PHASE_PX_B0(acc, f_cur, s_cur, f_next, s_next, idx_tap, sel, ch[0], dlf, dls, l16, nr_s, stmp,
                            __builtin_amdgcn_readfirstlane(edst), __builtin_amdgcn_readfirstlane(eoff), e_rsrc, xq_rsrc,
                            __builtin_amdgcn_readfirstlane(qoff));
            else
                PHASE_PX_B1(acc, f_cur, s_cur, f_next, s_next, idx_tap, sel, ch[1], dlf, dls, l16, nr_s, stmp,
                            __builtin_amdgcn_readfirstlane(edst), __builtin_amdgcn_readfirstlane(eoff), e_rsrc, xq_rsrc,
                            __builtin_amdgcn_readfirstlane(qoff));
            (void)stmp;
            if (pcur + 2 < Ft)
                advance_cursor();
            __syncthreads();
        };
        for (int pcur = 0; pcur < Ft; pcur += 2) {
            phase(pcur, fA, sA, fB, sB, std::integral_constant<int, 0>());
            if (pcur + 1 < Ft)
                phase(pcur + 1, fB, sB, fA, sA, std::integral_constant<int, 1>());
        }
        // An odd count of fills ends on buffer 0, which every wavefront has now left: the next tile's first fill
        // goes there while the epilogue runs.  The epilogue turns its outputs through buffer 1 either way.
        if ((Ft & 1) && has_next)
            load_first_fill(ctv_next);
        fix_even_columns<R, NT>(acc);
        store_tile<NT, OUT_I32>(p, acc, t, ct, ksi, nr_s, lane, wave, lds_px + kPxFillBytes);
    }
}

// Control block in LDS, the last 32 bytes (see gen_lookup_asm.py): EVENTS[0], EVENTS[1], ABORT.  EVENTS[b] only grows,
// by one per wavefront and event: eight arrivals of the buffer's fill j, then its eight readers, then the arrivals of
// fill j + 1, ...
constexpr uint32_t kPxCb = 2 * kPxFillBytes + kDenseParkBytes - 32;
constexpr uint32_t kPxAll = kDenseWaves;
constexpr uint32_t kPxIssued = 0xfffffffeu;   // TGT of a phase whose loads are issued
constexpr uint32_t kPxCounted = 0xffffffffu;  // ... and whose wavefront has counted their arrival (or has none to issue)
// EVENTS of a buffer when its fill j is whole / when all have read it
__device__ __forceinline__ uint32_t px_whole(const uint32_t j) { return kPxAll * (2u * j + 1u); }
__device__ __forceinline__ uint32_t px_free(const uint32_t j) { return kPxAll * (2u * j + 2u); }

// One look at the two counters: an 8-byte LDS read that every lane makes of the same address, waited for here.
__device__ __forceinline__ void px_read_events(uint32_t (&ev)[2])
{
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    u32x2 v;
    asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(kPxCb) : "memory");
    ev[0] = __builtin_amdgcn_readfirstlane(v.x);
    ev[1] = __builtin_amdgcn_readfirstlane(v.y);
}
__device__ __forceinline__ uint32_t px_read_abort()
{
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1 offset:8\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(kPxCb) : "memory");
    return __builtin_amdgcn_readfirstlane(v);
}
// EVENTS[buffer] += 1 by one lane of the wavefront (64 atomics on one address would hold the LDS for as many turns;
// LDS atomics of one CU execute in the order they arrive)
__device__ __forceinline__ void px_count(const uint32_t buffer, const int lane)
{
    if (lane == 0)
        asm volatile("ds_add_u32 %0, %1" : : "v"(kPxCb + 4u * buffer), "v"(1u) : "memory");
}

// The wavefronts of a workgroup stream through the same sequence of fills g = 0, 1, 2, ... (all fills of the
// workgroup's first tile, then of its second, ...), fill g in buffer g & 1, without a barrier between fills:
//   * a wavefront reads fill g once all eight eighths of it have arrived (EVENTS[g & 1] at px_whole(g / 2));
//   * it copies its eighth of fill g + 1 into the other buffer once all eight wavefronts have finished fill g - 1, the
//     last one to use that buffer (EVENTS[(g + 1) & 1] at px_free((g - 1) / 2)).  It looks at that counter once per
//     pixel inside the phase body, issues the loads at the first look that finds the buffer free and counts its
//     arrival at the first later look that finds none of its loads in flight; what the body has not done by its end
//     is done behind it.
//     Then it counts itself as a reader of fill g and goes on.
// Each wavefront is therefore at most one fill ahead of the slowest one, the slowest one never waits, and two
// wavefronts of a SIMD ramp their read windows up and down at different times.  Every wait is a bounded number of
// polls; a wavefront whose wait runs out raises ABORT, reports through p.wait_error and leaves the kernel, and so do
// the others when they next wait.
template <bool OUT_I32, bool OWN_SPLIT>
__global__ void __launch_bounds__(kDenseThreads) lutgemm_pxf_kernel(const DenseParams p)
{
    constexpr int NT = 16, R = 8, PS = 64;   // PS: dwords between a thread's geometry slots (wavefront-major)
    const ConvGeom &g = p.g;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

    // ---- lane constants ----
    // A pixel is looked up in two units of eight steps, one per activation dword.  Step s of a unit reads chunk
    // (c0 + s) & 7 of one half of the 256-byte row; lanes with bit 3 set keep their two dwords swapped and read the
    // upper half first, so the 16 lanes of an LDS pass touch 16 different chunks whatever their codes are.
    // Chunk c of a half holds input channel c >> 1 of its quad, column group c & 1.  The address
    // (buffer << 16 | row << 8 | half << 7 | c << 4) is one v_perm_b32: byte 2 <- byte 3 of the chunk register (the
    // buffer the phase reads: flipped between phases), byte 1 <- activation byte c >> 1, byte 0 <- the chunk byte.
    const int c0 = lane & 7;
    const uint32_t upper = ((uint32_t)lane >> 3) & 1u;
    uint32_t sel[8];
    uint32_t ch[6] = {0, 0, 0, 0, 0, 0};   // [unit * 3 + step / 3]: chunk bytes of three steps, then the buffer byte
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        const uint32_t c = (uint32_t)(c0 + s) & 7u;
        sel[s] = 0x0c030000u | ((4u + (c >> 1)) << 8) | (uint32_t)(s % 3);
#pragma unroll
        for (int unit = 0; unit < 2; ++unit) {
            const uint32_t half = (uint32_t)unit ^ upper;
            ch[unit * 3 + s / 3] |= (((half << 3) | c) << 4) << (8 * (s % 3));
        }
    }
    const uint32_t l16 = (uint32_t)lane * 16u;
    // per-wavefront 4 KiB behind the two fill buffers: the parked geometry, overwritten by the epilogue (which turns
    // its outputs through the first 2.5 KiB) and rebuilt for every tile.  The control block is the tail of the last
    // wavefront's piece: pixel slot 7 of wavefront 7, which a tile of at most 63 wavefront-rows never has.
    unsigned char *const wave_lds = lds_px + 2 * kPxFillBytes + wave * (kDenseParkBytes / kDenseWaves);
    uint32_t *const park = reinterpret_cast<uint32_t *>(wave_lds) + lane;
    const int skip_row = wave == kDenseWaves - 1 ? R - 1 : -1;

    if (tid < 8)
        reinterpret_cast<volatile uint32_t *>(lds_px + kPxCb)[tid] = 0u;
    __syncthreads();   // the only barrier of the kernel

    // a tile = (row tile, column tile, K split); the K splits of a column tile count as further column tiles
    const int n_col = p.plan.n_col_tiles * p.plan.k_splits, n_row = p.plan.n_row_tiles;
    const int ntiles = n_row * n_col;
    const int F = p.plan.fills / 2;                 // pre-expanded fills over K
    const int Fs = p.plan.k_splits > 1 ? p.plan.fills_per_split / 2 : F;   // ... and per K split
    const int qpairs = g.C4 / 2;                    // fills per tap
    const uint32_t quad_bytes = p.quad_bytes;        // between the channel quads of a pixel in xq
    const uint32_t dlf = upper ? quad_bytes : 0u;   // this lane's FIRST dword is the pair's second quad if swapped
    const uint32_t dls = upper ? 0u : quad_bytes;
    const uint32_t zp_row = p.xq_bytes;             // one extra input row of the zero-point code behind xq
    const rsrc_t xq_rsrc = make_rsrc(p.xq, p.xq_bytes + p.zp_tail_bytes);
    const rsrc_t e_rsrc = make_rsrc(p.px_rows, p.px_bytes);

    // Tiles in blocks of kPxBlockCols column tiles: inside a block row tile after row tile, the column tile fastest.
    // The workgroups of an XCD (own L2) work on neighbouring tiles at the same time: the same few column tiles (same
    // pre-expanded rows) of a few row tiles (same activations).
    auto decode = [&](const int tile, int &rt, int &ct) __attribute__((always_inline)) {
        const int per_block = n_row * kPxBlockCols;
        const int cb = tile / per_block;
        const int in_block = tile - cb * per_block;
        const int left = n_col - cb * kPxBlockCols;
        const int w = left < kPxBlockCols ? left : kPxBlockCols;
        rt = in_block / w;
        ct = cb * kPxBlockCols + in_block - rt * w;
    };
    // Workgroups are handed to the 8 XCDs round-robin.  Each XCD gets one contiguous eighth of the tiles and its
    // workgroups walk it side by side (workgroup i of the XCD takes its tiles i, i + 32, ...): an XCD stays with the
    // same few column blocks for the whole launch, so their rows are fetched into its L2 once.
    const int G = (int)gridDim.x;
    int tile_first, tile_end, tile_step;
    if ((G & 7) == 0) {
        const int xcd = (int)blockIdx.x & 7, i = (int)blockIdx.x >> 3;
        tile_first = (int)((int64_t)ntiles * xcd / 8) + i;
        tile_end = (int)((int64_t)ntiles * (xcd + 1) / 8);
        tile_step = G >> 3;
    } else {
        tile_first = (int)blockIdx.x;
        tile_end = ntiles;
        tile_step = G;
    }
    if (p.stagger_sleeps) {
        const int late = p.stagger_sleeps * ((tile_first / (n_col < kPxBlockCols ? n_col : kPxBlockCols)) % p.stagger_groups);
        for (int i = 0; i < late; ++i)
            __builtin_amdgcn_s_sleep(127);
    }

    const uint32_t edst = (uint32_t)wave * 8192u;   // this wavefront's eighth of a fill, in memory and in LDS
    // this wavefront's eighth of the fill at `fill` (an index into the rows in memory) -> LDS buffer `buf`: eight loads
    // of 1 KiB, memory straight into LDS
    auto load_fill = [&](const uint32_t fill, const uint32_t buf) __attribute__((always_inline)) {
        const uint32_t eoff = fill * (uint32_t)kPxFillBytes + edst;
        // LDS addresses as integers: the kernel's dynamic LDS starts at 0 (checked at launch)
        const uint32_t dst = __builtin_amdgcn_readfirstlane(edst + buf * (uint32_t)kPxFillBytes);
#pragma unroll
        for (int j = 0; j < 8; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(e_rsrc, (__attribute__((address_space(3))) void *)(uintptr_t)(dst + j * 1024u), 16,
                                                     (int)l16, (int)(eoff + j * 1024u), 0, 0);
    };
    auto first_fill_of = [&](const int ctv) __attribute__((always_inline)) {
        const int ksi = ctv / p.plan.n_col_tiles;
        return (uint32_t)((ctv - ksi * p.plan.n_col_tiles) * F + ksi * Fs);
    };
    // A wait that ran out: tell the host and the other wavefronts.
    auto give_up = [&](const uint32_t code) __attribute__((always_inline)) {
        if (lane == 0) {
            reinterpret_cast<volatile uint32_t *>(lds_px + kPxCb)[2] = 1u;
            if (p.wait_error)
                __hip_atomic_store(p.wait_error, code, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        }
    };
    // Polls until EVENTS[buffer] has reached `target`; false if the wait ran out or another wavefront has given up.
    // `ev` returns the last look at both counters.
    auto wait_for = [&](const uint32_t buffer, const uint32_t target, uint32_t (&ev)[2]) __attribute__((always_inline)) {
        for (uint32_t polls = 0;; ++polls) {
            px_read_events(ev);
            if ((buffer ? ev[1] : ev[0]) >= target)
                return true;
            if (polls >= p.spin_limit || px_read_abort() != 0u)
                return false;
            __builtin_amdgcn_s_sleep(2);
        }
    };

    uint32_t gf = 0;   // fills this workgroup has begun, over all its tiles: the next fill to look up is fill gf
    uint32_t seen = 0;   // EVENTS of the buffer of fill gf as the last poll of the phase before saw it
    if (tile_first < tile_end) {
        int rt0, ct0;
        decode(tile_first, rt0, ct0);
        load_fill(first_fill_of(ct0), 0u);
    }
    bool first_tile = true;
    for (int tile = tile_first; tile < tile_end; tile += tile_step) {
        int rt, ctv;
        decode(tile, rt, ctv);
        int ctv_next = ctv;
        const bool has_next = tile + tile_step < tile_end;
        if (has_next) {
            int rt_next;
            decode(tile + tile_step, rt_next, ctv_next);
        }
        const int ksi = ctv / p.plan.n_col_tiles;           // K split of this tile
        const int ct = ctv - ksi * p.plan.n_col_tiles;
        const int f0 = ksi * Fs;                            // its fills: [f0, f0 + Ft)
        const int Ft = F - f0 < Fs ? F - f0 : Fs;
        const uint32_t first_fill = (uint32_t)(ct * F + f0);
        const uint32_t first_fill_next = first_fill_of(ctv_next);
        const TileRows t = tile_rows_of<R, true, true, OWN_SPLIT>(p, rt, wave);
        const uint32_t nr = park_geometry<R, PS>(p, t, lane, park, skip_row);
        const uint32_t nr_s = __builtin_amdgcn_readfirstlane(nr);

        // ---- activation cursor: (tap, quad pair) of the fill whose activations are fetched next ----
        int cur_fill = 0, cur_qp = 0, cur_kh = 0, cur_kw = 0;   // cur_fill counts from the tile's first fill
        if (f0) {
            const int tap = f0 / qpairs;
            cur_qp = f0 - tap * qpairs;
            cur_kh = tap / g.KW;
            cur_kw = tap - cur_kh * g.KW;
        }
        uint32_t idx_tap[R];
        tap_offsets<R, PS>(p, park, cur_kh, cur_kw, zp_row, idx_tap);
        auto advance_cursor = [&]() __attribute__((always_inline)) {
            ++cur_fill;
            if (++cur_qp == qpairs) {
                cur_qp = 0;
                if (++cur_kw == g.KW) { cur_kw = 0; ++cur_kh; }
                if (cur_fill < Ft)   // pixel 0's activations are fetched whether the wavefront has a pixel or not
                    tap_offsets<R, PS>(p, park, cur_kh, cur_kw, zp_row, idx_tap, nr_s > 1u ? nr_s : 1u);
            }
        };
        uint32_t fA[R], sA[R], fB[R], sB[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            fA[r] = ld_u32(xq_rsrc, idx_tap[r] + dlf, (uint32_t)cur_qp * 2u * quad_bytes);
            sA[r] = ld_u32(xq_rsrc, idx_tap[r] + dls, (uint32_t)cur_qp * 2u * quad_bytes);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0): the activations are there
        if (first_tile) {                     // ... and this wavefront's part of the workgroup's very first fill
            px_count(0u, lane);
            first_tile = false;
        }

        int32_t acc[R][NT];
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int j = 0; j < NT; ++j)
                acc[r][j] = 0;

        if (Ft > 1)
            advance_cursor();   // entering phase p the cursor stands on fill p + 1
        // One fill: returns false if a wait ran out.
        auto phase = [&](const int pcur, uint32_t (&f_cur)[R], uint32_t (&s_cur)[R], uint32_t (&f_next)[R],
                         uint32_t (&s_next)[R]) __attribute__((always_inline)) {
            const uint32_t buf = __builtin_amdgcn_readfirstlane(gf & 1u), other = buf ^ 1u;
            // the fill that goes into the other buffer while this one is looked up: the next one of this tile, or
            // the first one of the workgroup's next tile; none behind the last fill of the last tile
            const bool loads = pcur + 1 < Ft || has_next;
            const uint32_t fill_next = pcur + 1 < Ft ? first_fill + (uint32_t)(pcur + 1) : first_fill_next;
            const uint32_t eoff = fill_next * (uint32_t)kPxFillBytes + edst;
            const uint32_t qoff = (uint32_t)cur_qp * 2u * quad_bytes;
            // the other buffer is free once all have read its fill (gf - 1) / 2; fill 1 goes into a buffer never used
            uint32_t tgt = !loads ? kPxCounted : gf == 0u ? 0u : px_free((gf - 1u) >> 1);
            if (seen < px_whole(gf >> 1)) {   // the polls of the phase before have not seen this fill whole
                uint32_t ev[2];
                if (!wait_for(buf, px_whole(gf >> 1), ev)) {
                    give_up(1u);
                    return false;
                }
                if (loads && (other ? ev[1] : ev[0]) >= tgt) {   // the other buffer is free already
                    load_fill(fill_next, other);
                    tgt = kPxIssued;
                }
            }
            tgt = __builtin_amdgcn_readfirstlane(tgt);
            uint32_t stmp;
            uint64_t sx;
            PHASE_PXF(acc, f_cur, s_cur, f_next, s_next, idx_tap, sel, ch, dlf, dls, l16, nr_s, stmp, sx, tgt, seen,
                     __builtin_amdgcn_readfirstlane(kPxCb + 4u * other),
                     __builtin_amdgcn_readfirstlane(edst + other * (uint32_t)kPxFillBytes),
                     __builtin_amdgcn_readfirstlane(eoff), e_rsrc, xq_rsrc, __builtin_amdgcn_readfirstlane(qoff));
            (void)stmp;
            (void)sx;
            if (tgt < kPxIssued) {   // the phase body never saw the other buffer free: wait for it here
                uint32_t ev[2];
                if (!wait_for(other, tgt, ev)) {
                    give_up(2u);
                    return false;
                }
                load_fill(fill_next, other);
                __builtin_amdgcn_s_waitcnt(0x0F70);   // vmcnt(0)
                tgt = kPxIssued;
            }
            // the body ends with every load landed and every lookup returned: this wavefront's eighth of the next
            // fill is in LDS (counted, unless the body has done that), and it is done with this buffer
            if (tgt != kPxCounted)
                px_count(other, lane);
            px_count(buf, lane);
            ++gf;
#pragma unroll
            for (int i = 0; i < 6; ++i)
                ch[i] ^= 0x01000000u;   // the next fill is in the other buffer
            if (pcur + 2 < Ft)
                advance_cursor();
            return true;
        };
        for (int pcur = 0; pcur < Ft; pcur += 2) {
            if (!phase(pcur, fA, sA, fB, sB))
                return;
            if (pcur + 1 < Ft && !phase(pcur + 1, fB, sB, fA, sA))
                return;
        }
        fix_even_columns<R, NT>(acc);
        store_tile<NT, OUT_I32, true>(p, acc, t, ct, ksi, nr_s, lane, wave, wave_lds);
    }
}

// FREE_RUNNING: 0 = lutgemm_px_kernel, 1 = lutgemm_pxf_kernel, 2 = lutgemm_pxf_kernel dividing a tile's rows by its
// own rule (a kernel of its own, so that the other keeps its register allocation: with the rule inside, layers it
// does not apply to ran 0.3-0.9 % slower)
template <bool OUT_I32, int FREE_RUNNING>
static hipError_t launch_px_one(const DenseParams &p, hipStream_t stream)
{
    auto kernel = FREE_RUNNING == 2   ? lutgemm_pxf_kernel<OUT_I32, true>
                  : FREE_RUNNING == 1 ? lutgemm_pxf_kernel<OUT_I32, false>
                                      : lutgemm_px_kernel<OUT_I32>;
    // The generated assembly addresses LDS from offset 0: that holds as long as the kernel has no static LDS in
    // front of its dynamic allocation (checked when the attribute is set, once per device).
    const int lds_bytes = 2 * kPxFillBytes + kDenseParkBytes;
    const hipError_t e = set_max_dynamic_lds_once(reinterpret_cast<const void *>(kernel), lds_bytes, true);
    if (e != hipSuccess)
        return e;
    hipLaunchKernelGGL(kernel, dim3(p.plan.grid), dim3(kDenseThreads), lds_bytes, stream, p);
    return hipGetLastError();
}

hipError_t launch_dense_px(const DenseParams &p, bool out_i32, hipStream_t stream)
{
    if (p.plan.nt != 16 || (p.plan.fills & 1) || (p.g.C4 & 1) || !p.px_rows)
        return hipErrorInvalidValue;
    if (p.plan.k_splits > 1 && ((p.plan.fills_per_split & 1) || !out_i32))   // a split covers whole pre-expanded fills
        return hipErrorInvalidValue;
    if (px_free_running(p.plan, p.g.KH * p.g.KW)) {
        if (p.plan.rows_per_tile > 64 * kPxMaxTileWaveRows)   // the control block sits in the last wavefront's last slot
            return hipErrorInvalidValue;
        // tiles whose rows tile_rows_of's OWN_SPLIT divides differently: the full ones or the layer's last
        const int full = p.plan.rows_per_tile / 64;
        const int last = (int)((p.g.M - (int64_t)(p.plan.n_row_tiles - 1) * p.plan.rows_per_tile + 63) / 64);
        if ((full >= kOwnSplitFrom && full <= kOwnSplitTo) || (last >= kOwnSplitFrom && last <= kOwnSplitTo))
            return out_i32 ? launch_px_one<true, 2>(p, stream) : launch_px_one<false, 2>(p, stream);
        return out_i32 ? launch_px_one<true, 1>(p, stream) : launch_px_one<false, 1>(p, stream);
    }
    return out_i32 ? launch_px_one<true, 0>(p, stream) : launch_px_one<false, 0>(p, stream);
}

// Which of the two kernels a plan with pre-expanded rows runs.  Without barriers the wavefronts of a SIMD drift apart
// and fill each other's gaps: measured 3 to 4.5 % faster from 16 fills per tile on with a filter of several taps (3x3
// 64->64 @56x56, the 7x7 stem, 3x3 128->128 @28x28 with its K split), 1 to 2 % at 32 fills of a 1x1 filter (whose
// phases change no tap offsets in either kernel), and slower below (1x1: 4 fills +5 %, 8 fills +1 %, 24 fills +1.5 %: a
// tile's prologue and epilogue, longer in this kernel, weigh more) and on tiles of a single wavefront-row per
// wavefront (+6 %).
bool px_free_running(const DensePlan &plan, int taps)
{
    const int fills_per_tile = (plan.k_splits > 1 ? plan.fills_per_split : plan.fills) / 2;
    const int wrows = plan.rows_per_tile / 64;
    return plan.px && fills_per_tile >= (taps > 1 ? 16 : 32) && wrows >= 2 * kDenseWaves && wrows <= kPxMaxTileWaveRows;
}

} // namespace axc
