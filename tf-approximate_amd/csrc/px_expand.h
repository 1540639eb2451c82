// Building the pre-expanded rows that lutgemm_px_kernel.hip reads:
//
//   E[column tile][fill][phys_row(a)][slot] = T[a][filter code of slot],   256 rows x 128 slots x uint16 = 64 KiB
//
// A "part" is the rows of CB activation codes of one (column tile, fill), built by 4 * CB threads.  Thread
// (a, quarter) gathers 32 of the 128 entries of activation code a - 32 independent two-byte loads out of the
// L2-resident table, coalesced over a - into LDS (row a, 65 dwords apart: no bank conflicts); then every wavefront
// copies whole 256-byte rows to memory, one row per store instruction, to the rows phys_row() gives the codes.
// Parts rather than whole fills where workgroups are small: several fit a CU, so a layer's few hundred fills spread
// evenly over the CUs instead of as one round and a remainder.
//
// Used by px_expand_rows_kernel (a launch of its own, filter codes read from the packed filter) and by the patch-sum
// launches of prepass_kernels.hip, which carry the same work in further workgroups (filter codes computed from the
// filter itself, since the packed filter is written by other workgroups of the same launch).
#pragma once
#include "axconv_internal.h"

namespace axc {

constexpr int kPxFillBytes = 65536;     // one pre-expanded fill: 256 activation rows x 128 slots x uint16
constexpr int kPxExpandPitch = 65;      // dwords per activation row in the LDS stage

template <int CB>
constexpr int px_expand_stage_dwords() { return CB * kPxExpandPitch; }

// stage: CB * kPxExpandPitch dwords of LDS; code_of(s): filter code of slot s (0..127) of the fill; dst: the fill's
// 64 KiB in memory; part: which CB activation codes.  All 4 * CB threads of the workgroup's first wavefronts call it
// (threadIdx.x < 4 * CB); contains a barrier that every thread of the workgroup must reach: threads beyond 4 * CB
// call px_expand_idle() instead.
template <int CB, typename CodeOf>
__device__ __forceinline__ void px_expand_part(uint32_t *__restrict__ stage, const int part, CodeOf code_of,
                                               const uint16_t *__restrict__ tableT, uint32_t *__restrict__ dst)
{
    const uint32_t al = threadIdx.x % CB, a = (uint32_t)part * CB + al;
    const int quarter = __builtin_amdgcn_readfirstlane((int)(threadIdx.x / CB));
#pragma unroll
    for (int d = 0; d < 16; ++d) {
        const uint32_t lo = tableT[(uint32_t)code_of(quarter * 32 + 2 * d) * 256u + a];
        const uint32_t hi = tableT[(uint32_t)code_of(quarter * 32 + 2 * d + 1) * 256u + a];
        stage[al * kPxExpandPitch + quarter * 16 + d] = lo | (hi << 16);
    }
    __syncthreads();
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    constexpr int kWaves = 4 * CB / 64, kPer = CB / kWaves;
#pragma unroll
    for (int i = 0; i < kPer; ++i) {
        const uint32_t cl = wave * kPer + i;                     // code of this part
        const uint32_t code = (uint32_t)part * CB + cl;
        dst[phys_row(code) * 64u + lane] = stage[cl * kPxExpandPitch + lane];
    }
}

} // namespace axc
