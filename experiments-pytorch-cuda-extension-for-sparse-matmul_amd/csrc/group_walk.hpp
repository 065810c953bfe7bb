// Pieces the walks over groups of a block table share (matmul.hip, bin_walk.hip): where a wave's
// 32 x 64 result tile goes, and how the parts of a group that was cut across workgroups meet.
#pragma once

#include "bsa_device.hpp"

namespace bsa {

constexpr int GW_LDS_PER_WAVE = 8192;   // staging tiles (2 KB + 4 KB), reused for the fp32 partial tile

// workgroup barrier that orders LDS traffic only: global loads in flight stay in flight
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <bool DSD>
__device__ __forceinline__ size_t gw_out_offset(int g, int y0, int yt, int l, int DN, int XT)
{
    int h = l >> 5, i = l & 31;
    if (DSD) return (size_t)(BS * g + i) * DN + y0 + 32 * yt + 16 * h;
    return (size_t)(y0 + 32 * yt + i) * XT + BS * g + 16 * h;
}

// Split groups: every part parks its fp32 partial tile in the workspace and bumps
// the group's counter; the part that arrives last adds the tiles up in part order
// (so the sum does not depend on arrival order), resets the counter and returns
// true: it stores the result.  Publication follows the release / acquire pattern
// of split_publish / split_consume (bsa_device.hpp).
struct SplitWorkspace {
    int *counters;     // [batches][strips][split_groups], zero between launches
    float *tiles;      // [batches][strips][tile_slots][2048]
    int tile_slots, split_groups;
};

// part `part` of `parts`; the group's tiles start at `tile_slot`, its counter is number `counter_index`
template <class V, int NT, int EV>
__device__ __forceinline__ bool split_combine_at(V (&acc)[NT], int part, int parts, int tile_slot, int counter_index,
                                                 const SplitWorkspace &ws, int batch)
{
    const int l = lane_id();
    const size_t cell = (size_t)batch * gridDim.y + blockIdx.y;
    float *tile0 = ws.tiles + (cell * ws.tile_slots + tile_slot) * 2048;
    float *mine = tile0 + (size_t)part * 2048;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < EV; ++v) park_store(mine + (t * EV + v) * WAVE + l, acc[t][v]);
    int *counter = ws.counters + cell * ws.split_groups + counter_index;
    if (split_publish(counter) != parts - 1) return false;
    split_consume();
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int v = 0; v < EV; ++v) acc[t][v] = 0.f;
    for (int p = 0; p < parts; ++p) {
        const float *src = tile0 + (size_t)p * 2048;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int v = 0; v < EV; ++v) acc[t][v] += park_load(src + (t * EV + v) * WAVE + l);
    }
    split_reset(counter);
    return true;
}

template <class V, int NT, int EV>
__device__ __forceinline__ bool split_combine(V (&acc)[NT], const SchedEntry &e, const SchedGroup &sg,
                                              const SplitWorkspace &ws, int batch)
{
    return split_combine_at<V, NT, EV>(acc, e.part(), e.parts(), sg.tile_slot, sg.split_index, ws, batch);
}

}  // namespace bsa
