// Device-side building blocks shared by the gfx950 kernels: table decode,
// MFMA fragments, the wave-private LDS transpose and the workgroup -> (batch,
// schedule slot) mapping.  gfx950 only: 64-wide wavefronts, v_mfma_f32_32x32x16_f16,
// v_mfma_f32_32x32x2_f32, ds_read_b64_tr_b16.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "lds_index_math.hpp"

namespace bsa {

typedef _Float16 half_t;
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef __fp16 tr4 __attribute__((__vector_size__(4 * sizeof(__fp16))));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));

constexpr int BS = 32;          // block edge
constexpr int BS2 = BS * BS;    // elements per block
constexpr int WAVE = 64;

// One pair of the block table (sparse/native/sparse_layout.cuh:13-21 keeps the
// same two ints; the column is decoded from 16 bits here, not 8).
struct BlockDesc {
    int idx;
    int pos;
    __device__ __forceinline__ int row() const { return (int)((unsigned)pos >> 16); }
    __device__ __forceinline__ int col() const { return pos & 0xFFFF; }
};

// One wavefront slot of a schedule.  A group is cut into `parts` pieces, one team of
// wavefronts each; a team sits inside one workgroup.
struct SchedEntry {
    int group;   // -1: unused slot
    int begin;   // first pair of the chunk
    int end;     // one past the last pair
    int team;    // see sched_team_word
    __device__ __forceinline__ int first_wave() const { return team & 0xF; }           // slot of the team's first wave
    __device__ __forceinline__ int team_waves() const { return (team >> 4) & 0xF; }
    __device__ __forceinline__ int part() const { return (team >> 8) & 0xFFF; }
    __device__ __forceinline__ int parts() const { return (int)((unsigned)team >> 20); }
};

constexpr int SCHED_MAX_PARTS = 4095;
__host__ __device__ __forceinline__ int sched_team_word(int first_wave, int team_waves, int part, int parts)
{
    return first_wave | (team_waves << 4) | (part << 8) | (int)((unsigned)parts << 20);
}

// Per-group record in front of the slots.
struct SchedGroup {
    int first_slot;    // slot of part 0's first wave
    int tile_slot;     // first partial-tile slot of a split group, else -1
    int split_index;   // ordinal among the split groups, else -1
    int parts;
};

__device__ __forceinline__ int lane_id();

// Up to 64 consecutive pairs of the block table, fetched with ONE vector load (lane t
// keeps pair first + t) and handed out with v_readlane.  A scalar load of blocks[p]
// inside the loop would put a full memory round trip on the critical path of every
// block; this way the walk over a chunk touches the table once.
struct DescWindow {
    int idx, pos, first;
    __device__ __forceinline__ void fetch(const BlockDesc *blocks, int begin, int end)
    {
        first = begin;
        int t = begin + (int)(threadIdx.x & 63u);
        idx = 0;
        pos = 0;
        if (t < end) {
            const BlockDesc d = blocks[t];
            idx = d.idx;
            pos = d.pos;
        }
    }
    // p must be uniform across the wave and inside [first, first + 64)
    __device__ __forceinline__ BlockDesc get(int p) const
    {
        BlockDesc d;
        d.idx = __builtin_amdgcn_readlane(idx, p - first);
        d.pos = __builtin_amdgcn_readlane(pos, p - first);
        return d;
    }
};

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & 63u); }
__device__ __forceinline__ int wave_id() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// Workgroup -> (batch, schedule workgroup).  Hardware deals consecutive
// workgroup ids round-robin to the 8 XCDs, each with its own 4 MB L2; batch b
// is pinned to XCD b % 8 so that its dense operand is fetched into one L2 only.
// The grid holds 8 * n_swg * ceil(batches / 8) workgroups.
__device__ __forceinline__ bool map_workgroup(int n_swg, int batches, int &batch, int &swg)
{
    int w = (int)blockIdx.x;
    int t = w >> 3;
    batch = (w & 7) + 8 * (t / n_swg);
    swg = t % n_swg;
    return batch < batches;
}

// The same grid for kernels without a dense operand (the softmax reads and writes every byte
// once, so there is nothing to keep in an L2): schedule order first, i.e. workgroup s of every
// batch entry is dispatched before workgroup s + 1 of any.  A schedule lists long work first, and
// in batch-major order the long rows of the last batch entries would start near the end of the
// launch and finish on an empty machine.
__device__ __forceinline__ bool map_workgroup_schedule_major(int n_swg, int batches, int &batch, int &swg)
{
    int w = (int)blockIdx.x;
    int t = w >> 3;
    const int nb8 = (batches + 7) >> 3;
    batch = (w & 7) + 8 * (t % nb8);
    swg = t / nb8;
    return batch < batches;
}

// Orders the LDS traffic of ONE wavefront: what its lanes wrote before is
// visible to all its lanes after.  LDS executes a wave's instructions in
// order, so this only has to stop the compiler from moving accesses across.
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---- partial results that workgroups hand to one another through global memory ----------------
// A part of a split group parks its values (park_store), then all its lanes call split_publish();
// the part that finds every other part arrived calls split_consume() and reads the parked values
// (park_load).  Which compute units or L2 slices the parts run on plays no role; what orders the
// accesses is the gfx942 / gfx950 memory model (LLVM AMDGPU backend, "memory model" code sequences):
//   * park_store / park_load are agent-scope monotonic atomic accesses: they carry sc1, so a store
//     writes through to the memory every compute unit of the agent sees and a load does not hit in a
//     cache that is not coherent at agent scope;
//   * split_publish waits until every parked value of the wave has been acknowledged
//     (s_waitcnt vmcnt(0): stores count too) before lane 0 bumps the counter with an agent-scope
//     read-modify-write, which is what a release at agent scope needs after ATOMIC stores (the L2
//     write-back of the full fence only concerns plain stores);
//   * the consumer's loads are issued after the counter value is back (a control dependence on its
//     return value) and are agent-scope atomics themselves, so nothing stale can be served to them.
// BSA_SPLIT_MODE 1 puts full release / acquire fences around the counter instead, 2 also moves the
// parked values with plain accesses; both are equivalent under the model and were measured at twice the
// launch time of the DDS walk (41 against 21 us at 4096 tokens: buffer_wbl2 / buffer_inv per part).
#ifndef BSA_SPLIT_MODE
#define BSA_SPLIT_MODE 0
#endif
#if BSA_SPLIT_MODE == 2
__device__ __forceinline__ void park_store(float *p, float v) { *p = v; }
__device__ __forceinline__ float park_load(const float *p) { return *p; }
#else
__device__ __forceinline__ void park_store(float *p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float park_load(const float *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
#endif
// returns the number of parts that had arrived before this one (uniform across the wave)
__device__ __forceinline__ int split_publish(int *counter)
{
#if BSA_SPLIT_MODE == 0
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#else
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
#endif
    int old = 0;
    if (lane_id() == 0) old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return __builtin_amdgcn_readfirstlane(old);
}
__device__ __forceinline__ void split_consume()
{
#if BSA_SPLIT_MODE != 0
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
#endif
}
__device__ __forceinline__ void split_reset(int *counter)
{
    if (lane_id() == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// ds_read_b64_tr_b16: inside every group of 16 lanes, source lane s hands in
// the address of 4 consecutive halves; result lane i receives, as element e,
// element (i % 4) of source lane 4 * e + i / 4.  With source lane s pointing at
// row s / 4, column chunk s % 4 of a [k][x] tile, result lane 4 * a + c holds
// k = 0..3 of column chunk(a) + c: the MFMA operand layout out of a tile whose
// contraction index is the slow one.
__device__ __forceinline__ h4 lds_read_tr16(const half_t *p)
{
    typedef tr4 __attribute__((address_space(3))) *lds_tr4_ptr;
    tr4 r = __builtin_amdgcn_ds_read_tr16_b64_v4f16((lds_tr4_ptr)(uintptr_t)p);
    return __builtin_bit_cast(h4, r);
}

__device__ __forceinline__ f16v mfma_f16(h8 a, h8 b, f16v c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// 16-bit operands travel as h8 whatever they mean (tiles, LDS maps and requests only see 16-bit
// elements); BF tells the matrix core and the conversions that the bits are bfloat16.
template <bool BF>
__device__ __forceinline__ f16v mfma_16(h8 a, h8 b, f16v c)
{
    if (BF) return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}
// 16 x 16 x 32 products: operand lane (g = lane / 16, i = lane % 16) holds index i, k = 8 g .. 8 g + 7;
// accumulator lane (g, i) holds column i (the second operand's index), rows 4 g + v (the first's).
template <bool BF>
__device__ __forceinline__ f4v mfma_16x16(h8 a, h8 b, f4v c)
{
    if (BF) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, b), c, 0, 0, 0);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
template <bool BF>
__device__ __forceinline__ half_t narrow_16(float x)      // fp32 -> the 16-bit storage type, round to nearest even
{
    if (BF) return __builtin_bit_cast(half_t, (__bf16)x);
    return (half_t)x;
}
template <bool BF>
__device__ __forceinline__ float widen_16(half_t x)
{
    if (BF) return (float)__builtin_bit_cast(__bf16, x);
    return (float)x;
}

__device__ __forceinline__ f16v mfma_f32(float a, float b, f16v c)
{
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ uint4 ldg16(const void *p) { return *reinterpret_cast<const uint4 *>(p); }
__device__ __forceinline__ void stg16(void *p, uint4 v) { *reinterpret_cast<uint4 *>(p) = v; }

// Streaming variants for data that is touched once (sparse blocks, softmax scores, block results):
// the nt hint keeps it from displacing the dense operand tiles that are re-read out of L2.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ldg16_stream(const void *p)
{
    u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stg16_stream(void *p, uint4 v)
{
    u32x4 w = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(w, reinterpret_cast<u32x4 *>(p));
}

__device__ __forceinline__ h8 as_h8(uint4 v) { return __builtin_bit_cast(h8, v); }

// 16 fp32 accumulators -> 16 halves (or bfloat16) in two 16-byte registers.
template <bool BF = false>
__device__ __forceinline__ void pack16(const f16v &acc, uint4 &lo, uint4 &hi)
{
    h8 a, b;
#pragma unroll
    for (int v = 0; v < 8; ++v) {
        a[v] = narrow_16<BF>(acc[v]);
        b[v] = narrow_16<BF>(acc[v + 8]);
    }
    lo = __builtin_bit_cast(uint4, a);
    hi = __builtin_bit_cast(uint4, b);
}

}  // namespace bsa
