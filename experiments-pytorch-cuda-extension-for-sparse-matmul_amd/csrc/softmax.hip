// Block-sparse row softmax, forward and backward, for gfx950.
//
// Replaces sparse_softmax_32x32_forward_kernel / _backward_kernel and their two
// block-wide reductions (sparse_softmax.cu:14-205).  The reference runs a
// 1024-thread workgroup per ELEMENT row and makes three passes over global
// memory; here a team of wavefronts owns a BLOCK row (32 element rows), every
// wave pulls whole 32x32 blocks with 16-byte loads (a block is one or two fully
// coalesced 1 KB requests per wave), keeps its chunk in registers, and the
// data is read once and written once.
//
// Lane map of a block: 16-byte chunk c = lane + 64 * q of the block belongs to
// element row c / LPR, so the LPR = 4 (fp16) or 8 (fp32) lanes of one row are
// neighbours and row reductions are DPP moves (quad_perm, row_half_mirror); only
// the (max, sum) of a row crosses waves, through 512 bytes of LDS per wave.
//
// Additions over the reference: `scale` (folded with log2(e) into one constant
// so the exponential is v_exp_f32 of one fused multiply-add) and the causal
// mask (global column > global row counts as -inf; only blocks on or above the
// diagonal are touched by it).  Chunks longer than the register capacity fall
// back to a two-pass walk (online max/sum, then re-read).
#include "bsa_device.hpp"
#include "bsa_internal.hpp"
#include "../../include/bsa.h"

namespace bsa {

constexpr int SM_MAX_WAVES = 8;
constexpr int SM_STREAM_REGS = 16;  // 16-byte registers a batch of the streaming walks (rows too long for registers) may hold

template <typename T> struct Chunk;
template <> struct Chunk<half_t> {
    static constexpr int NQ = 2;    // 16-byte chunks per lane per block
    static constexpr int EPC = 8;   // elements per chunk
    static constexpr int LPR = 4;   // lanes per element row
    static __device__ __forceinline__ void unpack(const uint4 &r, float (&v)[8])
    {
        h8 h = __builtin_bit_cast(h8, r);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (float)h[i];
    }
    static __device__ __forceinline__ uint4 pack(const float (&v)[8])
    {
        h8 h;
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = (half_t)v[i];
        return __builtin_bit_cast(uint4, h);
    }
    // smallest and largest of the 8 halves, with packed fp16 min / max
    static __device__ __forceinline__ void minmax(const uint4 &r, float &lo, float &hi)
    {
        const h2 a = __builtin_bit_cast(h2, r.x), b = __builtin_bit_cast(h2, r.y);
        const h2 c = __builtin_bit_cast(h2, r.z), d = __builtin_bit_cast(h2, r.w);
        const h2 mx = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
        const h2 mn = __builtin_elementwise_min(__builtin_elementwise_min(a, b), __builtin_elementwise_min(c, d));
        hi = fmaxf((float)mx[0], (float)mx[1]);
        lo = fminf((float)mn[0], (float)mn[1]);
    }
    // every element times f, in fp32 and rounded once.  Written as a fused multiply-add with a zero
    // addend, this becomes one v_fma_mixlo / mixhi_f16 per element (widen, multiply and narrow in
    // one instruction) instead of two conversions, a multiply and half a packing conversion.
    static __device__ __forceinline__ uint4 scaled(const uint4 &r, float f)
    {
        h8 h = __builtin_bit_cast(h8, r);
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = (half_t)__builtin_fmaf((float)h[i], f, 0.f);
        return __builtin_bit_cast(uint4, h);
    }
    // element i := `fill` where col0 + i > limit
    static __device__ __forceinline__ void mask_right_of(uint4 &r, int col0, int limit, float fill)
    {
        h8 h = __builtin_bit_cast(h8, r);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (col0 + i > limit) h[i] = (half_t)fill;
        r = __builtin_bit_cast(uint4, h);
    }
};
// bfloat16: the same 16-byte chunks as fp16; a value widens by a 16-bit shift and narrows with
// v_cvt_pk_bf16_f32 (round to nearest even).  No packed min / max for this type.
struct bf16_t { unsigned short bits; };
template <> struct Chunk<bf16_t> {
    static constexpr int NQ = 2;
    static constexpr int EPC = 8;
    static constexpr int LPR = 4;
    static __device__ __forceinline__ void unpack(const uint4 &r, float (&v)[8])
    {
        const unsigned w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = __uint_as_float(w[i] << 16);
            v[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
        }
    }
    static __device__ __forceinline__ uint4 pack(const float (&v)[8])
    {
        bf8 h;
#pragma unroll
        for (int i = 0; i < 8; ++i) h[i] = (__bf16)v[i];
        return __builtin_bit_cast(uint4, h);
    }
    static __device__ __forceinline__ void minmax(const uint4 &r, float &lo, float &hi)
    {
        float v[8];
        unpack(r, v);
        hi = fmaxf(fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3])), fmaxf(fmaxf(v[4], v[5]), fmaxf(v[6], v[7])));
        lo = fminf(fminf(fminf(v[0], v[1]), fminf(v[2], v[3])), fminf(fminf(v[4], v[5]), fminf(v[6], v[7])));
    }
    static __device__ __forceinline__ uint4 scaled(const uint4 &r, float f)
    {
        float v[8];
        unpack(r, v);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] *= f;
        return pack(v);
    }
    static __device__ __forceinline__ void mask_right_of(uint4 &r, int col0, int limit, float fill)
    {
        float v[8];
        unpack(r, v);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (col0 + i > limit) v[i] = fill;
        r = pack(v);
    }
};
template <> struct Chunk<float> {
    static constexpr int NQ = 4;
    static constexpr int EPC = 4;
    static constexpr int LPR = 8;
    static __device__ __forceinline__ void unpack(const uint4 &r, float (&v)[4])
    {
        v[0] = __uint_as_float(r.x); v[1] = __uint_as_float(r.y);
        v[2] = __uint_as_float(r.z); v[3] = __uint_as_float(r.w);
    }
    static __device__ __forceinline__ uint4 pack(const float (&v)[4])
    {
        return make_uint4(__float_as_uint(v[0]), __float_as_uint(v[1]),
                          __float_as_uint(v[2]), __float_as_uint(v[3]));
    }
    static __device__ __forceinline__ void minmax(const uint4 &r, float &lo, float &hi)
    {
        float v[4];
        unpack(r, v);
        hi = fmaxf(fmaxf(v[0], v[1]), fmaxf(v[2], v[3]));
        lo = fminf(fminf(v[0], v[1]), fminf(v[2], v[3]));
    }
    static __device__ __forceinline__ uint4 scaled(const uint4 &r, float f)
    {
        float v[4];
        unpack(r, v);
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] *= f;
        return pack(v);
    }
    static __device__ __forceinline__ void mask_right_of(uint4 &r, int col0, int limit, float fill)
    {
        float v[4];
        unpack(r, v);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (col0 + i > limit) v[i] = fill;
        r = pack(v);
    }
};

// value of the neighbour lane selected by a DPP control word
template <int CTRL>
__device__ __forceinline__ float dpp(float x)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, true));
}

// all-reduce over the LPR neighbouring lanes that hold one element row
template <int LPR, typename Op>
__device__ __forceinline__ float row_allreduce(float x, Op op)
{
    x = op(x, dpp<0xB1>(x));    // quad_perm [1,0,3,2]
    x = op(x, dpp<0x4E>(x));    // quad_perm [2,3,0,1]
    if (LPR == 8) x = op(x, dpp<0x141>(x));   // row_half_mirror: lane i <- lane 7 - i
    return x;
}

struct MaxOp { __device__ __forceinline__ float operator()(float a, float b) const { return fmaxf(a, b); } };
struct AddOp { __device__ __forceinline__ float operator()(float a, float b) const { return a + b; } };

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

// scaled scores of one 16-byte chunk that starts at (row, col0) of block column bcol of block row
// `group`; with `causal`, columns right of the diagonal count as -inf
template <typename T>
__device__ __forceinline__ void scaled_chunk(const uint4 &raw, int row, int col0, int bcol, int group,
                                             float scale2, int causal, float (&v)[Chunk<T>::EPC])
{
    constexpr int EPC = Chunk<T>::EPC;
    Chunk<T>::unpack(raw, v);
#pragma unroll
    for (int i = 0; i < EPC; ++i) v[i] *= scale2;
    if (causal && bcol >= group) {
        const int limit = (bcol > group) ? -1 : row;   // last visible column inside the block
#pragma unroll
        for (int i = 0; i < EPC; ++i)
            if (col0 + i > limit) v[i] = -__builtin_inff();
    }
}

// Register-resident chunks: the causal mask is burnt into the packed data once (only blocks on or
// right of the diagonal are touched, under a wave-uniform branch), the row max comes from packed
// min / max of the raw scores, and the exponential is exp2(fma(x, scale2, -max)).
template <typename T>
__device__ __forceinline__ void mask_chunk(uint4 &raw, int row, int col0, int bcol, int group, float scale2)
{
    if (bcol >= group) {
        const float fill = scale2 < 0.f ? __builtin_inff() : -__builtin_inff();   // -inf once scaled
        Chunk<T>::mask_right_of(raw, col0, bcol > group ? -1 : row, fill);
    }
}

template <typename T>
__device__ __forceinline__ float chunk_scaled_max(const uint4 &raw, float scale2)
{
    float lo, hi;
    Chunk<T>::minmax(raw, lo, hi);
    return fmaxf(lo * scale2, hi * scale2);
}

// v[i] = exp2(scale2 * x[i] - m); returns their sum
template <typename T>
__device__ __forceinline__ float chunk_exp(const uint4 &raw, float scale2, float m, float (&v)[Chunk<T>::EPC])
{
    Chunk<T>::unpack(raw, v);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < Chunk<T>::EPC; ++i) {
        v[i] = exp2_fast(__builtin_fmaf(v[i], scale2, -m));
        sum += v[i];
    }
    return sum;
}

// Pins a value to its four packed registers: without it the compiler forwards the unpacked floats
// of one pass over a register-resident slice to the next pass and keeps all of them alive (2-4x the
// registers of the slice itself).
__device__ __forceinline__ void launder(uint4 &r)
{
    asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
}

__device__ __forceinline__ float finite_or_zero(float m) { return m == -__builtin_inff() ? 0.f : m; }

// ---------------------------------------------------------------------------
// Row-sliced walk: a block row of at most CBS blocks goes whole to SLICES wavefronts,
// each owning 32 / SLICES of the 32 element rows, which it cuts into SUBS sub-slices of
// R = 32 / SLICES / SUBS element rows.  A sub-slice of one block is R * LPR lanes wide, so one
// load instruction covers BPI = 64 / (R * LPR) consecutive blocks of the row.  The
// wave issues every load of its slice at once, sub-slice by sub-slice, and then
// finishes the sub-slices one after the other: while it computes and stores
// sub-slice t the data of sub-slice t + 1 is still arriving, so loads, math and
// stores overlap although all waves of the launch run in lockstep.  No LDS
// storage and no barrier: a row lives in LPR neighbouring lanes of BPI lane groups.
// The code is specialised on the number of load instructions per sub-slice, which
// keeps every load unconditional (the wait counts the compiler derives are exact).
// ---------------------------------------------------------------------------
#ifndef BSA_SM_SUBS
#define BSA_SM_SUBS 2
#endif
constexpr int SM_SUBS = BSA_SM_SUBS;
#ifndef BSA_SM_FWD_SLICES
#define BSA_SM_FWD_SLICES 4
#endif
constexpr int SM_FWD_SLICES = BSA_SM_FWD_SLICES;   // slices the register-resident walks are compiled for
constexpr int SM_BWD_SLICES = 4;
// fp32 rows take twice the registers per block: eight slices keep rows of up to 24 blocks resident in the
// backward walk (two inputs), like four slices do for the 16-bit types
template <typename T> constexpr int sm_bwd_slices() { return sizeof(T) == 4 ? 8 : SM_BWD_SLICES; }

template <int MASK>
__device__ __forceinline__ float lane_xor(float x)
{
    return __int_as_float(__builtin_amdgcn_ds_bpermute((lane_id() ^ MASK) << 2, __float_as_int(x)));
}

// all-reduce over the lanes that hold one element row of a sub-slice
template <int LPR, int BPI, typename Op>
__device__ __forceinline__ float slice_allreduce(float x, Op op)
{
    x = row_allreduce<LPR>(x, op);
    if (BPI >= 2) x = op(x, lane_xor<32>(x));
    if (BPI >= 4) x = op(x, lane_xor<16>(x));
    return x;
}

template <typename T, int SLICES, int SUBS>
struct SliceMap {
    typedef Chunk<T> C;
    static constexpr int R = BS / SLICES / SUBS;              // element rows of a sub-slice
    static constexpr int LPB = R * C::LPR;                    // lanes on one block's part of a sub-slice
    static constexpr int BPI = WAVE / LPB;                    // blocks per load instruction
    static constexpr int SUB_STRIDE = R * BS;                 // elements between sub-slices inside a block
    static_assert(LPB <= WAVE && BPI <= 4, "sub-slice geometry");
    int seg, row0, col0, lane_off;
    __device__ __forceinline__ SliceMap(int slice)
    {
        const int l = lane_id();
        seg = l / LPB;
        row0 = (BS / SLICES) * slice + (l % LPB) / C::LPR;      // + R * t
        col0 = C::EPC * (l % C::LPR);
        lane_off = (BS2 / SLICES) * slice + (l % LPB) * C::EPC;  // + SUB_STRIDE * t, inside a block
    }
};

template <typename T, int SLICES, int SUBS, int NI>
__device__ __forceinline__ void softmax_fwd_sliced_body(const T *__restrict__ xb, T *__restrict__ yb,
                                                        const DescWindow &win, const SchedEntry &e,
                                                        float scale2, int causal)
{
    typedef Chunk<T> C;
    typedef SliceMap<T, SLICES, SUBS> Map;
    constexpr int EPC = C::EPC, LPR = C::LPR, BPI = Map::BPI;
    const Map map(e.part());
    const int n = e.end - e.begin;
    const float NEG_INF = -__builtin_inff();

    // The table is row-major and idx is the row-major ordinal of a block, so pair p of the table
    // IS block p of the operand and the blocks of a row lie one after the other in memory: the
    // loads need nothing from the table (only the causal mask reads the block columns, which
    // arrive while the data is in flight).  Lane's block of load instruction i is i * BPI + seg;
    // lanes past the end of the row (last instruction only) load the last block instead, are
    // masked out of the reductions and do not store.
    const size_t row_off = (size_t)e.begin * BS2;
    const T *xrow = xb + row_off;
    T *yrow = yb + row_off;
    const unsigned off = (unsigned)(map.seg * BS2 + map.lane_off);                        // + (i * BPI) * BS2 + t * SUB_STRIDE
    const unsigned off_last = (unsigned)(min((NI - 1) * BPI + map.seg, n - 1) * BS2 + map.lane_off);
    auto chunk_off = [&](int t, int i) {
        return (i == NI - 1 ? off_last : off + (unsigned)(i * BPI * BS2)) + (unsigned)(t * Map::SUB_STRIDE);
    };
    uint4 raw[SUBS][NI];
#pragma unroll
    for (int t = 0; t < SUBS; ++t) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
            raw[t][i] = ldg16_stream(xrow + chunk_off(t, i));
        __builtin_amdgcn_sched_barrier(0);   // sub-slice t is requested in full before t + 1: it is needed first
    }
    __builtin_amdgcn_sched_barrier(0);

#pragma unroll
    for (int t = 0; t < SUBS; ++t) {
        const int row = map.row0 + t * Map::R;
        float m = NEG_INF, s = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const bool tail = i == NI - 1 && n < NI * BPI;
            const int last_col = win.get(e.begin + min(i * BPI + BPI - 1, n - 1)).col();
            if (tail || (causal && last_col >= e.group)) {     // wave-uniform
                const int j = i * BPI + map.seg;
                const int pos = BPI == 1 ? win.get(e.begin + min(j, n - 1)).pos
                                         : __builtin_amdgcn_ds_bpermute(min(j, n - 1) << 2, win.pos);
                const int bcol = pos & 0xFFFF;
                int limit = BS;                                 // last visible column inside the block
                if (causal && bcol >= e.group) limit = bcol > e.group ? -1 : row;
                if (j >= n) limit = -1;
                const float fill = scale2 < 0.f ? __builtin_inff() : NEG_INF;   // -inf once scaled
                C::mask_right_of(raw[t][i], map.col0, limit, fill);
            }
            m = fmaxf(m, chunk_scaled_max<T>(raw[t][i], scale2));
        }
        m = finite_or_zero(slice_allreduce<LPR, BPI>(m, MaxOp()));
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            float v[EPC];
            s += chunk_exp<T>(raw[t][i], scale2, m, v);
            raw[t][i] = C::pack(v);
            launder(raw[t][i]);                  // park the exponentials PACKED: the compiler would keep 8 floats
            __builtin_amdgcn_sched_barrier(0);   // one chunk at a time: unpacking them all at once spills
        }
        s = slice_allreduce<LPR, BPI>(s, AddOp());
        s = s > 0.f ? 1.f / s : 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const bool mine = i < NI - 1 || i * BPI + map.seg < n;
            if (mine) stg16_stream(yrow + chunk_off(t, i), C::scaled(raw[t][i], s));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// Lane map of whole blocks with a row filter, for sliced rows that the register-resident walk
// does not take (longer than its capacity, or cut into another number of slices): chunk q of a
// lane belongs to the wave when its element row lies in the wave's slice.
template <typename T>
struct SliceFilter {
    typedef Chunk<T> C;
    static constexpr int ROWS_PER_Q = WAVE / C::LPR;
    int row0, col0, lo, hi;
    __device__ __forceinline__ SliceFilter(const SchedEntry &e)
    {
        const int l = lane_id(), rows = BS / e.parts();
        row0 = l / C::LPR;
        col0 = C::EPC * (l % C::LPR);
        lo = rows * e.part();
        hi = lo + rows;
    }
    __device__ __forceinline__ int row(int q) const { return row0 + q * ROWS_PER_Q; }
    __device__ __forceinline__ bool mine(int q) const { return row(q) >= lo && row(q) < hi; }
};

template <typename T, int CBS, int SLICES>
__device__ __forceinline__ void softmax_fwd_sliced(const T *__restrict__ xb, T *__restrict__ yb,
                                                   const BlockDesc *__restrict__ blocks, const SchedEntry &e,
                                                   float scale2, int causal)
{
    typedef Chunk<T> C;
    constexpr int NQ = C::NQ, EPC = C::EPC, LPR = C::LPR;
    constexpr int BPI = SliceMap<T, SLICES, SM_SUBS>::BPI, NI_MAX = (CBS + BPI - 1) / BPI;
    static_assert(NI_MAX <= 12, "add cases to the switch below");
    const int l = lane_id();
    const int n = e.end - e.begin;
    DescWindow win;
    win.fetch(blocks, e.begin, e.end);

    if (e.parts() == SLICES && n <= CBS) {
#define BSA_SM_CASE(K) \
    case K: if constexpr (K <= NI_MAX) softmax_fwd_sliced_body<T, SLICES, SM_SUBS, K>(xb, yb, win, e, scale2, causal); break;
        switch ((n + BPI - 1) / BPI) {
            BSA_SM_CASE(1) BSA_SM_CASE(2) BSA_SM_CASE(3) BSA_SM_CASE(4) BSA_SM_CASE(5) BSA_SM_CASE(6)
            BSA_SM_CASE(7) BSA_SM_CASE(8) BSA_SM_CASE(9) BSA_SM_CASE(10) BSA_SM_CASE(11) BSA_SM_CASE(12)
            default: break;    // an empty row: nothing to write
        }
#undef BSA_SM_CASE
        return;
    }

    // two passes over global memory: online (max, sum), then normalise
    const SliceFilter<T> f(e);
    const float NEG_INF = -__builtin_inff();
    float m[NQ], s[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) { m[q] = NEG_INF; s[q] = 0.f; }
    for (int p = e.begin; p < e.end; ++p) {
        if (p > e.begin && ((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const BlockDesc d = win.get(p);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            if (!f.mine(q)) continue;
            float v[EPC];
            scaled_chunk<T>(ldg16_stream(xb + (size_t)d.idx * BS2 + (l + WAVE * q) * EPC),
                            f.row(q), f.col0, d.col(), e.group, scale2, causal, v);
            float bm = v[0];
#pragma unroll
            for (int i = 1; i < EPC; ++i) bm = fmaxf(bm, v[i]);
            const float nm = fmaxf(m[q], bm);
            const float mm = finite_or_zero(nm);
            float acc = s[q] * exp2_fast(m[q] - mm);
#pragma unroll
            for (int i = 0; i < EPC; ++i) acc += exp2_fast(v[i] - mm);
            s[q] = acc;
            m[q] = nm;
        }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {      // all lanes take part in the exchange; rows of other slices carry (-inf, 0)
        const float rm = finite_or_zero(row_allreduce<LPR>(m[q], MaxOp()));
        s[q] = row_allreduce<LPR>(s[q] * exp2_fast(m[q] - rm), AddOp());
        s[q] = s[q] > 0.f ? 1.f / s[q] : 0.f;
        m[q] = rm;
    }
    for (int p = e.begin; p < e.end; ++p) {
        if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const BlockDesc d = win.get(p);
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            if (!f.mine(q)) continue;
            float v[EPC];
            scaled_chunk<T>(ldg16_stream(xb + (size_t)d.idx * BS2 + (l + WAVE * q) * EPC),
                            f.row(q), f.col0, d.col(), e.group, scale2, causal, v);
#pragma unroll
            for (int i = 0; i < EPC; ++i) v[i] = exp2_fast(v[i] - m[q]) * s[q];
            stg16_stream(yb + (size_t)d.idx * BS2 + (l + WAVE * q) * EPC, C::pack(v));
        }
    }
}

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename T, int CB, int CBS>
__global__ __launch_bounds__(64 * SM_MAX_WAVES) __attribute__((amdgpu_waves_per_eu(4))) void softmax_fwd_kernel(
    const T *__restrict__ x, T *__restrict__ y, const BlockDesc *__restrict__ blocks,
    const SchedEntry *__restrict__ sched, int n_swg, int batches, int nnz,
    float scale2 /* scale * log2(e) */, int causal)
{
    typedef Chunk<T> C;
    constexpr int NQ = C::NQ, EPC = C::EPC, LPR = C::LPR;
    constexpr int ROWS_PER_Q = WAVE / LPR;
    constexpr int SM_STREAM = SM_STREAM_REGS / NQ;            // blocks per batch: 8 (16-bit types) or 4; divides 64
    __shared__ float2 stats[SM_MAX_WAVES][BS];

    int batch, swg;
    if (!map_workgroup_schedule_major(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const bool active = e.group >= 0;
    const int n = active ? e.end - e.begin : 0;
    const T *xb = x + (size_t)batch * nnz * BS2;
    T *yb = y + (size_t)batch * nnz * BS2;

    // Row-sliced waves fill workgroups of their own (the schedule builder sees to that), so this
    // branch is uniform over the workgroup and the barrier below is never left waiting.
    if (active && e.parts() > 1) {
        softmax_fwd_sliced<T, CBS, SM_FWD_SLICES>(xb, yb, blocks, e, scale2, causal);
        return;
    }
    if (sched[swg * W].parts() > 1) return;   // an unused slot behind the last row-sliced waves

    const int col0 = EPC * (l % LPR);          // first column of this lane's chunk inside a block
    const int row0 = l / LPR;                  // element row of chunk q is row0 + q * ROWS_PER_Q
    const float NEG_INF = -__builtin_inff();

    float m[NQ], s[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) { m[q] = NEG_INF; s[q] = 0.f; }

    uint4 raw[CB][NQ];
    int bidx[CB], bcol[CB];
    const bool resident = n <= CB;

    DescWindow win;
    if (active) win.fetch(blocks, e.begin, e.end);
    if (resident) {
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j < n) {
                const BlockDesc d = win.get(e.begin + j);
                bidx[j] = d.idx; bcol[j] = d.col();
                const T *src = xb + (size_t)d.idx * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) raw[j][q] = ldg16_stream(src + (l + WAVE * q) * EPC);
            }
        }
        // pass 1 (registers): causal mask burnt in, row max
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j < n) {
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    if (causal) mask_chunk<T>(raw[j][q], row0 + q * ROWS_PER_Q, col0, bcol[j], e.group, scale2);
                    m[q] = fmaxf(m[q], chunk_scaled_max<T>(raw[j][q], scale2));
                }
            }
        }
#pragma unroll
        for (int q = 0; q < NQ; ++q) m[q] = row_allreduce<LPR>(m[q], MaxOp());
        // pass 2 (registers): exponentials in place, row sum
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j < n) {
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    float v[EPC];
                    s[q] += chunk_exp<T>(raw[j][q], scale2, finite_or_zero(m[q]), v);
                    raw[j][q] = C::pack(v);
                }
            }
        }
    } else if (active) {
        // Streaming pass 1: online max / sum, SM_STREAM blocks at a time.  All loads of a batch go out
        // before the first block is touched (one memory latency per batch instead of one per block;
        // a batch past the end of the chunk reloads the last block, so no load sits under a condition).
        for (int p0 = e.begin; p0 < e.end; p0 += SM_STREAM) {
            if (p0 > e.begin && ((p0 - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p0, e.end);
            uint4 rs[SM_STREAM][NQ];
            int cs[SM_STREAM];
#pragma unroll
            for (int j = 0; j < SM_STREAM; ++j) {
                const BlockDesc d = win.get(p0 + j < e.end ? p0 + j : e.end - 1);
                cs[j] = d.col();
                const T *src = xb + (size_t)d.idx * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) rs[j][q] = ldg16_stream(src + (l + WAVE * q) * EPC);
            }
#pragma unroll
            for (int j = 0; j < SM_STREAM; ++j) {
                if (p0 + j >= e.end) break;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    float v[EPC];
                    scaled_chunk<T>(rs[j][q], row0 + q * ROWS_PER_Q, col0, cs[j], e.group, scale2, causal, v);
                    float bm = v[0];
#pragma unroll
                    for (int i = 1; i < EPC; ++i) bm = fmaxf(bm, v[i]);
                    const float nm = fmaxf(m[q], bm);
                    const float mm = finite_or_zero(nm);
                    float acc = s[q] * exp2_fast(m[q] - mm);
#pragma unroll
                    for (int i = 0; i < EPC; ++i) acc += exp2_fast(v[i] - mm);
                    s[q] = acc;
                    m[q] = nm;
                }
            }
        }
        // lanes of a row hold different (m, s): bring them to the row max
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            const float rm = row_allreduce<LPR>(m[q], MaxOp());
            s[q] *= exp2_fast(m[q] - finite_or_zero(rm));
            m[q] = rm;
        }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) s[q] = row_allreduce<LPR>(s[q], AddOp());

    // team exchange of (max, sum) per element row
    const int slot0 = e.first_wave(), nw = e.team_waves();
    if (active && (l % LPR) == 0) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) stats[w][row0 + q * ROWS_PER_Q] = make_float2(m[q], s[q]);
    }
    __syncthreads();
    if (!active) return;

    float f[NQ], gm[NQ], inv_s[NQ];   // factor for this wave's exponentials; row max; 1 / row sum
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
        float M = m[q], S = s[q];
        if (nw > 1) {
            M = NEG_INF;
            for (int t = 0; t < nw; ++t) M = fmaxf(M, stats[slot0 + t][row0 + q * ROWS_PER_Q].x);
            const float MM = finite_or_zero(M);
            S = 0.f;
            for (int t = 0; t < nw; ++t) {
                const float2 st = stats[slot0 + t][row0 + q * ROWS_PER_Q];
                S += st.y * exp2_fast(st.x - MM);
            }
        }
        const float MM = finite_or_zero(M);
        const float inv = S > 0.f ? 1.f / S : 0.f;
        gm[q] = MM;
        inv_s[q] = inv;
        f[q] = (m[q] == NEG_INF) ? 0.f : exp2_fast(m[q] - MM) * inv;
    }

    if (resident) {
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j < n) {
                T *dst = yb + (size_t)bidx[j] * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    float v[EPC];
                    C::unpack(raw[j][q], v);
#pragma unroll
                    for (int i = 0; i < EPC; ++i) v[i] *= f[q];
                    stg16_stream(dst + (l + WAVE * q) * EPC, C::pack(v));
                }
            }
        }
    } else {
        // streaming pass 2: re-read, normalise, write, in the same batches
        for (int p0 = e.begin; p0 < e.end; p0 += SM_STREAM) {
            if (((p0 - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p0, e.end);
            uint4 rs[SM_STREAM][NQ];
            int cs[SM_STREAM], is[SM_STREAM];
#pragma unroll
            for (int j = 0; j < SM_STREAM; ++j) {
                const BlockDesc d = win.get(p0 + j < e.end ? p0 + j : e.end - 1);
                cs[j] = d.col();
                is[j] = d.idx;
                const T *src = xb + (size_t)d.idx * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) rs[j][q] = ldg16_stream(src + (l + WAVE * q) * EPC);
            }
#pragma unroll
            for (int j = 0; j < SM_STREAM; ++j) {
                if (p0 + j >= e.end) break;
                T *dst = yb + (size_t)is[j] * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    float v[EPC];
                    scaled_chunk<T>(rs[j][q], row0 + q * ROWS_PER_Q, col0, cs[j], e.group, scale2, causal, v);
#pragma unroll
                    for (int i = 0; i < EPC; ++i) v[i] = exp2_fast(v[i] - gm[q]) * inv_s[q];
                    stg16_stream(dst + (l + WAVE * q) * EPC, C::pack(v));
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// backward: dx = scale * (dy - sum_row(dy * y)) * y
// ---------------------------------------------------------------------------
// Row-sliced backward: the same sub-slice pipeline as the forward walk, over two inputs.
template <typename T, int SLICES, int SUBS, int NI>
__device__ __forceinline__ void softmax_bwd_sliced_body(const T *__restrict__ y, const T *__restrict__ dy,
                                                        T *__restrict__ dx, const SchedEntry &e, float scale)
{
    typedef Chunk<T> C;
    typedef SliceMap<T, SLICES, SUBS> Map;
    constexpr int EPC = C::EPC, LPR = C::LPR, BPI = Map::BPI;
    const Map map(e.part());
    const int n = e.end - e.begin;
    const size_t row_off = (size_t)e.begin * BS2;     // pair p of the row-major table is block p of the operand
    const unsigned off = (unsigned)(map.seg * BS2 + map.lane_off);
    const unsigned off_last = (unsigned)(min((NI - 1) * BPI + map.seg, n - 1) * BS2 + map.lane_off);
    auto chunk_off = [&](int t, int i) {
        return (i == NI - 1 ? off_last : off + (unsigned)(i * BPI * BS2)) + (unsigned)(t * Map::SUB_STRIDE);
    };
    const bool mine_last = (NI - 1) * BPI + map.seg < n;   // lanes past the row's end load its last block again

    uint4 ry[SUBS][NI], rd[SUBS][NI];
#pragma unroll
    for (int t = 0; t < SUBS; ++t) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            ry[t][i] = ldg16_stream(y + row_off + chunk_off(t, i));
            rd[t][i] = ldg16_stream(dy + row_off + chunk_off(t, i));
        }
        __builtin_amdgcn_sched_barrier(0);   // sub-slice t is requested in full before t + 1: it is needed first
    }
#pragma unroll
    for (int t = 0; t < SUBS; ++t) {
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            float a[EPC], b[EPC], part = 0.f;
            C::unpack(ry[t][i], a);
            C::unpack(rd[t][i], b);
#pragma unroll
            for (int k = 0; k < EPC; ++k) part += a[k] * b[k];
            dot += (i < NI - 1 || mine_last) ? part : 0.f;
        }
        dot = slice_allreduce<LPR, BPI>(dot, AddOp());
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            float a[EPC], b[EPC];
            launder(ry[t][i]);                // unpack again: the floats of the first pass are not kept
            launder(rd[t][i]);
            C::unpack(ry[t][i], a);
            C::unpack(rd[t][i], b);
#pragma unroll
            for (int k = 0; k < EPC; ++k) a[k] = scale * (b[k] - dot) * a[k];
            if (i < NI - 1 || mine_last) stg16_stream(dx + row_off + chunk_off(t, i), C::pack(a));
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

template <typename T, int CBS, int SLICES>
__device__ __forceinline__ void softmax_bwd_sliced(const T *__restrict__ y, const T *__restrict__ dy,
                                                   T *__restrict__ dx, const BlockDesc *__restrict__ blocks,
                                                   const SchedEntry &e, float scale)
{
    typedef Chunk<T> C;
    constexpr int NQ = C::NQ, EPC = C::EPC, LPR = C::LPR;
    constexpr int BPI = SliceMap<T, SLICES, SM_SUBS>::BPI, NI_MAX = (CBS + BPI - 1) / BPI;
    static_assert(NI_MAX <= 6, "add cases to the switch below");
    const int l = lane_id();
    const int n = e.end - e.begin;
    if (e.parts() == SLICES && n <= CBS) {
#define BSA_SM_CASE(K) \
    case K: if constexpr (K <= NI_MAX) softmax_bwd_sliced_body<T, SLICES, SM_SUBS, K>(y, dy, dx, e, scale); break;
        switch ((n + BPI - 1) / BPI) {
            BSA_SM_CASE(1) BSA_SM_CASE(2) BSA_SM_CASE(3) BSA_SM_CASE(4) BSA_SM_CASE(5) BSA_SM_CASE(6)
            default: break;    // an empty row: nothing to write
        }
#undef BSA_SM_CASE
        return;
    }

    // two passes over global memory (see SliceFilter)
    const SliceFilter<T> f(e);
    float dot[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) dot[q] = 0.f;
    DescWindow win;
    for (int p = e.begin; p < e.end; ++p) {
        if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const size_t o = (size_t)win.get(p).idx * BS2;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            if (!f.mine(q)) continue;
            float a[EPC], b[EPC];
            C::unpack(ldg16_stream(y + o + (l + WAVE * q) * EPC), a);
            C::unpack(ldg16_stream(dy + o + (l + WAVE * q) * EPC), b);
#pragma unroll
            for (int i = 0; i < EPC; ++i) dot[q] += a[i] * b[i];
        }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) dot[q] = row_allreduce<LPR>(dot[q], AddOp());
    for (int p = e.begin; p < e.end; ++p) {
        if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const size_t o = (size_t)win.get(p).idx * BS2;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            if (!f.mine(q)) continue;
            float a[EPC], b[EPC];
            C::unpack(ldg16_stream(y + o + (l + WAVE * q) * EPC), a);
            C::unpack(ldg16_stream(dy + o + (l + WAVE * q) * EPC), b);
#pragma unroll
            for (int i = 0; i < EPC; ++i) a[i] = scale * (b[i] - dot[q]) * a[i];
            stg16_stream(dx + o + (l + WAVE * q) * EPC, C::pack(a));
        }
    }
}

template <typename T, int CB, int CBS>
__global__ __launch_bounds__(64 * SM_MAX_WAVES) __attribute__((amdgpu_waves_per_eu(4))) void softmax_bwd_kernel(
    const T *__restrict__ y, const T *__restrict__ dy, T *__restrict__ dx,
    const BlockDesc *__restrict__ blocks, const SchedEntry *__restrict__ sched,
    int n_swg, int batches, int nnz, float scale)
{
    typedef Chunk<T> C;
    constexpr int NQ = C::NQ, EPC = C::EPC, LPR = C::LPR;
    constexpr int ROWS_PER_Q = WAVE / LPR;
    constexpr int SM_STREAM_BWD = SM_STREAM_REGS / (2 * NQ);  // two operands per block: 4 or 2 blocks per batch
    __shared__ float dots[SM_MAX_WAVES][BS];

    int batch, swg;
    if (!map_workgroup_schedule_major(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const bool active = e.group >= 0;
    const int n = active ? e.end - e.begin : 0;
    const size_t boff = (size_t)batch * nnz * BS2;
    const int row0 = l / LPR;

    if (active && e.parts() > 1) {   // row-sliced waves sit in workgroups of their own
        softmax_bwd_sliced<T, CBS, sm_bwd_slices<T>()>(y + boff, dy + boff, dx + boff, blocks, e, scale);
        return;
    }
    if (sched[swg * W].parts() > 1) return;

    float dot[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) dot[q] = 0.f;

    uint4 ry[CB][NQ], rd[CB][NQ];
    int bidx[CB];
    const bool resident = n <= CB;
    DescWindow win;
    if (active) win.fetch(blocks, e.begin, e.end);
    if (resident) {
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j < n) {
                bidx[j] = win.get(e.begin + j).idx;
                const size_t o = boff + (size_t)bidx[j] * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    ry[j][q] = ldg16_stream(y + o + (l + WAVE * q) * EPC);
                    rd[j][q] = ldg16_stream(dy + o + (l + WAVE * q) * EPC);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j < n) {
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    float a[EPC], b[EPC];
                    C::unpack(ry[j][q], a);
                    C::unpack(rd[j][q], b);
#pragma unroll
                    for (int i = 0; i < EPC; ++i) dot[q] += a[i] * b[i];
                }
            }
        }
    } else if (active) {
        // streaming, SM_STREAM_BWD blocks at a time: all loads of a batch go out before the first use
        for (int p0 = e.begin; p0 < e.end; p0 += SM_STREAM_BWD) {
            if (p0 > e.begin && ((p0 - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p0, e.end);
            uint4 sy[SM_STREAM_BWD][NQ], sd[SM_STREAM_BWD][NQ];
#pragma unroll
            for (int j = 0; j < SM_STREAM_BWD; ++j) {
                const size_t o = boff + (size_t)win.get(p0 + j < e.end ? p0 + j : e.end - 1).idx * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    sy[j][q] = ldg16_stream(y + o + (l + WAVE * q) * EPC);
                    sd[j][q] = ldg16_stream(dy + o + (l + WAVE * q) * EPC);
                }
            }
#pragma unroll
            for (int j = 0; j < SM_STREAM_BWD; ++j) {
                if (p0 + j >= e.end) break;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    float a[EPC], b[EPC];
                    C::unpack(sy[j][q], a);
                    C::unpack(sd[j][q], b);
#pragma unroll
                    for (int i = 0; i < EPC; ++i) dot[q] += a[i] * b[i];
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) dot[q] = row_allreduce<LPR>(dot[q], AddOp());

    const int slot0 = e.first_wave(), nw = e.team_waves();
    if (active && (l % LPR) == 0) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) dots[w][row0 + q * ROWS_PER_Q] = dot[q];
    }
    __syncthreads();
    if (!active) return;
    if (nw > 1) {
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
            float t = 0.f;
            for (int o = 0; o < nw; ++o) t += dots[slot0 + o][row0 + q * ROWS_PER_Q];
            dot[q] = t;
        }
    }

    auto finish = [&](const uint4 &uy, const uint4 &ud, int q) {
        float a[EPC], b[EPC];
        C::unpack(uy, a);
        C::unpack(ud, b);
#pragma unroll
        for (int i = 0; i < EPC; ++i) a[i] = scale * (b[i] - dot[q]) * a[i];
        return C::pack(a);
    };
    if (resident) {
#pragma unroll
        for (int j = 0; j < CB; ++j) {
            if (j < n) {
                const size_t o = boff + (size_t)bidx[j] * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) stg16_stream(dx + o + (l + WAVE * q) * EPC, finish(ry[j][q], rd[j][q], q));
            }
        }
    } else {
        for (int p0 = e.begin; p0 < e.end; p0 += SM_STREAM_BWD) {
            if (((p0 - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p0, e.end);
            uint4 sy[SM_STREAM_BWD][NQ], sd[SM_STREAM_BWD][NQ];
            size_t os[SM_STREAM_BWD];
#pragma unroll
            for (int j = 0; j < SM_STREAM_BWD; ++j) {
                os[j] = boff + (size_t)win.get(p0 + j < e.end ? p0 + j : e.end - 1).idx * BS2;
#pragma unroll
                for (int q = 0; q < NQ; ++q) {
                    sy[j][q] = ldg16_stream(y + os[j] + (l + WAVE * q) * EPC);
                    sd[j][q] = ldg16_stream(dy + os[j] + (l + WAVE * q) * EPC);
                }
            }
#pragma unroll
            for (int j = 0; j < SM_STREAM_BWD; ++j) {
                if (p0 + j >= e.end) break;
#pragma unroll
                for (int q = 0; q < NQ; ++q) stg16_stream(dx + os[j] + (l + WAVE * q) * EPC, finish(sy[j][q], sd[j][q], q));
            }
        }
    }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
static inline unsigned grid_x(int n_swg, int batches) { return 8u * (unsigned)n_swg * (unsigned)((batches + 7) / 8); }

hipError_t launch_softmax_forward(int dtype, const SoftmaxArgs &p, hipStream_t st)
{
    dim3 grid(grid_x(p.sched_wgs, p.batches)), block(64 * p.sched_waves);
    const float scale2 = p.scale * 1.4426950408889634f;
    if (dtype == BSA_F16)
        softmax_fwd_kernel<half_t, 4, 48><<<grid, block, 0, st>>>(
            (const half_t *)p.x, (half_t *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, scale2, p.causal ? 1 : 0);
    else if (dtype == BSA_BF16)
        softmax_fwd_kernel<bf16_t, 4, 48><<<grid, block, 0, st>>>(
            (const bf16_t *)p.x, (bf16_t *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, scale2, p.causal ? 1 : 0);
    else
        softmax_fwd_kernel<float, 2, 24><<<grid, block, 0, st>>>(
            (const float *)p.x, (float *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, scale2, p.causal ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_softmax_backward(int dtype, const SoftmaxArgs &p, hipStream_t st)
{
    dim3 grid(grid_x(p.sched_wgs, p.batches)), block(64 * p.sched_waves);
    if (dtype == BSA_F16)
        softmax_bwd_kernel<half_t, 2, 24><<<grid, block, 0, st>>>(
            (const half_t *)p.x, (const half_t *)p.dy, (half_t *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, p.scale);
    else if (dtype == BSA_BF16)
        softmax_bwd_kernel<bf16_t, 2, 24><<<grid, block, 0, st>>>(
            (const bf16_t *)p.x, (const bf16_t *)p.dy, (bf16_t *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, p.scale);
    else
        softmax_bwd_kernel<float, 1, 24><<<grid, block, 0, st>>>(
            (const float *)p.x, (const float *)p.dy, (float *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, p.scale);
    return hipGetLastError();
}

}  // namespace bsa
