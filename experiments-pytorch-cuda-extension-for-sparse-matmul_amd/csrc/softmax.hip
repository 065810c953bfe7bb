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

#ifdef BSA_TRACE
__device__ int g_sm_ablate = 0;   // debug builds: 8 = no stores, 16 = no loads
#define SM_ABLATE(bit) (g_sm_ablate & (bit))
#else
#define SM_ABLATE(bit) 0
#endif

constexpr int SM_MAX_WAVES = 8;

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

// Hides a register from common-subexpression elimination: the second pass over a register-resident
// slice must RE-derive the scaled scores from the packed data, not keep every unpacked float of the
// first pass alive (that is 2-4x the registers of the slice itself).
__device__ __forceinline__ void launder(uint4 &r)
{
    asm volatile("" : "+v"(r.x), "+v"(r.y), "+v"(r.z), "+v"(r.w));
}

__device__ __forceinline__ float finite_or_zero(float m) { return m == -__builtin_inff() ? 0.f : m; }

// ---------------------------------------------------------------------------
// Row-sliced walk: a block row of at most CBS blocks goes whole to two wavefronts,
// each owning 16 of the 32 element rows.  The wave issues every load of its slice
// at once (one 16-byte request per lane and block for fp16), keeps the slice in
// registers, and needs neither LDS nor a barrier: a row lives in LPR neighbouring
// lanes.  NS = 16-byte chunks per lane and block of a slice.
// ---------------------------------------------------------------------------
template <typename T, int CBS>
__device__ __forceinline__ void softmax_fwd_sliced(const T *__restrict__ xb, T *__restrict__ yb,
                                                   const BlockDesc *__restrict__ blocks, const SchedEntry &e,
                                                   float scale2, int causal)
{
    typedef Chunk<T> C;
    constexpr int NS = C::NQ / SCHED_ROW_SLICES, EPC = C::EPC, LPR = C::LPR;
    constexpr int ROWS_PER_Q = WAVE / LPR;
    const int l = lane_id();
    const int n = e.end - e.begin;
    const int row_base = (BS / SCHED_ROW_SLICES) * e.part() + l / LPR;   // + q * ROWS_PER_Q
    const int col0 = EPC * (l % LPR);
    const int slice_off = (BS2 / SCHED_ROW_SLICES) * e.part() + l * EPC;  // + q * 64 * EPC, inside a block
    const float NEG_INF = -__builtin_inff();

    float m[NS], s[NS];
#pragma unroll
    for (int q = 0; q < NS; ++q) { m[q] = NEG_INF; s[q] = 0.f; }
    DescWindow win;
    win.fetch(blocks, e.begin, e.end);

    if (n <= CBS) {
        // block indices and columns are re-read from the window (v_readlane) in every pass:
        // keeping 2 x CBS scalars alive would spill
        uint4 raw[CBS][NS];
#pragma unroll
        for (int j = 0; j < CBS; ++j) {
            if (j < n) {
                const BlockDesc d = win.get(e.begin + j);
#pragma unroll
                for (int q = 0; q < NS; ++q)
                    raw[j][q] = SM_ABLATE(16) ? make_uint4(d.idx, j, q, l)
                                              : ldg16_stream(xb + (size_t)d.idx * BS2 + slice_off + q * WAVE * EPC);
            }
        }
#pragma unroll
        for (int j = 0; j < CBS; ++j) {
            if (j < n) {
                const int bcol = win.get(e.begin + j).col();
#pragma unroll
                for (int q = 0; q < NS; ++q) {
                    if (causal) mask_chunk<T>(raw[j][q], row_base + q * ROWS_PER_Q, col0, bcol, e.group, scale2);
                    m[q] = fmaxf(m[q], chunk_scaled_max<T>(raw[j][q], scale2));
                }
            }
        }
#pragma unroll
        for (int q = 0; q < NS; ++q) m[q] = finite_or_zero(row_allreduce<LPR>(m[q], MaxOp()));
#pragma unroll
        for (int j = 0; j < CBS; ++j) {
            if (j < n) {
#pragma unroll
                for (int q = 0; q < NS; ++q) {
                    float v[EPC];
                    s[q] += chunk_exp<T>(raw[j][q], scale2, m[q], v);
                    raw[j][q] = C::pack(v);
                }
            }
            __builtin_amdgcn_sched_barrier(0);   // one block at a time: unpacking them all at once spills
        }
#pragma unroll
        for (int q = 0; q < NS; ++q) {
            s[q] = row_allreduce<LPR>(s[q], AddOp());
            s[q] = s[q] > 0.f ? 1.f / s[q] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < CBS; ++j) {
            if (j < n) {
#pragma unroll
                for (int q = 0; q < NS; ++q) {
                    float v[EPC];
                    C::unpack(raw[j][q], v);
#pragma unroll
                    for (int i = 0; i < EPC; ++i) v[i] *= s[q];
                    if (!SM_ABLATE(8) || v[0] == 1234.5f)
                        stg16_stream(yb + (size_t)win.get(e.begin + j).idx * BS2 + slice_off + q * WAVE * EPC, C::pack(v));
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }

    // longer than the register capacity (a schedule built with another slice_max): two passes
    for (int p = e.begin; p < e.end; ++p) {
        if (p > e.begin && ((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const BlockDesc d = win.get(p);
#pragma unroll
        for (int q = 0; q < NS; ++q) {
            float v[EPC];
            scaled_chunk<T>(ldg16_stream(xb + (size_t)d.idx * BS2 + slice_off + q * WAVE * EPC),
                            row_base + q * ROWS_PER_Q, col0, d.col(), e.group, scale2, causal, v);
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
    for (int q = 0; q < NS; ++q) {
        const float rm = finite_or_zero(row_allreduce<LPR>(m[q], MaxOp()));
        s[q] = row_allreduce<LPR>(s[q] * exp2_fast(m[q] - rm), AddOp());
        s[q] = s[q] > 0.f ? 1.f / s[q] : 0.f;
        m[q] = rm;
    }
    for (int p = e.begin; p < e.end; ++p) {
        if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const BlockDesc d = win.get(p);
#pragma unroll
        for (int q = 0; q < NS; ++q) {
            float v[EPC];
            scaled_chunk<T>(ldg16_stream(xb + (size_t)d.idx * BS2 + slice_off + q * WAVE * EPC),
                            row_base + q * ROWS_PER_Q, col0, d.col(), e.group, scale2, causal, v);
#pragma unroll
            for (int i = 0; i < EPC; ++i) v[i] = exp2_fast(v[i] - m[q]) * s[q];
            stg16_stream(yb + (size_t)d.idx * BS2 + slice_off + q * WAVE * EPC, C::pack(v));
        }
    }
}

// ---------------------------------------------------------------------------
// forward
// ---------------------------------------------------------------------------
template <typename T, int CB, int CBS>
__global__ __launch_bounds__(64 * SM_MAX_WAVES) void softmax_fwd_kernel(
    const T *__restrict__ x, T *__restrict__ y, const BlockDesc *__restrict__ blocks,
    const SchedEntry *__restrict__ sched, int n_swg, int batches, int nnz,
    float scale2 /* scale * log2(e) */, int causal)
{
    typedef Chunk<T> C;
    constexpr int NQ = C::NQ, EPC = C::EPC, LPR = C::LPR;
    constexpr int ROWS_PER_Q = WAVE / LPR;
    __shared__ float2 stats[SM_MAX_WAVES][BS];

    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
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
        softmax_fwd_sliced<T, CBS>(xb, yb, blocks, e, scale2, causal);
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
        // streaming pass 1: online max / sum
        for (int p = e.begin; p < e.end; ++p) {
            if (p > e.begin && ((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
            const BlockDesc d = win.get(p);
            const T *src = xb + (size_t)d.idx * BS2;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                float v[EPC];
                scaled_chunk<T>(ldg16_stream(src + (l + WAVE * q) * EPC), row0 + q * ROWS_PER_Q, col0, d.col(), e.group,
                                scale2, causal, v);
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
        // streaming pass 2: re-read, normalise, write
        for (int p = e.begin; p < e.end; ++p) {
            if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
            const BlockDesc d = win.get(p);
            const T *src = xb + (size_t)d.idx * BS2;
            T *dst = yb + (size_t)d.idx * BS2;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                float v[EPC];
                scaled_chunk<T>(ldg16_stream(src + (l + WAVE * q) * EPC), row0 + q * ROWS_PER_Q, col0, d.col(), e.group,
                                scale2, causal, v);
#pragma unroll
                for (int i = 0; i < EPC; ++i) v[i] = exp2_fast(v[i] - gm[q]) * inv_s[q];
                stg16_stream(dst + (l + WAVE * q) * EPC, C::pack(v));
            }
        }
    }
}

// ---------------------------------------------------------------------------
// backward: dx = scale * (dy - sum_row(dy * y)) * y
// ---------------------------------------------------------------------------
template <typename T, int CBS>
__device__ __forceinline__ void softmax_bwd_sliced(const T *__restrict__ y, const T *__restrict__ dy,
                                                   T *__restrict__ dx, const BlockDesc *__restrict__ blocks,
                                                   const SchedEntry &e, float scale)
{
    typedef Chunk<T> C;
    constexpr int NS = C::NQ / SCHED_ROW_SLICES, EPC = C::EPC, LPR = C::LPR;
    const int l = lane_id();
    const int n = e.end - e.begin;
    const int slice_off = (BS2 / SCHED_ROW_SLICES) * e.part() + l * EPC;
    float dot[NS];
#pragma unroll
    for (int q = 0; q < NS; ++q) dot[q] = 0.f;
    DescWindow win;
    win.fetch(blocks, e.begin, e.end);

    auto finish = [&](const uint4 &uy, const uint4 &ud, int q) {
        float a[EPC], b[EPC];
        C::unpack(uy, a);
        C::unpack(ud, b);
#pragma unroll
        for (int i = 0; i < EPC; ++i) a[i] = scale * (b[i] - dot[q]) * a[i];
        return C::pack(a);
    };
    auto accumulate = [&](const uint4 &uy, const uint4 &ud, int q) {
        float a[EPC], b[EPC];
        C::unpack(uy, a);
        C::unpack(ud, b);
#pragma unroll
        for (int i = 0; i < EPC; ++i) dot[q] += a[i] * b[i];
    };

    if (n <= CBS) {
        uint4 ry[CBS][NS], rd[CBS][NS];
#pragma unroll
        for (int j = 0; j < CBS; ++j) {
            if (j < n) {
                const size_t o = (size_t)win.get(e.begin + j).idx * BS2 + slice_off;
#pragma unroll
                for (int q = 0; q < NS; ++q) {
                    ry[j][q] = ldg16_stream(y + o + q * WAVE * EPC);
                    rd[j][q] = ldg16_stream(dy + o + q * WAVE * EPC);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < CBS; ++j)
            if (j < n)
#pragma unroll
                for (int q = 0; q < NS; ++q) accumulate(ry[j][q], rd[j][q], q);
#pragma unroll
        for (int q = 0; q < NS; ++q) dot[q] = row_allreduce<LPR>(dot[q], AddOp());
#pragma unroll
        for (int j = 0; j < CBS; ++j)
            if (j < n)
#pragma unroll
                for (int q = 0; q < NS; ++q)
                    stg16_stream(dx + (size_t)win.get(e.begin + j).idx * BS2 + slice_off + q * WAVE * EPC,
                          finish(ry[j][q], rd[j][q], q));
        return;
    }
    for (int p = e.begin; p < e.end; ++p) {
        if (p > e.begin && ((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const size_t o = (size_t)win.get(p).idx * BS2 + slice_off;
#pragma unroll
        for (int q = 0; q < NS; ++q) accumulate(ldg16_stream(y + o + q * WAVE * EPC), ldg16_stream(dy + o + q * WAVE * EPC), q);
    }
#pragma unroll
    for (int q = 0; q < NS; ++q) dot[q] = row_allreduce<LPR>(dot[q], AddOp());
    for (int p = e.begin; p < e.end; ++p) {
        if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
        const size_t o = (size_t)win.get(p).idx * BS2 + slice_off;
#pragma unroll
        for (int q = 0; q < NS; ++q)
            stg16_stream(dx + o + q * WAVE * EPC, finish(ldg16_stream(y + o + q * WAVE * EPC), ldg16_stream(dy + o + q * WAVE * EPC), q));
    }
}

template <typename T, int CB, int CBS>
__global__ __launch_bounds__(64 * SM_MAX_WAVES) void softmax_bwd_kernel(
    const T *__restrict__ y, const T *__restrict__ dy, T *__restrict__ dx,
    const BlockDesc *__restrict__ blocks, const SchedEntry *__restrict__ sched,
    int n_swg, int batches, int nnz, float scale)
{
    typedef Chunk<T> C;
    constexpr int NQ = C::NQ, EPC = C::EPC, LPR = C::LPR;
    constexpr int ROWS_PER_Q = WAVE / LPR;
    __shared__ float dots[SM_MAX_WAVES][BS];

    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const bool active = e.group >= 0;
    const int n = active ? e.end - e.begin : 0;
    const size_t boff = (size_t)batch * nnz * BS2;
    const int row0 = l / LPR;

    if (active && e.parts() > 1) {   // row-sliced waves sit in workgroups of their own
        softmax_bwd_sliced<T, CBS>(y + boff, dy + boff, dx + boff, blocks, e, scale);
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
        for (int p = e.begin; p < e.end; ++p) {
            if (p > e.begin && ((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
            const size_t o = boff + (size_t)win.get(p).idx * BS2;
#pragma unroll
            for (int q = 0; q < NQ; ++q) {
                float a[EPC], b[EPC];
                C::unpack(ldg16_stream(y + o + (l + WAVE * q) * EPC), a);
                C::unpack(ldg16_stream(dy + o + (l + WAVE * q) * EPC), b);
#pragma unroll
                for (int i = 0; i < EPC; ++i) dot[q] += a[i] * b[i];
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
        for (int p = e.begin; p < e.end; ++p) {
            if (((p - e.begin) & (WAVE - 1)) == 0) win.fetch(blocks, p, e.end);
            const size_t o = boff + (size_t)win.get(p).idx * BS2;
#pragma unroll
            for (int q = 0; q < NQ; ++q)
                stg16_stream(dx + o + (l + WAVE * q) * EPC,
                      finish(ldg16_stream(y + o + (l + WAVE * q) * EPC), ldg16_stream(dy + o + (l + WAVE * q) * EPC), q));
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
        softmax_fwd_kernel<half_t, 4, 24><<<grid, block, 0, st>>>(
            (const half_t *)p.x, (half_t *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, scale2, p.causal ? 1 : 0);
    else
        softmax_fwd_kernel<float, 2, 12><<<grid, block, 0, st>>>(
            (const float *)p.x, (float *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, scale2, p.causal ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_softmax_backward(int dtype, const SoftmaxArgs &p, hipStream_t st)
{
    dim3 grid(grid_x(p.sched_wgs, p.batches)), block(64 * p.sched_waves);
    if (dtype == BSA_F16)
        softmax_bwd_kernel<half_t, 2, 12><<<grid, block, 0, st>>>(
            (const half_t *)p.x, (const half_t *)p.dy, (half_t *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, p.scale);
    else
        softmax_bwd_kernel<float, 1, 6><<<grid, block, 0, st>>>(
            (const float *)p.x, (const float *)p.dy, (float *)p.out, (const BlockDesc *)p.blocks,
            (const SchedEntry *)p.sched + p.groups, p.sched_wgs, p.batches, p.nnz, p.scale);
    return hipGetLastError();
}

#ifdef BSA_TRACE
}  // namespace bsa
extern "C" int bsa_debug_sm_ablate(int bits)
{
    return (int)hipMemcpyToSymbol(HIP_SYMBOL(bsa::g_sm_ablate), &bits, sizeof(bits));
}
namespace bsa {
#endif

}  // namespace bsa
