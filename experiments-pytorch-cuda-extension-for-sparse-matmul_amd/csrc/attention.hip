// Fused block-sparse attention forward for gfx950: out = softmax(scale * q k^T, over the stored
// blocks of a row, causal if asked) v, without the scores ever leaving the chip.
//
// The reference computes this as three launches with the scores written and read twice in between
// (SDD sparse/native/sparse_smm_gpu.cu:22-95, softmax sparse_softmax.cu:113-155, DSD
// sparse_smm_gpu.cu:106-181, chained by the caller); per stored block that is 2 KB written + 2 KB
// read + 2 KB written + 2 KB read of HBM traffic that this kernel does not have.
//
// One wavefront walks a chunk of the blocks (r, c) of block row r:
//   S^T = K_c Q_r^T        32 keys x 32 queries, 4 MFMAs over head dim 64; Q_r stays in registers
//   online softmax          a lane holds ONE query column of S^T (16 keys; the other 16 sit in lane
//                           l ^ 32), so max, sum and the rescaling factor are per-lane scalars and
//                           one cross-lane exchange per block
//   O^T += V_c^T P^T        the probabilities go from the accumulators of the first product straight
//                           into the operand registers of the second: accumulator value v of lane
//                           half h is key 8 (v / 4) + 4 h + v % 4, and V_c is parked in LDS with
//                           its rows exchanged to match (put_strip_swapped_addr).  No LDS round
//                           trip, no shuffle.
// The waves of a row (a team of the schedule) merge their (max, sum, O^T) through LDS.
#include "bsa_device.hpp"
#include "lds_tiles.hpp"
#include "bsa_internal.hpp"
#include "../../include/bsa.h"

namespace bsa {

// per wave: K tiles (HD / 32 of 2 KB) + V strips (HD / 64 of 4 KB), reused for the O^T partial of the
// team merge (HD x 32 floats: the same size), + row stats
constexpr int at_lds_per_wave(int hd) { return 128 * hd + 512; }
constexpr float AT_LAZY = 8.f;                // log2 of the growth of a row maximum that forces a rescale

__device__ __forceinline__ float at_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float at_lane_xor32(float x)
{
    return __int_as_float(__builtin_amdgcn_ds_bpermute((lane_id() ^ 32) << 2, __float_as_int(x)));
}
__device__ __forceinline__ float at_finite_or_zero(float m) { return m == -__builtin_inff() ? 0.f : m; }

// Split rows of the forward walk: a block row longer than one workgroup's share is cut into parts
// that run in different workgroups.  Every part parks (O^T, max, sum) of its 32 queries in the
// workspace and bumps the row's counter; the part that arrives last merges the parts in part order
// (so the result does not depend on arrival order), resets the counter and stores the row.  Parked
// values are published and consumed with park_store / split_publish / split_consume / park_load
// (bsa_device.hpp: release and acquire at agent scope).
struct AtSplitWorkspace {
    int *counters;     // [batches][split_groups], zero between launches
    float *tiles;      // [batches][tile_slots][at_split_tile_floats(head dim)]
    int tile_slots, split_groups;
};
constexpr int at_split_tile_floats(int hd) { return 32 * hd + 2 * WAVE; }   // O^T, then every lane's max and sum
static size_t at_split_counter_bytes(int split_groups, int batches)
{
    return (((size_t)split_groups * batches * sizeof(int)) + 255) / 256 * 256;
}
size_t attention_workspace_bytes(int tile_slots, int split_groups, int batches, int head_dim)
{
    if (tile_slots <= 0 || split_groups <= 0) return 0;
    return at_split_counter_bytes(split_groups, batches) +
           (size_t)tile_slots * batches * at_split_tile_floats(head_dim) * sizeof(float);
}

// The backward walks split a group the same way, but their parts only add up (the row statistics are
// known): a part parks NT accumulator tiles, bumps the counter, and the last to arrive sums in part order.
template <int NT>
__device__ __forceinline__ void at_park(const f16v (&acc)[NT], float *dst)
{
    const int l = lane_id();
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i)
            park_store(dst + (t * 16 + i) * WAVE + l, acc[t][i]);
}
template <int NT>
__device__ __forceinline__ void at_sum_parts(f16v (&acc)[NT], const float *first, int stride, int parts)
{
    const int l = lane_id();
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = f16v{0};
    for (int p = 0; p < parts; ++p) {
        const float *src = first + (size_t)p * stride;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                acc[t][i] += park_load(src + (t * 16 + i) * WAVE + l);
    }
}
// workspace of the two backward walks: [row counters | row tiles of 32 hd floats | column counters | column
// tiles of 2 x 32 hd floats (dv^T, dk^T)]
static size_t at_bwd_region_bytes(int tile_slots, int split_groups, int batches, int tile_floats)
{
    if (tile_slots <= 0 || split_groups <= 0) return 0;
    return at_split_counter_bytes(split_groups, batches) + (size_t)tile_slots * batches * tile_floats * sizeof(float);
}
size_t attention_backward_workspace_bytes(int row_tile_slots, int row_split_groups, int col_tile_slots,
                                          int col_split_groups, int batches, int head_dim)
{
    return at_bwd_region_bytes(row_tile_slots, row_split_groups, batches, 32 * head_dim) +
           at_bwd_region_bytes(col_tile_slots, col_split_groups, batches, 64 * head_dim);
}

template <int HD, bool BF>
__global__ __launch_bounds__(512) void attention_fwd_f16_kernel(
    const half_t *__restrict__ q, const half_t *__restrict__ k, const half_t *__restrict__ v,
    half_t *__restrict__ out, float *__restrict__ lse, const BlockDesc *__restrict__ blocks,
    const SchedGroup *__restrict__ sched_groups, const SchedEntry *__restrict__ sched, AtSplitWorkspace ws,
    int n_swg, int batches, int rows_q, int rows_k, float scale2 /* scale * log2(e) */, int causal)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const bool active = e.group >= 0;
    const int r = e.group;
    const int qq = l & 31, h = l >> 5;          // query column of this lane, lane half
    const float NEG_INF = -__builtin_inff();

    constexpr int AT_HEAD = HD, AT_LDS_PER_WAVE = at_lds_per_wave(HD);
    constexpr int KT = HD / 32, VS = HD / 64;   // 32-wide K tiles, 64-wide V strips
    unsigned char *my_lds = lds_raw + (size_t)w * AT_LDS_PER_WAVE;
    half_t *tile_k = reinterpret_cast<half_t *>(my_lds);                 // KT [key][32 d] tiles
    half_t *tile_v = reinterpret_cast<half_t *>(my_lds + 2048 * KT);     // VS [key][64 n] strips, rows exchanged
    const half_t *kb = k + (size_t)batch * rows_k * AT_HEAD;
    const half_t *vb = v + (size_t)batch * rows_k * AT_HEAD;

    // Q_r as the column operand of S^T: lane (qq, h) holds d = 16 s + 8 h .. + 7 of query qq
    h8 qop[AT_HEAD / 16];
    if (active) {
        const half_t *qrow = q + ((size_t)batch * rows_q + BS * r + qq) * AT_HEAD + 8 * h;
#pragma unroll
        for (int s = 0; s < AT_HEAD / 16; ++s) qop[s] = as_h8(ldg16(qrow + 16 * s));
    }

    struct Frag { uint4 kk[KT][2], vv[VS][4]; };   // K_c as 32 x 32 tiles (d slices), V_c as 4 KB strips (n slices)
    DescWindow win;
    auto load = [&](int p, Frag &f) {
        const int c = win.get(p).col();
#pragma unroll
        for (int dt = 0; dt < KT; ++dt) ldg_tile32(kb + (size_t)(BS * c) * AT_HEAD + 32 * dt, AT_HEAD, f.kk[dt]);
        const half_t *vs = vb + (size_t)(BS * c) * AT_HEAD;
#pragma unroll
        for (int u = 0; u < VS; ++u)
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int piece = l + 64 * t;               // key row piece / 8, 16-byte piece % 8 of the 128-byte strip row
                f.vv[u][t] = ldg16(vs + (size_t)(piece >> 3) * AT_HEAD + 64 * u + 8 * (piece & 7));
            }
    };

    float m = NEG_INF, lsum = 0.f;               // running max of the query (both lane halves agree), this half's sum
    f16v oacc[KT];                               // O^T: lane = query column, values = head dims 32 t + 8 (v / 4) + 4 h + v % 4
#pragma unroll
    for (int t = 0; t < KT; ++t) oacc[t] = f16v{0};

    // registers -> staging tiles; the registers are free for the next block's loads afterwards
    auto stage = [&](const Frag &f) {
        wave_lds_fence();
#pragma unroll
        for (int dt = 0; dt < KT; ++dt) lds_put_kc<false>(tile_k + dt * BS2, f.kk[dt]);
#pragma unroll
        for (int u = 0; u < VS; ++u) lds_put_strip_swapped(tile_v + u * 2048, f.vv[u]);
        wave_lds_fence();
    };
    auto step = [&](int c) {
        f16v sacc = {0};
#pragma unroll
        for (int dt = 0; dt < KT; ++dt)
#pragma unroll
            for (int s = 0; s < 2; ++s)
                sacc = mfma_16<BF>(lds_get_kc(tile_k + dt * BS2, s), qop[2 * dt + s], sacc);

        // Row maximum of the scaled scores.  Off the diagonal nothing is masked and the scale is
        // folded into the exponent (one fused multiply-add per score); the diagonal block of a
        // causal launch takes the explicit route.
        float bm;
        const bool masked = causal && c >= r;
        float mul = scale2;                      // what is still to be applied to sacc in the exponent
        if (masked) {
            bm = NEG_INF;
            mul = 1.f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = 8 * (i >> 2) + 4 * h + (i & 3);
                sacc[i] = (c > r || key > qq) ? NEG_INF : sacc[i] * scale2;
                bm = fmaxf(bm, sacc[i]);
            }
        } else {
            float hi = sacc[0], lo = sacc[0];
#pragma unroll
            for (int i = 1; i < 16; ++i) {
                hi = fmaxf(hi, sacc[i]);
                if (scale2 < 0.f) lo = fminf(lo, sacc[i]);     // uniform: a negative scale turns the order round
            }
            bm = scale2 < 0.f ? lo * scale2 : hi * scale2;
        }
        bm = fmaxf(bm, at_lane_xor32(bm));
        // Lazy rescaling: the reference point m only moves when some row's maximum has grown by
        // more than 2^AT_LAZY since it was set, so the 32 multiplies of O^T (and the branch is
        // uniform) are skipped for most blocks; until then probabilities may reach 2^AT_LAZY,
        // which fp16 holds without loss of relative precision.
        if (__builtin_amdgcn_ballot_w64(bm > m + AT_LAZY) != 0ull) {
            const float m_new = fmaxf(m, bm);
            const float alpha = at_exp2(at_finite_or_zero(m) - at_finite_or_zero(m_new));
            const float keep = m == NEG_INF ? 0.f : alpha;      // nothing accumulated so far
            m = m_new;
            lsum *= keep;
#pragma unroll
            for (int t = 0; t < KT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[t][i] *= keep;
        }
        const float mm = at_finite_or_zero(m);
        float psum = 0.f;
        h8 pop[2];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float pv = at_exp2(__builtin_fmaf(sacc[i], mul, -mm));
            psum += pv;
            pop[i >> 3][i & 7] = narrow_16<BF>(pv);
        }
        lsum += psum;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int s = 0; s < 2; ++s)
                oacc[t] = mfma_16<BF>(lds_get_strip<false>(tile_v + (t / 2) * 2048, 32 * (t % 2), s), pop[s], oacc[t]);
    };

    // One block in flight: its tiles are requested as soon as the previous block's have been copied
    // to LDS, so the loads run under the previous block's products and softmax.  (A second set of
    // load registers costs an occupancy step, which measured worse than the shorter prefetch.)
    if (active) {
        Frag fr;
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            win.fetch(blocks, seg, seg_end);
            load(seg, fr);
            for (int p = seg; p < seg_end; ++p) {
                stage(fr);
                if (p + 1 < seg_end) load(p + 1, fr);
                step(win.get(p).col());
            }
        }
    }
    lsum += at_lane_xor32(lsum);                 // both halves used the same max

    // team merge: every wave but the leader parks (max, sum, O^T); the leader rescales and adds
    const int slot0 = e.first_wave(), nw = e.team_waves();
    const bool leader = active && w == slot0;
    constexpr int STAT_OFF = 128 * HD;                                // behind the HD x 32 floats of O^T
    float *park = reinterpret_cast<float *>(my_lds);
    float2 *stat = reinterpret_cast<float2 *>(my_lds + STAT_OFF);     // 32 (max, sum)
    if (active && !leader) {
        wave_lds_fence();
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) park[(t * 16 + i) * WAVE + l] = oacc[t][i];
        if (h == 0) stat[qq] = make_float2(m, lsum);
    }
    __syncthreads();
    if (!leader) return;
    if (nw > 1) {
        float M = m;
        for (int o = 1; o < nw; ++o)
            M = fmaxf(M, reinterpret_cast<const float2 *>(lds_raw + (size_t)(w + o) * AT_LDS_PER_WAVE + STAT_OFF)[qq].x);
        const float MM = at_finite_or_zero(M);
        const float mine = at_exp2(m - MM);
        lsum *= mine;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) oacc[t][i] *= mine;
        for (int o = 1; o < nw; ++o) {
            const unsigned char *other = lds_raw + (size_t)(w + o) * AT_LDS_PER_WAVE;
            const float2 st = reinterpret_cast<const float2 *>(other + STAT_OFF)[qq];
            const float f = at_exp2(st.x - MM);
            lsum += st.y * f;
            const float *op = reinterpret_cast<const float *>(other);
#pragma unroll
            for (int t = 0; t < KT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) oacc[t][i] += op[(t * 16 + i) * WAVE + l] * f;
        }
        m = M;                                   // the sums are relative to the team's reference point now
    }
    if (e.parts() > 1) {
        constexpr int TILE = at_split_tile_floats(HD);
        const SchedGroup sg = sched_groups[r];
        float *tile0 = ws.tiles + ((size_t)batch * ws.tile_slots + sg.tile_slot) * TILE;
        float *mine = tile0 + (size_t)e.part() * TILE;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i)
                park_store(mine + (t * 16 + i) * WAVE + l, oacc[t][i]);
        park_store(mine + 32 * HD + l, m);
        park_store(mine + 32 * HD + WAVE + l, lsum);
        int *counter = ws.counters + (size_t)batch * ws.split_groups + sg.split_index;
        const int parts = e.parts();
        if (split_publish(counter) != parts - 1) return;
        split_consume();
        float M = NEG_INF;
        for (int p = 0; p < parts; ++p)
            M = fmaxf(M, park_load(tile0 + (size_t)p * TILE + 32 * HD + l));
        const float MM = at_finite_or_zero(M);
        lsum = 0.f;
#pragma unroll
        for (int t = 0; t < KT; ++t) oacc[t] = f16v{0};
        for (int p = 0; p < parts; ++p) {
            const float *src = tile0 + (size_t)p * TILE;
            const float f = at_exp2(park_load(src + 32 * HD + l) - MM);
            lsum += park_load(src + 32 * HD + WAVE + l) * f;
#pragma unroll
            for (int t = 0; t < KT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                    oacc[t][i] += park_load(src + (t * 16 + i) * WAVE + l) * f;
        }
        m = M;
        split_reset(counter);
    }
    const float inv = lsum > 0.f ? 1.f / lsum : 0.f;
    // log2 of the row's sum of exponentials of the scaled scores (what the backward pass needs to
    // rebuild the probabilities); +inf for a row that sees nothing, so that they come out as zeros
    if (lse != nullptr && h == 0)
        lse[(size_t)batch * rows_q + BS * r + qq] = lsum > 0.f ? at_finite_or_zero(m) + __builtin_amdgcn_logf(lsum)
                                                               : __builtin_inff();
    half_t *orow = out + ((size_t)batch * rows_q + BS * r + qq) * AT_HEAD + 4 * h;
#pragma unroll
    for (int t = 0; t < KT; ++t) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = narrow_16<BF>(oacc[t][4 * g + j] * inv);
            *reinterpret_cast<h4 *>(orow + 32 * t + 8 * g) = o;
        }
    }
}

// ---------------------------------------------------------------------------
// Backward, first half: the probabilities P and the score gradients dS of every stored block, and
// dq, in one launch, from q, k, v, dO, O and the row statistics of the forward pass:
//   P  = exp2(scale2 * q k^T - lse)                         (no second softmax pass: lse is known)
//   dS = scale * P o (dO v^T - delta),  delta_q = sum_d dO_qd O_qd
//   dq^T += K_c^T dS^T                                       (K_c is on the chip already)
// This replaces SDD(q, k), softmax forward, SDD(dO, v), softmax backward and the DSD product dS k
// of the unfused chain (five launches, 350 MB of score traffic at seq 4096 and dS read once more) by
// one kernel that only WRITES the two block stacks.  Same walk as the forward kernel: a lane holds
// one query column of S^T and dP^T, and the fp16 dS values feed the dq product straight from those
// registers (the K_c tiles are read a second time along their rows, the reader exchanging rows the way
// the forward kernel parks V_c).
// The waves of a row add their dq^T parts through LDS.  The two products that follow
// (dk = dS^T q, dv = P^T dO) walk the columns and are DSD launches on P and dS.
// ---------------------------------------------------------------------------
// per wave: K tiles + V tiles, [key][32 d] each; the V tiles take the two result blocks afterwards, and
// the whole the dq^T part of the merge (HD x 32 floats)
constexpr int at_bwd_lds_per_wave(int hd) { return 128 * hd; }

template <int HD, bool BF>
__global__ __launch_bounds__(512) void attention_bwd_scores_kernel(
    const half_t *__restrict__ q, const half_t *__restrict__ k, const half_t *__restrict__ v,
    const half_t *__restrict__ dout, const half_t *__restrict__ out, const float *__restrict__ lse,
    half_t *__restrict__ p_out, half_t *__restrict__ ds_out, half_t *__restrict__ dq_out,
    float *__restrict__ delta_out,
    const BlockDesc *__restrict__ blocks, const SchedGroup *__restrict__ sched_groups,
    const SchedEntry *__restrict__ sched, AtSplitWorkspace ws,
    int n_swg, int batches, int rows_q, int rows_k, int nnz, float scale, int causal)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const bool active = e.group >= 0;
    const int r = e.group;
    const int qq = l & 31, h = l >> 5;
    constexpr int KT = HD / 32, LDS_PER_WAVE = at_bwd_lds_per_wave(HD);
    const float scale2 = scale * 1.4426950408889634f;

    unsigned char *my_lds = lds_raw + (size_t)w * LDS_PER_WAVE;
    half_t *tile_k = reinterpret_cast<half_t *>(my_lds);
    half_t *tile_v = tile_k + KT * BS2;
    const half_t *kb = k + (size_t)batch * rows_k * HD;
    const half_t *vb = v + (size_t)batch * rows_k * HD;
    half_t *pb = p_out + (size_t)batch * nnz * BS2;
    half_t *dsb = ds_out + (size_t)batch * nnz * BS2;

    f16v dqacc[KT];                              // dq^T: lane = query column, values = head dims as in the forward kernel
#pragma unroll
    for (int t = 0; t < KT; ++t) dqacc[t] = f16v{0};

    if (active && e.begin < e.end) {
        // column operands of the two products: lane (qq, h) holds d = 16 s + 8 h .. + 7 of query qq
        const size_t qoff = ((size_t)batch * rows_q + BS * r + qq) * HD + 8 * h;
        h8 qop[HD / 16], dop[HD / 16];
        float delta = 0.f;
#pragma unroll
        for (int s = 0; s < HD / 16; ++s) {
            qop[s] = as_h8(ldg16(q + qoff + 16 * s));
            dop[s] = as_h8(ldg16(dout + qoff + 16 * s));
            const h8 o = as_h8(ldg16(out + qoff + 16 * s));
#pragma unroll
            for (int i = 0; i < 8; ++i) delta += widen_16<BF>(dop[s][i]) * widen_16<BF>(o[i]);
        }
        delta += at_lane_xor32(delta);           // the other half of the head dim sits in lane l ^ 32
        const float row_lse = lse[(size_t)batch * rows_q + BS * r + qq];
        if (delta_out != nullptr && w == e.first_wave() && e.part() == 0 && h == 0)
            delta_out[(size_t)batch * rows_q + BS * r + qq] = delta;

        struct Frag { uint4 kk[KT][2], vv[KT][2]; };
        DescWindow win;
        auto load = [&](int p, Frag &f) {
            const int c = win.get(p).col();
#pragma unroll
            for (int dt = 0; dt < KT; ++dt) {
                ldg_tile32(kb + (size_t)(BS * c) * HD + 32 * dt, HD, f.kk[dt]);
                ldg_tile32(vb + (size_t)(BS * c) * HD + 32 * dt, HD, f.vv[dt]);
            }
        };
        Frag fr;
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            win.fetch(blocks, seg, seg_end);
            load(seg, fr);
            for (int p = seg; p < seg_end; ++p) {
                const BlockDesc d = win.get(p);
                const int c = d.col();
                wave_lds_fence();
#pragma unroll
                for (int dt = 0; dt < KT; ++dt) {
                    lds_put_kc<false>(tile_k + dt * BS2, fr.kk[dt]);
                    lds_put_kc<false>(tile_v + dt * BS2, fr.vv[dt]);
                }
                wave_lds_fence();
                if (p + 1 < seg_end) load(p + 1, fr);
                f16v sacc = {0}, dpacc = {0};
#pragma unroll
                for (int dt = 0; dt < KT; ++dt)
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        sacc = mfma_16<BF>(lds_get_kc(tile_k + dt * BS2, s), qop[2 * dt + s], sacc);
                        dpacc = mfma_16<BF>(lds_get_kc(tile_v + dt * BS2, s), dop[2 * dt + s], dpacc);
                    }
                // Accumulator value i of lane half h is key 8 (i / 4) + 4 h + i % 4 of query qq: four runs of 4
                // keys.  Written from here a store instruction would touch 64 separate 8-byte pieces, so
                // the two result blocks go through the (now idle) V tiles and leave as whole 2 KB
                // pieces, like the SDD result.  The K tiles stay: dq reads them once more.
                wave_lds_fence();
                h8 dsop[2];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    h4 pv, dv;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int i = 4 * g + j, key = 8 * g + 4 * h + j;
                        float pr = at_exp2(__builtin_fmaf(sacc[i], scale2, -row_lse));
                        if (causal && (c > r || (c == r && key > qq))) pr = 0.f;
                        pv[j] = narrow_16<BF>(pr);
                        dv[j] = narrow_16<BF>(scale * pr * (dpacc[i] - delta));
                        dsop[i >> 3][i & 7] = dv[j];
                    }
                    if (p_out != nullptr) {
                        const int at = 16 * kc_slot(qq, g) + 8 * h;   // 16-byte piece g of row qq, its half h
                        *reinterpret_cast<h4 *>(lds_bytes(tile_v) + at) = pv;
                        *reinterpret_cast<h4 *>(lds_bytes(tile_v + BS2) + at) = dv;
                    }
                }
                if (dq_out != nullptr) {
#pragma unroll
                    for (int t = 0; t < KT; ++t)
#pragma unroll
                        for (int s = 0; s < 2; ++s)
                            dqacc[t] = mfma_16<BF>(lds_get_kc_tr_swapped(tile_k + t * BS2, s), dsop[s], dqacc[t]);
                }
                if (p_out != nullptr) {
                    wave_lds_fence();
                    uint4 raw[2];
                    lds_get_linear(tile_v, raw);
                    stg_tile32(pb + (size_t)d.idx * BS2, raw);
                    lds_get_linear(tile_v + BS2, raw);
                    stg_tile32(dsb + (size_t)d.idx * BS2, raw);
                }
            }
        }
    }
    if (dq_out == nullptr) return;               // uniform over the launch

    // team merge: every wave of a row but the leader parks its dq^T part, the leader adds and stores
    const int slot0 = e.first_wave(), nw = e.team_waves();
    const bool leader = active && w == slot0;
    float *park = reinterpret_cast<float *>(my_lds);
    if (active && !leader) {
        wave_lds_fence();
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) park[(t * 16 + i) * WAVE + l] = dqacc[t][i];
    }
    __syncthreads();
    if (!leader) return;
    for (int o = 1; o < nw; ++o) {
        const float *op = reinterpret_cast<const float *>(lds_raw + (size_t)(w + o) * LDS_PER_WAVE);
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int i = 0; i < 16; ++i) dqacc[t][i] += op[(t * 16 + i) * WAVE + l];
    }
    if (e.parts() > 1) {                         // a row cut into parts: they add up in the workspace
        constexpr int TILE = 32 * HD;
        const SchedGroup sg = sched_groups[r];
        float *tile0 = ws.tiles + ((size_t)batch * ws.tile_slots + sg.tile_slot) * TILE;
        at_park<KT>(dqacc, tile0 + (size_t)e.part() * TILE);
        int *counter = ws.counters + (size_t)batch * ws.split_groups + sg.split_index;
        if (split_publish(counter) != e.parts() - 1) return;
        split_consume();
        at_sum_parts<KT>(dqacc, tile0, TILE, e.parts());
        split_reset(counter);
    }
    half_t *drow = dq_out + ((size_t)batch * rows_q + BS * r + qq) * HD + 4 * h;
#pragma unroll
    for (int t = 0; t < KT; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            h4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) o[j] = narrow_16<BF>(dqacc[t][4 * g + j]);
            *reinterpret_cast<h4 *>(drow + 32 * t + 8 * g) = o;
        }
}

hipError_t launch_attention_backward_scores(const AttentionArgs &p, hipStream_t st)
{
    dim3 grid(8u * (unsigned)p.sched_wgs * (unsigned)((p.batches + 7) / 8)), block(64 * p.sched_waves);
    const size_t lds = (size_t)p.sched_waves * at_bwd_lds_per_wave(p.head_dim);
#define BSA_AT_ARGS (const half_t *)p.q, (const half_t *)p.k, (const half_t *)p.v, (const half_t *)p.dout, \
                    (const half_t *)p.out, (const float *)p.lse, (half_t *)p.p_out, (half_t *)p.ds_out, (half_t *)p.dq_out, (float *)p.delta, \
                    (const BlockDesc *)p.blocks, (const SchedGroup *)p.sched, (const SchedEntry *)p.sched + p.groups, ws, \
                    p.sched_wgs, p.batches, \
                    32 * p.mask_rows, 32 * p.mask_cols, p.nnz, p.scale, p.causal ? 1 : 0
    AtSplitWorkspace ws;
    ws.tile_slots = p.tile_slots;
    ws.split_groups = p.split_groups;
    ws.counters = (int *)p.workspace;
    ws.tiles = (float *)((char *)p.workspace + at_split_counter_bytes(p.split_groups, p.batches));
    if (p.head_dim == 64) {
        if (p.bf16) attention_bwd_scores_kernel<64, true><<<grid, block, lds, st>>>(BSA_AT_ARGS);
        else attention_bwd_scores_kernel<64, false><<<grid, block, lds, st>>>(BSA_AT_ARGS);
    } else {
        if (lds > 65536) {
            const void *fn = p.bf16 ? (const void *)attention_bwd_scores_kernel<128, true>
                                    : (const void *)attention_bwd_scores_kernel<128, false>;
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        if (p.bf16) attention_bwd_scores_kernel<128, true><<<grid, block, lds, st>>>(BSA_AT_ARGS);
        else attention_bwd_scores_kernel<128, false><<<grid, block, lds, st>>>(BSA_AT_ARGS);
    }
#undef BSA_AT_ARGS
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Backward, the walk over the COLUMNS: dk and dv of block column c from the blocks (r, c) of the
// column table, with nothing but q, k, v, dO and two floats per query (lse of the forward pass,
// delta of the row walk above) read: the probabilities and the score gradients are rebuilt in
// registers a second time rather than stored by the row walk and read back (4 KB written + 4 KB
// read of HBM traffic per block that this pair of kernels does not have).
//   S  = Q_r K_c^T, dP = dO_r V_c^T    K_c and V_c stay in registers as the column operands; a lane
//                                      holds ONE key column, 16 queries
//   P, dS                              as in the row walk; lse and delta of the 16 queries come from a
//                                      256-byte LDS slot
//   dv^T += dO_r^T P,  dk^T += Q_r^T dS   the fp16 P and dS values are the column operands straight
//                                      from the accumulators, the Q_r and dO_r tiles are read a second
//                                      time along their rows (get_kc_tr_swapped_addr)
// The waves of a column add their parts through LDS.  Head dim 64 only: at 128 the four accumulator
// sets alone are 256 registers.
// ---------------------------------------------------------------------------
constexpr int at_bwd_col_lds_per_wave(int hd) { return 128 * hd + 256; }   // Q tiles + dO tiles (= one parked accumulator set) + stats

template <int HD, bool BF>
__global__ __launch_bounds__(512) void attention_bwd_dkdv_kernel(
    const half_t *__restrict__ q, const half_t *__restrict__ k, const half_t *__restrict__ v,
    const half_t *__restrict__ dout, const float *__restrict__ lse, const float *__restrict__ delta,
    half_t *__restrict__ dk_out, half_t *__restrict__ dv_out,
    const BlockDesc *__restrict__ blocks, const SchedGroup *__restrict__ sched_groups,
    const SchedEntry *__restrict__ sched, AtSplitWorkspace ws,
    int n_swg, int batches, int rows_q, int rows_k, float scale, int causal)
{
    extern __shared__ __align__(16) unsigned char lds_raw[];
    int batch, swg;
    if (!map_workgroup(n_swg, batches, batch, swg)) return;
    const int w = wave_id(), l = lane_id();
    const int W = (int)(blockDim.x >> 6);
    const SchedEntry e = sched[swg * W + w];
    const bool active = e.group >= 0;
    const int c = e.group;
    const int key = l & 31, h = l >> 5;          // key column of this lane, lane half
    constexpr int KT = HD / 32, LDS_PER_WAVE = at_bwd_col_lds_per_wave(HD);
    const float scale2 = scale * 1.4426950408889634f;

    unsigned char *my_lds = lds_raw + (size_t)w * LDS_PER_WAVE;
    half_t *tile_q = reinterpret_cast<half_t *>(my_lds);
    half_t *tile_do = tile_q + KT * BS2;
    float *stats = reinterpret_cast<float *>(my_lds + 128 * HD);      // 32 lse, 32 delta of the block's queries
    const half_t *qb = q + (size_t)batch * rows_q * HD;
    const half_t *dob = dout + (size_t)batch * rows_q * HD;
    const float *lse_b = lse + (size_t)batch * rows_q;
    const float *delta_b = delta + (size_t)batch * rows_q;

    f16v dvacc[KT], dkacc[KT];                   // dv^T, dk^T: lane = key column, values = head dims as in the forward kernel
#pragma unroll
    for (int t = 0; t < KT; ++t) dvacc[t] = dkacc[t] = f16v{0};

    if (active && e.begin < e.end) {
        // column operands of the first two products: lane (key, h) holds d = 16 s + 8 h .. + 7 of its key
        const size_t koff = ((size_t)batch * rows_k + BS * c + key) * HD + 8 * h;
        h8 kop[HD / 16], vop[HD / 16];
#pragma unroll
        for (int s = 0; s < HD / 16; ++s) {
            kop[s] = as_h8(ldg16(k + koff + 16 * s));
            vop[s] = as_h8(ldg16(v + koff + 16 * s));
        }
        struct Frag { uint4 qq[KT][2], dd[KT][2]; float stat; };
        DescWindow win;
        auto load = [&](int p, Frag &f) {
            const int r = win.get(p).row();
#pragma unroll
            for (int dt = 0; dt < KT; ++dt) {
                ldg_tile32(qb + (size_t)(BS * r) * HD + 32 * dt, HD, f.qq[dt]);
                ldg_tile32(dob + (size_t)(BS * r) * HD + 32 * dt, HD, f.dd[dt]);
            }
            f.stat = h == 0 ? lse_b[BS * r + key] : delta_b[BS * r + key];
        };
        Frag fr;
        for (int seg = e.begin; seg < e.end; seg += WAVE) {
            const int seg_end = seg + WAVE < e.end ? seg + WAVE : e.end;
            win.fetch(blocks, seg, seg_end);
            load(seg, fr);
            for (int p = seg; p < seg_end; ++p) {
                const int r = win.get(p).row();
                wave_lds_fence();
#pragma unroll
                for (int dt = 0; dt < KT; ++dt) {
                    lds_put_kc<false>(tile_q + dt * BS2, fr.qq[dt]);
                    lds_put_kc<false>(tile_do + dt * BS2, fr.dd[dt]);
                }
                stats[l] = fr.stat;
                wave_lds_fence();
                if (p + 1 < seg_end) load(p + 1, fr);
                f16v sacc = {0}, dpacc = {0};
#pragma unroll
                for (int dt = 0; dt < KT; ++dt)
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        sacc = mfma_16<BF>(lds_get_kc(tile_q + dt * BS2, s), kop[2 * dt + s], sacc);
                        dpacc = mfma_16<BF>(lds_get_kc(tile_do + dt * BS2, s), vop[2 * dt + s], dpacc);
                    }
                // accumulator value i of lane half h is query 8 (i / 4) + 4 h + i % 4 of this lane's key
                h8 pop[2], dsop[2];
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const float4 ls = *reinterpret_cast<const float4 *>(stats + 8 * g + 4 * h);
                    const float4 dl = *reinterpret_cast<const float4 *>(stats + 32 + 8 * g + 4 * h);
                    const float lsv[4] = {ls.x, ls.y, ls.z, ls.w}, dlv[4] = {dl.x, dl.y, dl.z, dl.w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int i = 4 * g + j, qrow = 8 * g + 4 * h + j;
                        float pr = at_exp2(__builtin_fmaf(sacc[i], scale2, -lsv[j]));
                        if (causal && (c > r || (c == r && key > qrow))) pr = 0.f;
                        pop[i >> 3][i & 7] = narrow_16<BF>(pr);
                        dsop[i >> 3][i & 7] = narrow_16<BF>(scale * pr * (dpacc[i] - dlv[j]));
                    }
                }
#pragma unroll
                for (int t = 0; t < KT; ++t)
#pragma unroll
                    for (int s = 0; s < 2; ++s) {
                        dvacc[t] = mfma_16<BF>(lds_get_kc_tr_swapped(tile_do + t * BS2, s), pop[s], dvacc[t]);
                        dkacc[t] = mfma_16<BF>(lds_get_kc_tr_swapped(tile_q + t * BS2, s), dsop[s], dkacc[t]);
                    }
            }
        }
    }

    // team merge, one accumulator set at a time (the staging tiles hold exactly one): every wave of a
    // column but the leader parks its part, the leader adds
    const int slot0 = e.first_wave(), nw = e.team_waves();
    const bool leader = active && w == slot0;
    float *park = reinterpret_cast<float *>(my_lds);
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        f16v (&acc)[KT] = which == 0 ? dvacc : dkacc;
        if (which == 1) __syncthreads();         // the leaders have read the first set
        if (active && !leader) {
            wave_lds_fence();
#pragma unroll
            for (int t = 0; t < KT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) park[(t * 16 + i) * WAVE + l] = acc[t][i];
        }
        __syncthreads();
        if (leader) {
            for (int o = 1; o < nw; ++o) {
                const float *op = reinterpret_cast<const float *>(lds_raw + (size_t)(w + o) * LDS_PER_WAVE);
#pragma unroll
                for (int t = 0; t < KT; ++t)
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[t][i] += op[(t * 16 + i) * WAVE + l];
            }
        }
    }
    if (!leader) return;
    if (e.parts() > 1) {                         // a column cut into parts: they add up in the workspace
        constexpr int HALF = 32 * HD, TILE = 2 * HALF;       // dv^T then dk^T
        const SchedGroup sg = sched_groups[c];
        float *tile0 = ws.tiles + ((size_t)batch * ws.tile_slots + sg.tile_slot) * TILE;
        at_park<KT>(dvacc, tile0 + (size_t)e.part() * TILE);
        at_park<KT>(dkacc, tile0 + (size_t)e.part() * TILE + HALF);
        int *counter = ws.counters + (size_t)batch * ws.split_groups + sg.split_index;
        if (split_publish(counter) != e.parts() - 1) return;
        split_consume();
        at_sum_parts<KT>(dvacc, tile0, TILE, e.parts());
        at_sum_parts<KT>(dkacc, tile0 + HALF, TILE, e.parts());
        split_reset(counter);
    }
#pragma unroll
    for (int which = 0; which < 2; ++which) {
        f16v (&acc)[KT] = which == 0 ? dvacc : dkacc;
        half_t *drow = (which == 0 ? dv_out : dk_out) + ((size_t)batch * rows_k + BS * c + key) * HD + 4 * h;
#pragma unroll
        for (int t = 0; t < KT; ++t)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                h4 o;
#pragma unroll
                for (int j = 0; j < 4; ++j) o[j] = narrow_16<BF>(acc[t][4 * g + j]);
                *reinterpret_cast<h4 *>(drow + 32 * t + 8 * g) = o;
            }
    }
}

hipError_t launch_attention_backward_dkdv(const AttentionArgs &p, hipStream_t st)
{
    dim3 grid(8u * (unsigned)p.sched_wgs * (unsigned)((p.batches + 7) / 8)), block(64 * p.sched_waves);
    const size_t lds = (size_t)p.sched_waves * at_bwd_col_lds_per_wave(64);
#define BSA_AT_ARGS (const half_t *)p.q, (const half_t *)p.k, (const half_t *)p.v, (const half_t *)p.dout, \
                    (const float *)p.lse, (const float *)p.delta, (half_t *)p.dk_out, (half_t *)p.dv_out, \
                    (const BlockDesc *)p.blocks, (const SchedGroup *)p.sched, (const SchedEntry *)p.sched + p.groups, ws, \
                    p.sched_wgs, p.batches, \
                    32 * p.mask_rows, 32 * p.mask_cols, p.scale, p.causal ? 1 : 0
    AtSplitWorkspace ws;
    ws.tile_slots = p.tile_slots;
    ws.split_groups = p.split_groups;
    ws.counters = (int *)p.workspace;
    ws.tiles = (float *)((char *)p.workspace + at_split_counter_bytes(p.split_groups, p.batches));
    if (lds > 65536) {
        const void *fn = p.bf16 ? (const void *)attention_bwd_dkdv_kernel<64, true>
                                : (const void *)attention_bwd_dkdv_kernel<64, false>;
        hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    if (p.bf16) attention_bwd_dkdv_kernel<64, true><<<grid, block, lds, st>>>(BSA_AT_ARGS);
    else attention_bwd_dkdv_kernel<64, false><<<grid, block, lds, st>>>(BSA_AT_ARGS);
#undef BSA_AT_ARGS
    return hipGetLastError();
}

hipError_t launch_attention_forward(const AttentionArgs &p, hipStream_t st)
{
    dim3 grid(8u * (unsigned)p.sched_wgs * (unsigned)((p.batches + 7) / 8)), block(64 * p.sched_waves);
    AtSplitWorkspace ws;
    ws.tile_slots = p.tile_slots;
    ws.split_groups = p.split_groups;
    ws.counters = (int *)p.workspace;
    ws.tiles = (float *)((char *)p.workspace + at_split_counter_bytes(p.split_groups, p.batches));
#define BSA_AT_ARGS (const half_t *)p.q, (const half_t *)p.k, (const half_t *)p.v, (half_t *)p.out, (float *)p.lse, \
                    (const BlockDesc *)p.blocks, (const SchedGroup *)p.sched, (const SchedEntry *)p.sched + p.groups, ws, \
                    p.sched_wgs, p.batches, \
                    32 * p.mask_rows, 32 * p.mask_cols, p.scale * 1.4426950408889634f, p.causal ? 1 : 0
    const size_t lds = (size_t)p.sched_waves * at_lds_per_wave(p.head_dim);
    if (p.head_dim == 64) {
        if (lds > 65536) {   // 8 waves x 8.5 KB
            const void *fn = p.bf16 ? (const void *)attention_fwd_f16_kernel<64, true>
                                    : (const void *)attention_fwd_f16_kernel<64, false>;
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        if (p.bf16) attention_fwd_f16_kernel<64, true><<<grid, block, lds, st>>>(BSA_AT_ARGS);
        else attention_fwd_f16_kernel<64, false><<<grid, block, lds, st>>>(BSA_AT_ARGS);
    } else {
        // more than 3 waves x 16.5 KB of staging exceed the 64 KB a launch gets without asking
        if (lds > 65536) {
            const void *fn = p.bf16 ? (const void *)attention_fwd_f16_kernel<128, true>
                                    : (const void *)attention_fwd_f16_kernel<128, false>;
            hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return e;
        }
        if (p.bf16) attention_fwd_f16_kernel<128, true><<<grid, block, lds, st>>>(BSA_AT_ARGS);
        else attention_fwd_f16_kernel<128, false><<<grid, block, lds, st>>>(BSA_AT_ARGS);
    }
#undef BSA_AT_ARGS
    return hipGetLastError();
}

}  // namespace bsa
