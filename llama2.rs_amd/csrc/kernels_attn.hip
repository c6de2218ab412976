// Decode attention for one query position (src/models.rs:131-176, :228-256):
// RoPE on q and on the new key, the cache write, scores, softmax and the
// weighted sum of values in one kernel; a second, small kernel merges the
// splits when the timesteps are cut across several blocks.  gfx950, wave64.
//
// The softmax is computed in the running-maximum form: every group of lanes
// keeps (m, l, acc) = (largest score so far, sum of e^(s - m), sum of
// e^(s - m) v) and rescales when m grows; groups, waves and splits are merged
// by the same rule.  That is the function softmax(src/util.rs:49-65) followed
// by the weighted sum (:160-174); only the order of the roundings differs.
// Scores are kept in units of log2: t = (q.k) * log2(e) / sqrt(head_size), so
// that e^(s - m) is one v_exp_f32 of t - m (1 ulp; the scaling of the argument
// adds a relative error of about |s - m| * 6e-8 to a weight).
//
// Compiled with -ffp-contract=off; FMAs appear only where written as fmaf().
#include <stdlib.h>
#include <string.h>

#include "l2_internal.h"

namespace {

template <int CTRL>
__device__ __forceinline__ float dpp_xchg(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
    return __builtin_bit_cast(float, r);
}

template <class T>
__device__ __forceinline__ T ld_at(const void *base, uint32_t byte_offset) {
    return *reinterpret_cast<const T *>(reinterpret_cast<const char *>(base) + byte_offset);
}

// Every kernel argument of a decode step, required in scalar registers at once: the arguments are cold in
// the scalar cache when a kernel starts, and loads placed where the values are first used follow each other
// (three round trips of some 0.3 us in front of the first cache row otherwise).
__device__ __forceinline__ void pin_args(const AttnDecode &A) {
    asm volatile("" ::"s"(A.q), "s"(A.k_new), "s"(A.v_new), "s"(A.kcache), "s"(A.vcache), "s"(A.cos_t), "s"(A.sin_t),
                 "s"(A.pos), "s"(A.dpos), "s"(A.out), "s"(A.scatter), "s"(A.part), "s"(A.n_heads), "s"(A.n_kv_heads),
                 "s"(A.ts), "s"(A.n_splits), "s"(A.max_splits));
}

constexpr float kNoScore = -1e30f; // "no timestep yet": finite, so that differences never give NaN

__device__ __forceinline__ float exp2_fast(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_xchg<0xB1>(v);
    v += dpp_xchg<0x4E>(v);
    v += dpp_xchg<0x141>(v);
    v += dpp_xchg<0x140>(v);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_xchg<0xB1>(v));
    v = fmaxf(v, dpp_xchg<0x4E>(v));
    v = fmaxf(v, dpp_xchg<0x141>(v));
    v = fmaxf(v, dpp_xchg<0x140>(v));
    v = fmaxf(v, __shfl_xor(v, 16));
    v = fmaxf(v, __shfl_xor(v, 32));
    return v;
}

// Floats per row of the LDS tiles in which rows of lanes, waves and splits meet: the 128 partial outputs, then
// (m, l).  The outputs are stored four at a time (16-byte LDS stores), so a row starts on a 16-byte boundary.
constexpr int kCombRow = 128 + 4;
static_assert(kCombRow * sizeof(float) % 16 == 0, "rows of the merge tiles are written with 16-byte stores");

// Layout of a block: NWV waves x 4 rows of 16 lanes.  One row of lanes handles
// one timestep at a time, each lane 8 of the 128 head dimensions; a block
// covers 4 NWV timesteps per step and PD steps per tile, all of a tile's loads
// being issued before its arithmetic.  NWV is 4 when the timesteps are cut
// into splits; wider blocks were measured slower for the single block per kv
// head of a short context (more waves to start and to merge).  All QG query heads of the kv head share
// each K and V load (grouped-query attention, src/models.rs:142-145).
template <int QG, int NWV>
__global__ __launch_bounds__(NWV * 64) void attn_decode_kernel(const AttnDecode A) {
    constexpr int NT = NWV * 64, TSTEP = NWV * 4;
    constexpr int HS = 128, HALF = 64;
    constexpr int PD = QG >= 8 ? 2 : 4; // steps in flight and per pass through the phases (4 at 8 heads: over 256 registers, one block per CU, slower)
    __shared__ float qs[QG * HS];
    __shared__ float kvnew[2][HS];
    // With 4 or 8 query heads per kv head the four 16-lane rows of every wave hand their partial results
    // over through (dynamic) LDS: merging them with cross-row shuffles first takes 10 shuffles per head and
    // step, 160 at 8 heads, a fifth of the kernel at long contexts.
    constexpr bool kRowsInLds = QG >= 4;
    constexpr int NR = kRowsInLds ? NWV * 4 : NWV; // partial results that meet in LDS
    __shared__ __align__(16) float comb_s[kRowsInLds ? 1 : NWV][QG][kCombRow];
    __shared__ float wts[QG][16], m_all[QG], den_all[QG];
    extern __shared__ __align__(16) float comb_d[]; // [NR][QG][kCombRow] when kRowsInLds
    float(*comb)[QG][kCombRow] = kRowsInLds ? reinterpret_cast<float(*)[QG][kCombRow]>(comb_d) : comb_s;
    pin_args(A);
    const int kvh = blockIdx.x, sp = blockIdx.y;
    const int pos = A.dpos ? A.dpos[0] : A.pos;
    const int t0 = sp * A.ts;
    if (t0 > pos) return;
    const int t1 = min(t0 + A.ts, pos + 1);
    const int n = t1 - t0;
    const int kv_dim = A.n_kv_heads * HS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ds = lane & 15;            // dims [8 ds, 8 ds + 8)
    const int tl = wave * 4 + (lane >> 4); // this row's timestep within a step

    const float *__restrict__ kc = A.kcache;
    const float *__restrict__ vc = A.vcache;
    const uint32_t row_bytes = (uint32_t)kv_dim * 4u;
    const uint32_t lane_off = (uint32_t)(kvh * HS + ds * 8) * 4u;
    const int t_last = t1 - 1;

    struct Step {
        float4 k0, k1, v0, v1;
    };
    // Unconditional loads: rows past the end re-read the last row, and the row
    // of the new position is read although its values are replaced below.
    auto fetch = [&](int it, Step &d) {
        const int t = min(t0 + it * TSTEP + tl, t_last);
        const uint32_t off = __umul24(t, row_bytes) + lane_off;
        d.k0 = ld_at<float4>(kc, off);
        d.k1 = ld_at<float4>(kc, off + 16);
        d.v0 = ld_at<float4>(vc, off);
        d.v1 = ld_at<float4>(vc, off + 16);
    };
    // The small loads that the staging below needs go out first: loads return in
    // order, so behind the first tile's loads they would wait for all of them.
    // Every thread stages something (threads beyond the work repeat another
    // thread's element), so that no load can move into a branch further down.
    const float *ct = A.cos_t + (size_t)pos * HALF;
    const float *st = A.sin_t + (size_t)pos * HALF;
    constexpr int NQ = (QG * HALF + NT - 1) / NT;
    float qa[NQ], qb[NQ], qc[NQ], qsn[NQ];
#pragma unroll
    for (int r = 0; r < NQ; r++) {
        const int idx = (tid + r * NT) % (QG * HALF);
        const int j = idx >> 6, i = idx & 63;
        const float *qh = A.q + (size_t)(kvh * QG + j) * HS;
        qa[r] = qh[i], qb[r] = qh[i + HALF];
        qc[r] = ct[i], qsn[r] = st[i];
    }
    const int hd = tid & 63;
    const float nk_a = A.k_new[(size_t)kvh * HS + hd], nk_b = A.k_new[(size_t)kvh * HS + hd + HALF];
    const float nv = A.v_new[(size_t)kvh * HS + (tid & 127)];
    const float nc = ct[hd], ns = st[hd];
    __builtin_amdgcn_sched_barrier(0);

    Step pipe[PD];
#pragma unroll
    for (int u = 0; u < PD; u++) fetch(u, pipe[u]); // first tile: in flight while q is staged
    __builtin_amdgcn_sched_barrier(0);

    // q with RoPE, src/models.rs:100-129 (the second half uses the rotated first half)
#pragma unroll
    for (int r = 0; r < NQ; r++) {
        const int idx = (tid + r * NT) % (QG * HALF);
        const int j = idx >> 6, i = idx & 63;
        const float first = qa[r] * qc[r] - qb[r] * qsn[r];
        qs[j * HS + i] = first;
        qs[j * HS + HALF + i] = qb[r] * qc[r] + first * qsn[r];
    }
    // the new key, rotated, and the new value; the block whose range ends at pos
    // also writes them to the cache (:236-249)
    const bool owns_new = (t1 == pos + 1);
    {
        const float first = nk_a * nc - nk_b * ns;
        const float second = nk_b * nc + first * ns;
        kvnew[0][hd] = first;
        kvnew[0][hd + HALF] = second;
        kvnew[1][tid & 127] = nv;
        if (owns_new) {
            if (tid < HALF) {
                float *kw = A.kcache + (size_t)pos * kv_dim + kvh * HS;
                kw[tid] = first;
                kw[tid + HALF] = second;
            } else if (tid >= 128 && tid < 256) {
                A.vcache[(size_t)pos * kv_dim + kvh * HS + (tid - 128)] = nv;
            }
        }
    }
    __syncthreads();

    // q in registers, except for 8 heads per kv head, where the registers go to the accumulators
    constexpr bool kQInLds = QG >= 8;
    float q[kQInLds ? 1 : QG][8];
    if constexpr (!kQInLds) {
#pragma unroll
        for (int j = 0; j < QG; j++) {
            const float4 a = *reinterpret_cast<const float4 *>(&qs[j * HS + ds * 8]);
            const float4 b = *reinterpret_cast<const float4 *>(&qs[j * HS + ds * 8 + 4]);
            q[j][0] = a.x, q[j][1] = a.y, q[j][2] = a.z, q[j][3] = a.w;
            q[j][4] = b.x, q[j][5] = b.y, q[j][6] = b.z, q[j][7] = b.w;
        }
    }
    float m[QG], l[QG], acc[QG][8];
#pragma unroll
    for (int j = 0; j < QG; j++) {
        m[j] = kNoScore;
        l[j] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[j][e] = 0.f;
    }
    // log2(e) / sqrt(head_size): src/models.rs:154 divides the score by sqrt(head_size)
    const float scale = 1.44269504088896340736f / sqrtf((float)HS);
    const int n_it = (n + TSTEP - 1) / TSTEP;
    const int n_tiles = (n_it + PD - 1) / PD;
    for (int tile = 0; tile < n_tiles; tile++) {
        if (tile > 0) { // all of the tile's loads, then its arithmetic
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < PD; u++) fetch(tile * PD + u, pipe[u]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // The tile's PD steps go through the phases together — all scores, one update of the running maxima,
        // all weights and weighted sums — so that the dependent chains of one step (dot product, four
        // cross-lane adds, exponential) interleave with those of the others: a block is often alone on its
        // CU, one wave per SIMD, and nothing else fills the gaps between dependent instructions.
        float k[PD][8], v[PD][8];
        float sc[PD][QG];
        bool valid[PD];
        float mt[QG];
#pragma unroll
        for (int u = 0; u < PD; u++) {
            const int t = t0 + (tile * PD + u) * TSTEP + tl;
            valid[u] = t < t1;
            const Step &d = pipe[u];
            const float kk[8] = {d.k0.x, d.k0.y, d.k0.z, d.k0.w, d.k1.x, d.k1.y, d.k1.z, d.k1.w};
            const float vv[8] = {d.v0.x, d.v0.y, d.v0.z, d.v0.w, d.v1.x, d.v1.y, d.v1.z, d.v1.w};
#pragma unroll
            for (int e = 0; e < 8; e++) k[u][e] = kk[e], v[u][e] = vv[e];
            if (__any(t == pos)) { // once per block: the row of the new position comes from LDS, not from the cache
                const bool is_new = t == pos;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    k[u][e] = is_new ? kvnew[0][ds * 8 + e] : k[u][e];
                    v[u][e] = is_new ? kvnew[1][ds * 8 + e] : v[u][e];
                }
            }
#pragma unroll
            for (int e = 0; e < 8; e++) v[u][e] = valid[u] ? v[u][e] : 0.f; // a row past the end may hold anything, NaN included
        }
#pragma unroll
        for (int j = 0; j < QG; j++) {
            float qj[8];
            if constexpr (kQInLds) { // one read of the head's q for all the steps of the tile
                const float4 a = *reinterpret_cast<const float4 *>(&qs[j * HS + ds * 8]);
                const float4 b = *reinterpret_cast<const float4 *>(&qs[j * HS + ds * 8 + 4]);
                qj[0] = a.x, qj[1] = a.y, qj[2] = a.z, qj[3] = a.w, qj[4] = b.x, qj[5] = b.y, qj[6] = b.z, qj[7] = b.w;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) qj[e] = q[j][e];
            }
            float mj = kNoScore;
#pragma unroll
            for (int u = 0; u < PD; u++) {
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) s = fmaf(qj[e], k[u][e], s);
                s += dpp_xchg<0xB1>(s);
                s += dpp_xchg<0x4E>(s);
                s += dpp_xchg<0x141>(s);
                s += dpp_xchg<0x140>(s);
                s = valid[u] ? s * scale : kNoScore;
                sc[u][j] = s;
                mj = fmaxf(mj, s);
            }
            mt[j] = mj;
        }
        bool grow = false;
#pragma unroll
        for (int j = 0; j < QG; j++) grow |= mt[j] > m[j];
        if (__any(grow)) { // some row's maximum moves: rescale what was summed so far
#pragma unroll
            for (int j = 0; j < QG; j++) {
                const float m_new = fmaxf(m[j], mt[j]);
                const float c = exp2_fast(m[j] - m_new);
                l[j] *= c;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[j][e] *= c;
                m[j] = m_new;
            }
        }
#pragma unroll
        for (int u = 0; u < PD; u++) {
#pragma unroll
            for (int j = 0; j < QG; j++) {
                const float p = valid[u] ? exp2_fast(sc[u][j] - m[j]) : 0.f;
                l[j] += p;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[j][e] = fmaf(p, v[u][e], acc[j][e]);
            }
        }
    }

    if constexpr (!kRowsInLds) {
        // merge the 4 rows of the wave (lanes 16 and 32 apart hold the same dims)
#pragma unroll
        for (int step = 16; step <= 32; step *= 2) {
#pragma unroll
            for (int j = 0; j < QG; j++) {
                const float mo = __shfl_xor(m[j], step);
                const float lo = __shfl_xor(l[j], step);
                const float M = fmaxf(m[j], mo);
                const float w1 = exp2_fast(m[j] - M), w2 = exp2_fast(mo - M);
                l[j] = l[j] * w1 + lo * w2;
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float ao = __shfl_xor(acc[j][e], step);
                    acc[j][e] = acc[j][e] * w1 + ao * w2;
                }
                m[j] = M;
            }
        }
    }
    if (kRowsInLds || lane < 16) {
        const int slot = kRowsInLds ? wave * 4 + (lane >> 4) : wave;
#pragma unroll
        for (int j = 0; j < QG; j++) {
            *reinterpret_cast<float4 *>(&comb[slot][j][ds * 8]) = make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
            *reinterpret_cast<float4 *>(&comb[slot][j][ds * 8 + 4]) =
                make_float4(acc[j][4], acc[j][5], acc[j][6], acc[j][7]);
            if (ds == 0) {
                comb[slot][j][HS] = m[j];
                comb[slot][j][HS + 1] = l[j];
            }
        }
    }
    __syncthreads();
    if constexpr (kRowsInLds) {
        // weights of the 16 partial results of every head: one thread per (head, partial), a head per 16-lane row
        if (tid < QG * 16) {
            const int j = tid >> 4, e = tid & 15;
            const float me = comb[e][j][HS];
            float M = me;
            M = fmaxf(M, dpp_xchg<0xB1>(M));
            M = fmaxf(M, dpp_xchg<0x4E>(M));
            M = fmaxf(M, dpp_xchg<0x141>(M));
            M = fmaxf(M, dpp_xchg<0x140>(M));
            const float w = exp2_fast(me - M);
            float wl = w * comb[e][j][HS + 1];
            wl += dpp_xchg<0xB1>(wl);
            wl += dpp_xchg<0x4E>(wl);
            wl += dpp_xchg<0x141>(wl);
            wl += dpp_xchg<0x140>(wl);
            wts[j][e] = w;
            if (e == 0) {
                m_all[j] = M;
                den_all[j] = wl;
            }
        }
        __syncthreads();
    }
    // merge; one thread per (head, dim)
    for (int idx = tid; idx < QG * HS; idx += NT) {
        const int j = idx >> 7, d = idx & 127;
        float M, num = 0.f, den = 0.f;
        if constexpr (kRowsInLds) {
#pragma unroll
            for (int w = 0; w < NR; w++) num = fmaf(wts[j][w], comb[w][j][d], num);
            M = m_all[j];
            den = den_all[j];
        } else {
            M = comb[0][j][HS];
#pragma unroll
            for (int w = 1; w < NR; w++) M = fmaxf(M, comb[w][j][HS]);
#pragma unroll
            for (int w = 0; w < NR; w++) {
                const float e = exp2_fast(comb[w][j][HS] - M);
                num = fmaf(e, comb[w][j][d], num);
                den = fmaf(e, comb[w][j][HS + 1], den);
            }
        }
        const int h = kvh * QG + j;
        if (A.n_splits == 1) {
            const int i = h * HS + d;
            A.out[A.scatter ? A.scatter[i] : i] = num / den;
        } else {
            float *p = A.part + ((size_t)h * A.max_splits + sp) * (HS + 2);
            p[d] = num;
            if (d == 0) {
                p[HS] = M;
                p[HS + 1] = den;
            }
        }
    }
}

// The same decode step for grouped-query models (4 or 8 query heads per kv head) on the matrix cores, all in
// fp32 (v_mfma_f32_16x16x4_f32): the query heads of the kv head are columns of the tile, so a cache row
// costs the same whatever their number, and the dot products need no cross-lane sums.
//
// A wave takes tiles of 16 timesteps.  With lane = (i = lane % 16, kb = lane / 16):
//   S^T = K Q^T      A: lane (timestep i, kb) holds K[t][16 m + 4 kb + e], B: lane (head i, kb) holds
//                    Q[head][16 m + 4 kb + e]; MFMA step (m, e), m < 8, e < 4, contracts over those four d.
//                    The A operand is what a 16-byte load of the cache row gives: no LDS on the way.
//   C layout         lane (head j, kb), register r -> timestep 4 kb + r: the four lanes of a head hold its
//                    16 scores, the running maximum is shared by them, the running sum is per lane.
//   O^T += V^T P^T   MFMA step (r, c) contracts over timesteps 4 kb + r, the lane's own register r of P: the
//                    B operand needs no data movement.  A: lane (i, kb) holds V[4 kb + r][d] with
//                    d = 64 (c / 4) + 4 i + c % 4, again a 16-byte load as it stands.  The accumulator c,
//                    register r of lane (head j, kb) is O[head][64 (c / 4) + 16 kb + 4 r + c % 4].
// Two tiles per wave are in flight (all their loads issued before any arithmetic); the four waves of a block
// merge through LDS, the splits through attn_combine_kernel, as in the kernel above.
typedef float v4f __attribute__((ext_vector_type(4)));

template <int QG>
__global__ __launch_bounds__(256, 2) void attn_decode_mfma_kernel(const AttnDecode A) {
    constexpr int NWV = 4, NT = 256, TK = 16;
    constexpr int HS = 128, HALF = 64;
    static_assert(QG == 4 || QG == 8, "the query heads of a kv head fill part of the 16 columns of a tile");
    __shared__ float qs[QG * HS];
    __shared__ float kvnew[2][HS];
    __shared__ __align__(16) float comb[NWV][QG][kCombRow];
    pin_args(A);
    const int kvh = blockIdx.x, sp = blockIdx.y;
    const int pos = A.dpos ? A.dpos[0] : A.pos;
    const int t0 = sp * A.ts;
    if (t0 > pos) return;
    const int t1 = min(t0 + A.ts, pos + 1);
    const int n = t1 - t0;
    const int kv_dim = A.n_kv_heads * HS;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, kb = lane >> 4;

    const float *__restrict__ kc = A.kcache;
    const float *__restrict__ vc = A.vcache;
    const uint32_t row_bytes = (uint32_t)kv_dim * 4u;
    const int t_last = t1 - 1;
    const uint32_t k_lane = (uint32_t)(kvh * HS + 4 * kb) * 4u; // + 64 m bytes
    const uint32_t v_lane = (uint32_t)(kvh * HS + 4 * li) * 4u; // + 256 bytes for the second half of d

    struct Tile {
        float4 k[8]; // k[m]: K[t = li][16 m + 4 kb ..]
        float4 v[8]; // v[2 r + half]: V[t = 4 kb + r][64 half + 4 li ..]
    };
    // Unconditional loads: rows past the end re-read the last row (masked below).
    auto fetch = [&](int tile, Tile &d) {
        const int tb = t0 + tile * TK;
        const uint32_t ko = __umul24(min(tb + li, t_last), row_bytes) + k_lane;
#pragma unroll
        for (int m = 0; m < 8; m++) d.k[m] = ld_at<float4>(kc, ko + 64u * m);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t vo = __umul24(min(tb + 4 * kb + r, t_last), row_bytes) + v_lane;
            d.v[2 * r] = ld_at<float4>(vc, vo);
            d.v[2 * r + 1] = ld_at<float4>(vc, vo + 256u);
        }
    };
    // The small loads that the staging needs go out first (loads return in order).
    const float *ct = A.cos_t + (size_t)pos * HALF;
    const float *st = A.sin_t + (size_t)pos * HALF;
    constexpr int NQ = (QG * HALF + NT - 1) / NT;
    float qa[NQ], qb[NQ], qc[NQ], qsn[NQ];
#pragma unroll
    for (int r = 0; r < NQ; r++) {
        const int idx = (tid + r * NT) % (QG * HALF);
        const int j = idx >> 6, i = idx & 63;
        const float *qh = A.q + (size_t)(kvh * QG + j) * HS;
        qa[r] = qh[i], qb[r] = qh[i + HALF];
        qc[r] = ct[i], qsn[r] = st[i];
    }
    // where this thread's outputs go when the step is not split: fetched now, used at the very end
    int sdst[QG * HS / NT];
#pragma unroll
    for (int u = 0; u < QG * HS / NT; u++) {
        const int i = kvh * QG * HS + tid + u * NT;
        sdst[u] = (A.scatter && A.n_splits == 1) ? A.scatter[i] : i;
    }
    const int hd = tid & 63;
    const float nk_a = A.k_new[(size_t)kvh * HS + hd], nk_b = A.k_new[(size_t)kvh * HS + hd + HALF];
    const float nv = A.v_new[(size_t)kvh * HS + (tid & 127)];
    const float nc = ct[hd], ns = st[hd];
    __builtin_amdgcn_sched_barrier(0);

    const int n_tiles = (n + TK - 1) / TK;
    Tile ta, tb2;
    fetch(wave, ta);
    fetch(wave + NWV, tb2);
    __builtin_amdgcn_sched_barrier(0);

    // q with RoPE, src/models.rs:100-129 (the second half uses the rotated first half)
#pragma unroll
    for (int r = 0; r < NQ; r++) {
        const int idx = (tid + r * NT) % (QG * HALF);
        const int j = idx >> 6, i = idx & 63;
        const float first = qa[r] * qc[r] - qb[r] * qsn[r];
        qs[j * HS + i] = first;
        qs[j * HS + HALF + i] = qb[r] * qc[r] + first * qsn[r];
    }
    // the new key, rotated, and the new value; the block whose range ends at pos also writes them to the
    // cache (:236-249)
    const bool owns_new = (t1 == pos + 1);
    {
        const float first = nk_a * nc - nk_b * ns;
        const float second = nk_b * nc + first * ns;
        kvnew[0][hd] = first;
        kvnew[0][hd + HALF] = second;
        kvnew[1][tid & 127] = nv;
        if (owns_new) {
            if (tid < HALF) {
                float *kw = A.kcache + (size_t)pos * kv_dim + kvh * HS;
                kw[tid] = first;
                kw[tid + HALF] = second;
            } else if (tid >= 128 && tid < 256) {
                A.vcache[(size_t)pos * kv_dim + kvh * HS + (tid - 128)] = nv;
            }
        }
    }
    __syncthreads();

    // B operands of the score MFMAs: this lane's head (columns beyond the QG heads are zero)
    float4 qf[8];
#pragma unroll
    for (int m = 0; m < 8; m++)
        qf[m] = li < QG ? *reinterpret_cast<const float4 *>(&qs[li * HS + 16 * m + 4 * kb]) : make_float4(0.f, 0.f, 0.f, 0.f);

    float m_run = kNoScore, l = 0.f;
    v4f acc[8];
#pragma unroll
    for (int c = 0; c < 8; c++) acc[c] = v4f{0.f, 0.f, 0.f, 0.f};
    // log2(e) / sqrt(head_size): src/models.rs:154 divides the score by sqrt(head_size)
    const float scale = 1.44269504088896340736f / sqrtf((float)HS);

    auto tile_math = [&](int tile, Tile &d) __attribute__((always_inline)) {
        const int tb = t0 + tile * TK;
        if (tb <= pos && pos < tb + TK) { // once per step: the row of the new position comes from LDS, not from the cache
            if (tb + li == pos) {
#pragma unroll
                for (int m = 0; m < 8; m++) d.k[m] = *reinterpret_cast<const float4 *>(&kvnew[0][16 * m + 4 * kb]);
            }
#pragma unroll
            for (int r = 0; r < 4; r++)
                if (tb + 4 * kb + r == pos) {
                    d.v[2 * r] = *reinterpret_cast<const float4 *>(&kvnew[1][4 * li]);
                    d.v[2 * r + 1] = *reinterpret_cast<const float4 *>(&kvnew[1][HALF + 4 * li]);
                }
        }
        // scores: two accumulators, so that consecutive MFMAs do not wait for each other
        v4f s0 = v4f{0.f, 0.f, 0.f, 0.f}, s1 = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].x, qf[m].x, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].x, qf[m + 1].x, s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].y, qf[m].y, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].y, qf[m + 1].y, s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].z, qf[m].z, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].z, qf[m + 1].z, s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].w, qf[m].w, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].w, qf[m + 1].w, s1, 0, 0, 0);
        }
        float sc[4], p[4];
        float mx = kNoScore;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool valid = tb + 4 * kb + r <= t_last;
            sc[r] = valid ? (s0[r] + s1[r]) * scale : kNoScore;
            mx = fmaxf(mx, sc[r]);
        }
        if (__any(mx > m_run)) { // some head's maximum moves: agree on it among the head's four lanes, rescale
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            const float c = exp2_fast(m_run - m_new);
            l *= c;
#pragma unroll
            for (int cc = 0; cc < 8; cc++) acc[cc] *= c;
            m_run = m_new;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool valid = tb + 4 * kb + r <= t_last;
            p[r] = valid ? exp2_fast(sc[r] - m_run) : 0.f;
            l += p[r];
        }
        // weighted sums: eight independent accumulators
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float4 v0 = d.v[2 * r], v1 = d.v[2 * r + 1];
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.x, p[r], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.y, p[r], acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.z, p[r], acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.w, p[r], acc[3], 0, 0, 0);
            acc[4] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.x, p[r], acc[4], 0, 0, 0);
            acc[5] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.y, p[r], acc[5], 0, 0, 0);
            acc[6] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.z, p[r], acc[6], 0, 0, 0);
            acc[7] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.w, p[r], acc[7], 0, 0, 0);
        }
    };
    // Tiles wave, wave + 4, ...: two buffers, each refilled right after its tile is done when the wave has a
    // further tile for it (a uniform branch; up to two tiles per wave, the usual case behind a long cache,
    // nothing is refilled).
    for (int tile = wave; tile < n_tiles; tile += 2 * NWV) {
        tile_math(tile, ta);
        if (tile + 2 * NWV < n_tiles) fetch(tile + 2 * NWV, ta);
        if (tile + NWV < n_tiles) {
            tile_math(tile + NWV, tb2);
            if (tile + 3 * NWV < n_tiles) fetch(tile + 3 * NWV, tb2);
        }
    }

    // this wave's (m, l, O) -> LDS.  The head's four lanes hold disjoint d: lane (j, kb), accumulators 0..3,
    // register r are d = 16 kb + 4 r + 0..3, accumulators 4..7 the same 64 further on.
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (li < QG) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            *reinterpret_cast<float4 *>(&comb[wave][li][16 * kb + 4 * r]) = make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
            *reinterpret_cast<float4 *>(&comb[wave][li][HALF + 16 * kb + 4 * r]) =
                make_float4(acc[4][r], acc[5][r], acc[6][r], acc[7][r]);
        }
        if (kb == 0) {
            comb[wave][li][HS] = m_run;
            comb[wave][li][HS + 1] = l;
        }
    }
    __syncthreads();
    // merge the four waves; one thread per (head, dim), the passes unrolled so that their LDS reads overlap
    constexpr int NP = QG * HS / NT;
    float num[NP], den[NP], Mx[NP];
#pragma unroll
    for (int u = 0; u < NP; u++) {
        const int idx = tid + u * NT;
        const int j = idx >> 7, d = idx & 127;
        float M = comb[0][j][HS];
#pragma unroll
        for (int w = 1; w < NWV; w++) M = fmaxf(M, comb[w][j][HS]);
        float nu = 0.f, de = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; w++) {
            const float e = exp2_fast(comb[w][j][HS] - M);
            nu = fmaf(e, comb[w][j][d], nu);
            de = fmaf(e, comb[w][j][HS + 1], de);
        }
        num[u] = nu, den[u] = de, Mx[u] = M;
    }
#pragma unroll
    for (int u = 0; u < NP; u++) {
        const int idx = tid + u * NT;
        const int j = idx >> 7, d = idx & 127;
        const int h = kvh * QG + j;
        if (A.n_splits == 1) {
            A.out[sdst[u]] = num[u] / den[u];
        } else {
            float *pp = A.part + ((size_t)h * A.max_splits + sp) * (HS + 2);
            pp[d] = num[u];
            if (d == 0) {
                pp[HS] = Mx[u];
                pp[HS + 1] = den[u];
            }
        }
    }
}

// Attention for a chunk of B positions (prefill, src/models.rs:131-176 with B > 1).  Every cache row of
// the chunk is already written and q already rotated (rope_kv_kernel).  The same layout as the decode
// kernel, with the 8 "heads" of a block being 8 / QG query positions x the QG query heads of one kv head:
// the K and V rows a block streams are shared by 8 score/value streams instead of being re-read per query.
// Query j sees timesteps 0..pos[j] (causal within the chunk as well).
template <int QG>
__global__ __launch_bounds__(256) void attn_prefill_kernel(float *__restrict__ out, _Float16 *__restrict__ out_h,
                                                            const float *__restrict__ q,
                                                            const float *__restrict__ kc, const float *__restrict__ vc,
                                                            const int32_t *__restrict__ pos,
                                                            const int32_t *__restrict__ scatter, int n_heads,
                                                            int n_kv_heads, int B) {
    constexpr int HS = 128, NQ = 8, QPB = NQ / QG, PD = 2, TSTEP = 16;
    __shared__ float qs[NQ * HS];
    __shared__ __align__(16) float comb[4][NQ][kCombRow];
    __shared__ int pj_s[NQ];
    const int kvh = blockIdx.x, qb = blockIdx.y;
    const int dim = n_heads * HS, kv_dim = n_kv_heads * HS;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int ds = lane & 15;
    const int tl = wave * 4 + (lane >> 4);
    // stream j: query qb * QPB + j / QG, head kvh * QG + j % QG
    if (tid < NQ) {
        const int qi = qb * QPB + tid / QG;
        pj_s[tid] = qi < B ? pos[qi] : -1;
    }
    for (int idx = tid; idx < NQ * HS; idx += 256) {
        const int j = idx >> 7, d = idx & 127;
        const int qi = min(qb * QPB + j / QG, B - 1);
        qs[idx] = q[(size_t)qi * dim + (kvh * QG + j % QG) * HS + d];
    }
    __syncthreads();
    int pj[NQ];
    int t_end = 0; // one past the last timestep any stream of the block sees
#pragma unroll
    for (int j = 0; j < NQ; j++) {
        pj[j] = pj_s[j];
        t_end = max(t_end, pj[j] + 1);
    }
    if (t_end == 0) return;
    const uint32_t row_bytes = (uint32_t)kv_dim * 4u;
    const uint32_t lane_off = (uint32_t)(kvh * HS + ds * 8) * 4u;
    struct Step {
        float4 k0, k1, v0, v1;
    };
    auto fetch = [&](int it, Step &d) {
        const int t = min(it * TSTEP + tl, t_end - 1);
        const uint32_t off = __umul24(t, row_bytes) + lane_off;
        d.k0 = ld_at<float4>(kc, off);
        d.k1 = ld_at<float4>(kc, off + 16);
        d.v0 = ld_at<float4>(vc, off);
        d.v1 = ld_at<float4>(vc, off + 16);
    };
    float m[NQ], l[NQ], acc[NQ][8];
#pragma unroll
    for (int j = 0; j < NQ; j++) {
        m[j] = kNoScore;
        l[j] = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) acc[j][e] = 0.f;
    }
    const float scale = 1.44269504088896340736f / sqrtf((float)HS);
    const int n_it = (t_end + TSTEP - 1) / TSTEP;
    const int n_tiles = (n_it + PD - 1) / PD;
    Step pipe[PD];
    for (int tile = 0; tile < n_tiles; tile++) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PD; u++) fetch(tile * PD + u, pipe[u]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < PD; u++) {
            const int t = (tile * PD + u) * TSTEP + tl;
            const Step &d = pipe[u];
            const float k[8] = {d.k0.x, d.k0.y, d.k0.z, d.k0.w, d.k1.x, d.k1.y, d.k1.z, d.k1.w};
            float v[8] = {d.v0.x, d.v0.y, d.v0.z, d.v0.w, d.v1.x, d.v1.y, d.v1.z, d.v1.w};
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = t < t_end ? v[e] : 0.f; // rows past the end may hold anything
            float sc[NQ];
            bool grow = false;
#pragma unroll
            for (int j = 0; j < NQ; j++) {
                const float4 a = *reinterpret_cast<const float4 *>(&qs[j * HS + ds * 8]);
                const float4 b = *reinterpret_cast<const float4 *>(&qs[j * HS + ds * 8 + 4]);
                const float qj[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
                float s = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) s = fmaf(qj[e], k[e], s);
                s += dpp_xchg<0xB1>(s);
                s += dpp_xchg<0x4E>(s);
                s += dpp_xchg<0x141>(s);
                s += dpp_xchg<0x140>(s);
                s = t <= pj[j] ? s * scale : kNoScore;
                sc[j] = s;
                grow |= s > m[j];
            }
            if (__any(grow)) {
#pragma unroll
                for (int j = 0; j < NQ; j++) {
                    const float m_new = fmaxf(m[j], sc[j]);
                    const float c = exp2_fast(m[j] - m_new);
                    l[j] *= c;
#pragma unroll
                    for (int e = 0; e < 8; e++) acc[j][e] *= c;
                    m[j] = m_new;
                }
            }
#pragma unroll
            for (int j = 0; j < NQ; j++) {
                const float p = t <= pj[j] ? exp2_fast(sc[j] - m[j]) : 0.f;
                l[j] += p;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[j][e] = fmaf(p, v[e], acc[j][e]);
            }
        }
    }
#pragma unroll
    for (int step = 16; step <= 32; step *= 2) {
#pragma unroll
        for (int j = 0; j < NQ; j++) {
            const float mo = __shfl_xor(m[j], step);
            const float lo = __shfl_xor(l[j], step);
            const float M = fmaxf(m[j], mo);
            const float w1 = exp2_fast(m[j] - M), w2 = exp2_fast(mo - M);
            l[j] = l[j] * w1 + lo * w2;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float ao = __shfl_xor(acc[j][e], step);
                acc[j][e] = acc[j][e] * w1 + ao * w2;
            }
            m[j] = M;
        }
    }
    if (lane < 16) {
#pragma unroll
        for (int j = 0; j < NQ; j++) {
            *reinterpret_cast<float4 *>(&comb[wave][j][ds * 8]) = make_float4(acc[j][0], acc[j][1], acc[j][2], acc[j][3]);
            *reinterpret_cast<float4 *>(&comb[wave][j][ds * 8 + 4]) =
                make_float4(acc[j][4], acc[j][5], acc[j][6], acc[j][7]);
            if (ds == 0) {
                comb[wave][j][HS] = m[j];
                comb[wave][j][HS + 1] = l[j];
            }
        }
    }
    __syncthreads();
    for (int idx = tid; idx < NQ * HS; idx += 256) {
        const int j = idx >> 7, d = idx & 127;
        const int qi = qb * QPB + j / QG;
        if (qi >= B) continue;
        float M = comb[0][j][HS];
#pragma unroll
        for (int w = 1; w < 4; w++) M = fmaxf(M, comb[w][j][HS]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float e = exp2_fast(comb[w][j][HS] - M);
            num = fmaf(e, comb[w][j][d], num);
            den = fmaf(e, comb[w][j][HS + 1], den);
        }
        const int i = (kvh * QG + j % QG) * HS + d;
        const int dst = scatter ? scatter[i] : i;
        if (out_h) // straight into the fp16 pair-interleaved order the next GEMM reads
            out_h[(size_t)qi * dim + h16_slot(dst)] = (_Float16)(num / den);
        else
            out[(size_t)qi * dim + dst] = num / den;
    }
}

// Chunk attention on the matrix cores, all in fp32 (v_mfma_f32_16x16x4_f32), for the prefill mode that hands fp16
// activations to the next GEMM.  Same function as attn_prefill_kernel (src/models.rs:131-176, causal per query over
// the cache rows 0..pos), in the layout of attn_decode_mfma_kernel: a block owns 16 columns of one kv head, column
// n = (query ct*16/QG + n/QG, head kvh*QG + n%QG), its NWV waves take the tiles of 16 cache rows w, w + NWV, ...
// and merge through LDS at the end.  With lane = (i = lane % 16, kb = lane / 16):
//   S^T = K Q^T      A: lane (row i, kb) holds K[t][16 m + 4 kb + e] -- what a 16-byte load of the cache row leaves
//                    in the lane; B: lane (column i, kb) holds Q[column][16 m + 4 kb + e], eight 16-byte loads of
//                    the query's row, kept for the whole kernel.  Nothing passes through LDS on the way.
//   C layout         lane (column j, kb), register r -> row 4 kb + r: the lane masks the rows behind ITS column's
//                    position (causal per query); the four lanes of a column share its running maximum.
//   O^T += V^T P^T   contracts over the lane's own registers of P; A is a 16-byte load of the V row as it stands.
// 128 tokens of a 32-head model are 256 blocks, one per compute unit.  (A form on 32 columns and tiles of 32 rows,
// v_mfma_f32_32x32x2_f32 with K and V turned through LDS, had half the blocks and took 16 to 31 us per chunk of a
// 512-token prompt where this one takes 11 to 19.)
template <int QG, int NWV>
__global__ __launch_bounds__(NWV * 64, NWV == 4 ? 2 : 1)
void attn_prefill_mfma16_kernel(_Float16 *__restrict__ out_h, const float *__restrict__ q, const float *__restrict__ kc,
                                const float *__restrict__ vc, const int32_t *__restrict__ pos,
                                const int32_t *__restrict__ scatter, int n_heads, int n_kv_heads, int B, int max_pos) {
    constexpr int NT = NWV * 64, TK = 16, HS = 128, HALF = 64, NC = 16, QPT = NC / QG;
    __shared__ __align__(16) float comb[NWV][NC][kCombRow];
    // the last columns of a chunk see the most cache rows: their blocks are dispatched first
    const int kvh = blockIdx.x, ct = gridDim.y - 1 - blockIdx.y;
    const int dim = n_heads * HS, kv_dim = n_kv_heads * HS;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int li = lane & 15, kb = lane >> 4;
    const uint32_t row_bytes = (uint32_t)kv_dim * 4u;
    const uint32_t k_lane = (uint32_t)(kvh * HS + 4 * kb) * 4u; // + 64 m bytes
    const uint32_t v_lane = (uint32_t)(kvh * HS + 4 * li) * 4u; // + 256 bytes for the second half of d

    struct Tile {
        float4 k[8]; // k[m]: K[t = li][16 m + 4 kb ..]
        float4 v[8]; // v[2 r + half]: V[t = 4 kb + r][64 half + 4 li ..]
    };
    // Unconditional loads: rows past the last one written re-read it (masked below).
    auto fetch = [&](int tile, Tile &d) {
        const int tb = tile * TK;
        const uint32_t ko = __umul24(min(tb + li, max_pos), row_bytes) + k_lane;
#pragma unroll
        for (int m = 0; m < 8; m++) d.k[m] = ld_at<float4>(kc, ko + 64u * m);
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const uint32_t vo = __umul24(min(tb + 4 * kb + r, max_pos), row_bytes) + v_lane;
            d.v[2 * r] = ld_at<float4>(vc, vo);
            d.v[2 * r + 1] = ld_at<float4>(vc, vo + 256u);
        }
    };
    // this lane's column: its query, its position, its B operands
    const int my_qi = ct * QPT + li / QG;
    const int my_pos = my_qi < B ? pos[my_qi] : -1;
    const float *qrow = q + (size_t)min(my_qi, B - 1) * dim + (size_t)(kvh * QG + li % QG) * HS + 4 * kb;
    float4 qf[8];
#pragma unroll
    for (int m = 0; m < 8; m++) qf[m] = *reinterpret_cast<const float4 *>(qrow + 16 * m);
    Tile ta, tb2;
    fetch(wave, ta);
    fetch(wave + NWV, tb2);
    __builtin_amdgcn_sched_barrier(0);
    int t_end = my_pos + 1; // the block's tiles end with the last row any of its columns sees
#pragma unroll
    for (int off = 8; off > 0; off >>= 1) t_end = max(t_end, __shfl_xor(t_end, off));
    t_end = __builtin_amdgcn_readfirstlane(t_end);
    const int n_tiles = (t_end + TK - 1) / TK;

    float m_run = kNoScore, l = 0.f;
    v4f acc[8];
#pragma unroll
    for (int c = 0; c < 8; c++) acc[c] = v4f{0.f, 0.f, 0.f, 0.f};
    const float scale = 1.44269504088896340736f / sqrtf((float)HS); // log2(e) / sqrt(head_size), src/models.rs:154

    auto tile_math = [&](int tile, Tile &d) __attribute__((always_inline)) {
        const int tb = tile * TK;
        v4f s0 = v4f{0.f, 0.f, 0.f, 0.f}, s1 = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int m = 0; m < 8; m += 2) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].x, qf[m].x, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].x, qf[m + 1].x, s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].y, qf[m].y, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].y, qf[m + 1].y, s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].z, qf[m].z, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].z, qf[m + 1].z, s1, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m].w, qf[m].w, s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(d.k[m + 1].w, qf[m + 1].w, s1, 0, 0, 0);
        }
        float sc[4], p[4];
        float mx = kNoScore;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool valid = tb + 4 * kb + r <= my_pos; // causal: this column's query sees rows 0..pos
            sc[r] = valid ? (s0[r] + s1[r]) * scale : kNoScore;
            mx = fmaxf(mx, sc[r]);
        }
        if (__any(mx > m_run)) { // some column's maximum moves: agree on it among the column's four lanes, rescale
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m_run, mx);
            const float c = exp2_fast(m_run - m_new);
            l *= c;
#pragma unroll
            for (int cc = 0; cc < 8; cc++) acc[cc] *= c;
            m_run = m_new;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const bool valid = tb + 4 * kb + r <= my_pos;
            p[r] = valid ? exp2_fast(sc[r] - m_run) : 0.f;
            l += p[r];
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float4 v0 = d.v[2 * r], v1 = d.v[2 * r + 1];
            acc[0] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.x, p[r], acc[0], 0, 0, 0);
            acc[1] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.y, p[r], acc[1], 0, 0, 0);
            acc[2] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.z, p[r], acc[2], 0, 0, 0);
            acc[3] = __builtin_amdgcn_mfma_f32_16x16x4f32(v0.w, p[r], acc[3], 0, 0, 0);
            acc[4] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.x, p[r], acc[4], 0, 0, 0);
            acc[5] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.y, p[r], acc[5], 0, 0, 0);
            acc[6] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.z, p[r], acc[6], 0, 0, 0);
            acc[7] = __builtin_amdgcn_mfma_f32_16x16x4f32(v1.w, p[r], acc[7], 0, 0, 0);
        }
    };
    // two buffers, each refilled right after its tile is done when the wave has a further tile for it (uniform)
    for (int tile = wave; tile < n_tiles; tile += 2 * NWV) {
        tile_math(tile, ta);
        if (tile + 2 * NWV < n_tiles) fetch(tile + 2 * NWV, ta);
        if (tile + NWV < n_tiles) {
            tile_math(tile + NWV, tb2);
            if (tile + 3 * NWV < n_tiles) fetch(tile + 3 * NWV, tb2);
        }
    }

    // this wave's (m, l, O) -> LDS: lane (column j, kb), accumulators 0..3, register r are d = 16 kb + 4 r + 0..3,
    // accumulators 4..7 the same 64 further on
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
#pragma unroll
    for (int r = 0; r < 4; r++) {
        *reinterpret_cast<float4 *>(&comb[wave][li][16 * kb + 4 * r]) = make_float4(acc[0][r], acc[1][r], acc[2][r], acc[3][r]);
        *reinterpret_cast<float4 *>(&comb[wave][li][HALF + 16 * kb + 4 * r]) =
            make_float4(acc[4][r], acc[5][r], acc[6][r], acc[7][r]);
    }
    if (kb == 0) {
        comb[wave][li][HS] = m_run;
        comb[wave][li][HS + 1] = l;
    }
    __syncthreads();
    // merge the waves; a thread owns 8 consecutive d of one column, so that what it stores is one 16-byte piece of
    // the fp16 pair-interleaved row when the consumer's order keeps those 8 together, and 8 two-byte stores otherwise
    constexpr int NP = NC * HS / NT; // outputs per thread
#pragma unroll
    for (int u = 0; u < NP; u++) {
        const int idx = tid + u * NT;
        const int j = idx >> 7, d = idx & 127;
        const int qi = ct * QPT + j / QG;
        float M = comb[0][j][HS];
#pragma unroll
        for (int w = 1; w < NWV; w++) M = fmaxf(M, comb[w][j][HS]);
        float nu = 0.f, de = 0.f;
#pragma unroll
        for (int w = 0; w < NWV; w++) {
            const float e = exp2_fast(comb[w][j][HS] - M);
            nu = fmaf(e, comb[w][j][d], nu);
            de = fmaf(e, comb[w][j][HS + 1], de);
        }
        if (qi < B) {
            const int i = (kvh * QG + j % QG) * HS + d;
            const int dst = scatter ? scatter[i] : i;
            out_h[(size_t)qi * dim + h16_slot(dst)] = (_Float16)(nu / de); // the order the next GEMM reads
        }
    }
}

// Merge the splits of one q head: out = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s.
// Every load goes out before anything is waited for (the partial outputs of this thread's splits, the
// (m_s, l_s) pairs, the scatter target: one round trip to memory instead of three); wave 0 then turns the
// (m_s, l_s) of up to 64 splits into weights and 4 groups of 128 threads sum the weighted partial outputs.
__global__ __launch_bounds__(512) void attn_combine_kernel(const AttnDecode A) {
    constexpr int HS = 128, NU = 16; // splits per thread: 64 over 4 groups
    pin_args(A);
    __shared__ float w[64];
    __shared__ float den_s;
    __shared__ float red[3][HS];
    const int h = blockIdx.x, tid = threadIdx.x, d = tid & 127, grp = tid >> 7;
    const int pos = A.dpos ? A.dpos[0] : A.pos;
    const int ns = min(A.n_splits, pos / A.ts + 1);
    const float *p = A.part + (size_t)h * A.max_splits * (HS + 2);
    float pv[NU];
#pragma unroll
    for (int u = 0; u < NU; u++) pv[u] = p[min(grp + 4 * u, ns - 1) * (HS + 2) + d]; // past the end: the last split again, unused
    const int i = h * HS + d;
    const int dst = A.scatter ? A.scatter[i] : i;
    const int sl = min(tid & 63, ns - 1);
    const float ms_r = p[sl * (HS + 2) + HS], ls_r = p[sl * (HS + 2) + HS + 1];
    if (tid < 64) {
        const bool on = tid < ns;
        const float ms = on ? ms_r : kNoScore;
        const float ls = on ? ls_r : 0.f;
        const float M = wave_max(ms);
        const float ws = on ? exp2_fast(ms - M) : 0.f;
        w[tid] = ws;
        const float den = wave_sum(ws * ls);
        if (tid == 0) den_s = den;
    }
    __syncthreads();
    float num = 0.f;
#pragma unroll
    for (int u = 0; u < NU; u++) num = fmaf(w[grp + 4 * u], pv[u], num); // w is 0 beyond the last split
    if (grp > 0) red[grp - 1][d] = num;
    __syncthreads();
    if (grp == 0) {
        num += red[0][d];
        num += red[1][d];
        num += red[2][d];
        A.out[dst] = num / den_s;
    }
}

template <int QG>
int attn_launch_qg(const AttnDecode &a, hipStream_t st) {
    if constexpr (QG >= 4) {
        static const bool valu = []() {
            const char *v = getenv("L2_ATTN_IMPL");
            return v && !strcmp(v, "valu");
        }();
        if (!valu) {
            hipLaunchKernelGGL((attn_decode_mfma_kernel<QG>), dim3(a.n_kv_heads, a.n_splits), dim3(256), 0, st, a);
            L2_HIP(hipGetLastError());
            return L2_OK;
        }
    }
    constexpr size_t lds = QG >= 4 ? (size_t)16 * QG * kCombRow * sizeof(float) : 0; // the partial results of 16 rows
    if (lds > 48 * 1024) {
        static LdsLimit limit; // per instantiation
        L2_TRY(limit.ensure(reinterpret_cast<const void *>(attn_decode_kernel<QG, 4>), lds));
    }
    hipLaunchKernelGGL((attn_decode_kernel<QG, 4>), dim3(a.n_kv_heads, a.n_splits), dim3(256), lds, st, a);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

} // namespace

int attention_decode_launch(const AttnDecode &a, hipStream_t st) {
    const int qg = a.n_heads / a.n_kv_heads;
    if (a.ts < 64 || a.ts % 64 || a.n_splits < 1 || a.n_splits > a.max_splits || a.max_splits > 64)
        return l2_fail(L2_ERR_ARG, "attention: ts=%d splits=%d/%d", a.ts, a.n_splits, a.max_splits);
    switch (qg) {
        case 1: L2_TRY(attn_launch_qg<1>(a, st)); break;
        case 2: L2_TRY(attn_launch_qg<2>(a, st)); break;
        case 4: L2_TRY(attn_launch_qg<4>(a, st)); break;
        case 8: L2_TRY(attn_launch_qg<8>(a, st)); break;
        default: return l2_fail(L2_ERR_ARG, "attention: %d query heads per kv head (1, 2, 4 or 8)", qg);
    }
    if (a.n_splits > 1) {
        hipLaunchKernelGGL(attn_combine_kernel, dim3(a.n_heads), dim3(512), 0, st, a);
        L2_HIP(hipGetLastError());
    }
    return L2_OK;
}

int attention_launch(float *out, void *out_f16, const float *q, const float *kcache_l, const float *vcache_l,
                     const int32_t *pos, const int32_t *scatter, int n_heads, int n_kv_heads,
                     int head_size, int max_pos, int B, hipStream_t st) {
    if (head_size != 128) return l2_fail(L2_ERR_ARG, "attention: head_size=%d (128 only)", head_size);
    const int qg = n_heads / n_kv_heads;
    if (qg != 1 && qg != 2 && qg != 4 && qg != 8)
        return l2_fail(L2_ERR_ARG, "attention: %d query heads per kv head (1, 2, 4 or 8)", qg);
    if (out_f16) { // the matrix-core form: 16 columns (queries x heads of the group) per block
        dim3 grid(n_kv_heads, (B * qg + 15) / 16), block(256);
        switch (qg) {
            case 1: hipLaunchKernelGGL((attn_prefill_mfma16_kernel<1, 4>), grid, block, 0, st, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B, max_pos); break;
            case 2: hipLaunchKernelGGL((attn_prefill_mfma16_kernel<2, 4>), grid, block, 0, st, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B, max_pos); break;
            case 4: hipLaunchKernelGGL((attn_prefill_mfma16_kernel<4, 4>), grid, block, 0, st, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B, max_pos); break;
            default: hipLaunchKernelGGL((attn_prefill_mfma16_kernel<8, 4>), grid, block, 0, st, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B, max_pos); break;
        }
        L2_HIP(hipGetLastError());
        return L2_OK;
    }
    const int qpb = 8 / qg;
    dim3 grid(n_kv_heads, (B + qpb - 1) / qpb), block(256);
    switch (qg) {
        case 1: hipLaunchKernelGGL(attn_prefill_kernel<1>, grid, block, 0, st, out, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B); break;
        case 2: hipLaunchKernelGGL(attn_prefill_kernel<2>, grid, block, 0, st, out, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B); break;
        case 4: hipLaunchKernelGGL(attn_prefill_kernel<4>, grid, block, 0, st, out, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B); break;
        default: hipLaunchKernelGGL(attn_prefill_kernel<8>, grid, block, 0, st, out, (_Float16 *)out_f16, q, kcache_l, vcache_l, pos, scatter, n_heads, n_kv_heads, B); break;
    }
    L2_HIP(hipGetLastError());
    return L2_OK;
}
