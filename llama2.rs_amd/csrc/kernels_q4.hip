// GPTQ 4-bit dequant matvec for gfx950 (wave64), with the neighbouring
// element-wise steps of the decode schedule folded into its two ends.
//
// Computes, per output row o and batch column b (QLinear::matvec,
// src/gptq.rs:94-176, in exact arithmetic):
//   y[b][o] = sum_j scales[o][j/G] * (nib(qweight[o], j) - (nib(qzeros[o/8][j/G], o%8) + 1)) * xg[b][j]
// where xg is the input already gathered through g_index by its producer.
//
// Mapping.  The `.bin` layout keeps the IN/8 packed words of one output row
// contiguous, so a wave reads a row with 128-bit loads, lane l taking chunk
// c = l, l+64, ... (one chunk = 4 words = 32 nibbles = 32 consecutive K).  A
// chunk never straddles a group (G is a multiple of 32).  The block stages the
// gathered input once in LDS, each chunk padded to 36 floats so that the
// 128-bit LDS reads of 64 lanes hit distinct banks, together with the sum of
// each chunk.  A wave keeps R rows in flight against one chunk of x held in
// registers, so LDS traffic per weight byte falls with R.
//
// Arithmetic.  The zero point is factored out of the inner loop:
//   sum_{j in chunk} s (n_j - z) x_j = s * (sum n_j x_j - z * sum x_j)
// Nibbles are turned into floats two at a time by v_cvt_pk_f32_fp8 (see
// chunk_dot), so one nibble costs half a convert, one FMA and 3/8 of a mask
// operation.  All accumulation is fp32; the reduction order is fixed (no
// atomics), so results are bit-stable from run to run.
//
// Prologue (optional): rmsnorm (src/models.rs:53-66).  The input buffer then
// holds the raw residual stream in this layer's g_index order and `wn` the norm
// weights in the same order; the block stages wn[j]*x[j], sums x^2 on the way,
// and applies ss = 1/sqrt(mean + eps) once per output row (W(ss v) = ss W v).
//
// Epilogues: plain store; residual add (src/models.rs:263-264, 283-285) that
// also delivers the new residual stream in the input order of up to three
// following layers; SiLU gate over a (w1, w3) pair of rows
// (src/models.rs:271-276) delivered in w2's input order.
#include <string.h>

#include <stdio.h>

#include "q4_common.h"

namespace {

using namespace q4;

struct RowLoad {
    uint4 w;
    float s;
};

// G: group size, R: rows per wave (per matrix), NW: waves per block,
// PAIR: the block walks rows of m[0] and m[1] together (SiLU gate).
template <int G, int R, int NW, bool PAIR>
__global__ __launch_bounds__(NW * 64) void q4_matvec_kernel(const Q4Launch L) {
    extern __shared__ float lds[];
    constexpr int NM = PAIR ? 2 : 1;
    const int in = L.in;
    const int C = in >> 5;                 // chunks per row
    const int xstride = C * kChunkPad + C; // floats per staged vector: [C][36] then [C] sums
    __shared__ float red[NW];

    // which matrix, which rows
    int rb = blockIdx.x;
    int mi = 0;
    if (!PAIR) {
        while (mi + 1 < L.n_mats && rb >= L.m[mi].row_blocks) {
            rb -= L.m[mi].row_blocks;
            mi++;
        }
    }
    const int b = blockIdx.y;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int n_out = L.m[mi].out;
    const int o0 = (rb * NW + wave) * R; // first row of this wave; multiple of R
    const bool active = o0 < n_out;
    const int groups = L.groups;
    constexpr int CPG = G / 32; // chunks per group

    // First chunk's weights are requested before anything else so that the HBM
    // latency overlaps with staging x.
    RowLoad cur[NM][R];
    int32_t zcur[NM];
    int c = lane;
    if (active && c < C) {
        const int g = c / CPG;
#pragma unroll
        for (int q = 0; q < NM; q++) {
            const Q4Mat &M = L.m[mi + q];
            zcur[q] = M.qzeros[(size_t)(o0 >> 3) * groups + g];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int o = min(o0 + r, n_out - 1);
                cur[q][r].w = M.qweight[(size_t)o * C + c];
                cur[q][r].s = M.scales[(size_t)o * groups + g];
            }
        }
    }

    float ssq = 0.f;
#pragma unroll
    for (int q = 0; q < NM; q++) {
        const Q4Mat &M = L.m[mi + q];
        const float part = stage_input<NW>(M.x + (size_t)b * in, M.wn, in, lds + q * xstride,
                                           lds + q * xstride + C * kChunkPad, tid);
        if (q == 0) ssq = part;
    }
    const bool norm = L.m[mi].wn != nullptr;
    if (norm) {
        ssq = wave_sum(ssq);
        if (lane == 0) red[wave] = ssq;
    }
    __syncthreads();
    if (!active) return;
    float ss = 1.0f;
    if (norm) { // rmsnorm scale, src/models.rs:55-60
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < NW; i++) t += red[i];
        t /= (float)in;
        t += L.eps;
        ss = 1.0f / sqrtf(t);
    }

    float acc[NM][R];
#pragma unroll
    for (int q = 0; q < NM; q++)
#pragma unroll
        for (int r = 0; r < R; r++) acc[q][r] = 0.f;

    while (c < C) {
        // request the next chunk's weights before computing on this one
        const int cn = c + 64;
        RowLoad nxt[NM][R];
        int32_t znext[NM];
#pragma unroll
        for (int q = 0; q < NM; q++) znext[q] = 0;
        if (cn < C) {
            const int g = cn / CPG;
#pragma unroll
            for (int q = 0; q < NM; q++) {
                const Q4Mat &M = L.m[mi + q];
                znext[q] = M.qzeros[(size_t)(o0 >> 3) * groups + g];
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const int o = min(o0 + r, n_out - 1);
                    nxt[q][r].w = M.qweight[(size_t)o * C + cn];
                    nxt[q][r].s = M.scales[(size_t)o * groups + g];
                }
            }
        }
#pragma unroll
        for (int q = 0; q < NM; q++) {
            const float *xs = lds + q * xstride;
            float x[32];
            {
                const float4 *p = reinterpret_cast<const float4 *>(&xs[c * kChunkPad]);
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float4 v = p[i];
                    x[4 * i + 0] = v.x;
                    x[4 * i + 1] = v.y;
                    x[4 * i + 2] = v.z;
                    x[4 * i + 3] = v.w;
                }
            }
            const float sx = xs[C * kChunkPad + c];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const float p = chunk_dot(cur[q][r].w, x);
                const int zn = (zcur[q] >> (4 * ((o0 + r) & 7))) & 15;
                const float z1 = (float)(zn + 1);
                const float t = fmaf(p, 512.0f, -z1 * sx);
                acc[q][r] = fmaf(cur[q][r].s, t, acc[q][r]);
            }
        }
#pragma unroll
        for (int q = 0; q < NM; q++) {
#pragma unroll
            for (int r = 0; r < R; r++) cur[q][r] = nxt[q][r];
            zcur[q] = znext[q];
        }
        c = cn;
    }

    // wave reduction, then lane r finishes row o0 + r
    float mine[NM];
#pragma unroll
    for (int q = 0; q < NM; q++) mine[q] = 0.f;
#pragma unroll
    for (int q = 0; q < NM; q++)
#pragma unroll
        for (int r = 0; r < R; r++) {
            const float v = wave_sum(acc[q][r]);
            if (lane == r) mine[q] = v;
        }
    const int o = o0 + lane;
    if (lane < R && o < n_out) {
        const Q4Epi &E = L.e;
        const size_t row = (size_t)b * n_out;
        float v = mine[0] * ss;
        if (PAIR) { // silu(w1 x) * (w3 x), src/models.rs:92-98
            const float u = mine[NM - 1] * ss;
            v = v * (1.0f / (1.0f + expf(-v)));
            v = v * u;
        } else if (E.kind == Q4_EPI_RESIDUAL) {
            v = E.res[row + o] + v;
        }
        if (E.kind != Q4_EPI_SCATTER_ONLY) L.m[mi].y[row + o] = v;
        for (int t = 0; t < E.n_scatter; t++) E.sc_out[t][row + E.sc_idx[t][o]] = v;
    }
}

template <int G, int R, int NW, bool PAIR>
int launch_t(Q4Launch &L, hipStream_t stream) {
    int total = 0;
    for (int i = 0; i < L.n_mats; i++) {
        L.m[i].row_blocks = (L.m[i].out + NW * R - 1) / (NW * R);
        total += L.m[i].row_blocks;
    }
    if (PAIR) total = L.m[0].row_blocks;
    const int C = L.in / 32;
    const size_t lds = (size_t)(C * kChunkPad + C) * sizeof(float) * (PAIR ? 2 : 1);
    auto kern = q4_matvec_kernel<G, R, NW, PAIR>;
    if (g_q4_name.armed) {
        g_q4_name.armed = false;
        snprintf(g_q4_name.buf, (size_t)g_q4_name.cap, "q4_matvec_kernel<%d, %d, %d, %s>", G, R, NW, PAIR ? "true" : "false");
        g_q4_name.grid = total, g_q4_name.block = NW * 64, g_q4_name.rows_per_block = NW * R, g_q4_name.lds = lds;
        return L2_OK;
    }
    if (lds + 256 > 160 * 1024) return l2_fail(L2_ERR_ARG, "q4 matvec: in=%d needs %zu B of LDS", L.in, lds);
    if (lds > 48 * 1024) {
        static LdsLimit limit; // per instantiation
        L2_TRY(limit.ensure(reinterpret_cast<const void *>(kern), lds));
    }
    dim3 grid(total, L.batch), block(NW * 64);
    if (g_q4_prof.armed) {
        g_q4_prof.armed = false;
        hipExtLaunchKernelGGL(kern, grid, block, lds, stream, g_q4_prof.start, g_q4_prof.stop, 0, L);
    } else {
        hipLaunchKernelGGL(kern, grid, block, lds, stream, L);
    }
    L2_HIP(hipGetLastError());
    return L2_OK;
}

template <int G>
int launch_g(Q4Launch &L, hipStream_t stream, int R, int NW) {
#define Q4_CASE(r, nw) \
    if (!L.pair && R == r && NW == nw) return launch_t<G, r, nw, false>(L, stream);
#define Q4_PAIR(r, nw) \
    if (L.pair && R == r && NW == nw) return launch_t<G, r, nw, true>(L, stream);
    Q4_CASE(2, 4) Q4_CASE(4, 4) Q4_CASE(8, 4)
    Q4_CASE(2, 8) Q4_CASE(4, 8) Q4_CASE(8, 8)
    Q4_CASE(2, 16) Q4_CASE(4, 16)
    Q4_PAIR(2, 4) Q4_PAIR(4, 4) Q4_PAIR(2, 8) Q4_PAIR(4, 8) Q4_PAIR(2, 16)
#undef Q4_CASE
#undef Q4_PAIR
    return l2_fail(L2_ERR_ARG, "q4 matvec: no kernel for R=%d NW=%d pair=%d", R, NW, L.pair);
}

int env_int(const char *name, int dflt) {
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : dflt;
}

} // namespace

int q4_matvec_launch(Q4Launch &L, hipStream_t stream) {
    if (L.n_mats < 1 || L.n_mats > 3) return l2_fail(L2_ERR_ARG, "q4 matvec: n_mats=%d", L.n_mats);
    if (L.in % 32 != 0 || L.in % L.group_size != 0)
        return l2_fail(L2_ERR_ARG, "q4 matvec: in=%d must be a multiple of 32 and of the group size %d",
                       L.in, L.group_size);
    if (L.batch < 1 || L.batch > 65535) return l2_fail(L2_ERR_RANGE, "q4 matvec: batch=%d", L.batch);
    if (L.e.n_scatter < 0 || L.e.n_scatter > 3) return l2_fail(L2_ERR_ARG, "q4 matvec: %d scatter targets", L.e.n_scatter);
    if (L.pair && (L.n_mats != 2 || L.m[0].out != L.m[1].out))
        return l2_fail(L2_ERR_ARG, "q4 matvec: a pair launch takes two matrices of equal height");
    long rows = 0;
    for (int i = 0; i < L.n_mats; i++) {
        if (L.m[i].out % 8 != 0) return l2_fail(L2_ERR_ARG, "q4 matvec: out=%d not a multiple of 8", L.m[i].out);
        rows += L.m[i].out;
    }
    // The row-streaming form is the default; L2_Q4_IMPL=tile selects the row-tile form.
    static const int impl_tile = []() {
        const char *v = getenv("L2_Q4_IMPL");
        return (v && !strcmp(v, "tile")) ? 1 : 0;
    }();
    for (int i = 0; i < L.n_mats; i++)
        if (L.m[i].gidx && !q4_gathers_in_kernel(L))
            return l2_fail(L2_ERR_ARG, "q4 matvec: this launch cannot gather x itself (in=%d, %d matrices)", L.in, L.n_mats);
    if (!impl_tile && q4_stream_supports(L)) return q4_stream_launch(L, stream);
    // Rows per wave: enough waves to cover 256 CUs several times over, more
    // rows per wave (less LDS traffic per weight byte) once there are plenty.
    static const int forced_r = env_int("L2_Q4_R", 0);
    static const int forced_nw = env_int("L2_Q4_NW", 0);
    const int C = L.in / 32;
    int R = rows >= 32768 ? 4 : 2;
    if (L.pair) R = 2;
    // Waves per block: big inputs need most of a CU's LDS for x, so one block
    // must bring enough waves by itself.
    const size_t lds = (size_t)(C * kChunkPad + C) * 4 * (L.pair ? 2 : 1);
    int NW = lds > 80 * 1024 ? 16 : lds > 40 * 1024 ? 8 : 4;
    if (forced_r) R = forced_r;
    if (forced_nw) NW = forced_nw;
    if (NW == 16 && R > 4) R = 4; // 1024-thread blocks leave 128 VGPRs per lane
    if (L.pair && R > 4) R = 4;
    if (L.pair && NW == 16) R = 2;
    switch (L.group_size) {
        case 32: return launch_g<32>(L, stream, R, NW);
        case 64: return launch_g<64>(L, stream, R, NW);
        case 128: return launch_g<128>(L, stream, R, NW);
    }
    return l2_fail(L2_ERR_ARG, "q4 matvec: group size %d (32, 64 or 128)", L.group_size);
}
