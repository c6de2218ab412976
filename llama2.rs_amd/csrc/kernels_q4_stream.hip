// Row-streaming form of the GPTQ 4-bit dequant matvec (gfx950, wave64).
//
// Same function, prologue and epilogues as the row-tile kernel in
// kernels_q4.hip; what differs is who walks what.  Here every lane owns ONE
// chunk of K (32 consecutive inputs) for the whole kernel and keeps that slice
// of x in registers, so the main loop reads nothing from LDS.  NWK = ceil(C/64)
// waves side by side cover a full row; S such wave groups ("streams") per block
// take rows s, s+S, s+2S, ... of the block's row range.  A stream keeps P rows
// in flight: the loads of row i+P are issued before row i is consumed, so once
// the pipe is primed the HBM stream and the dequant arithmetic overlap inside
// every wave rather than only across blocks.
//
// Reduction: four DPP adds fold a wave's 64 partials into 4 (one per 16-lane
// row); those go to a small double-buffered LDS tile [row][NWK*4]; after one
// barrier per tile of P*S rows, one thread per row adds them in a fixed order
// and runs the epilogue.  No atomics: results are bit-stable.
#include "q4_common.h"

namespace {

using namespace q4;

struct RowData {
    uint4 w;
    float s;
    int32_t z;
};

template <int G, int NWK, int S, bool PAIR>
__global__ __launch_bounds__(NWK *S * 64) void q4_stream_kernel(const Q4Launch L) {
    constexpr int NM = PAIR ? 2 : 1;
    constexpr int NW = NWK * S;
#ifndef Q4S_P
#define Q4S_P 4
#endif
    constexpr int P = PAIR ? Q4S_P / 2 : Q4S_P; // rows (row pairs) in flight per stream
    constexpr int TR = P * S;       // rows per reduction tile
    constexpr int PW = NWK * 4;     // partials per row
    constexpr int CPG = G / 32;     // chunks per group
    extern __shared__ float lds[];
    __shared__ float red[NW];
    __shared__ float part[2][TR][NM][PW];

    const int in = L.in;
    const int C = in >> 5;
    const int xstride = C * kChunkPad + C;

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
    const int kslice = wave % NWK;
    const int stream = wave / NWK;
    const int n_out = L.m[mi].out;
    const int groups = L.groups;
    const int row0 = rb * L.rows_per_block;
    const int row1 = min(row0 + L.rows_per_block, n_out);
    const int c = kslice * 64 + lane; // this lane's chunk, for good
    const bool has_chunk = c < C;
    const int g = has_chunk ? c / CPG : 0;

    // row i of this stream is row0 + stream + i * S
    auto fetch = [&](int i, RowData(&d)[NM]) {
        const int o = row0 + stream + i * S;
        if (has_chunk && o < row1) {
#pragma unroll
            for (int q = 0; q < NM; q++) {
                const Q4Mat &M = L.m[mi + q];
                d[q].w = M.qweight[(size_t)o * C + c];
#ifdef L2_Q4_DEBUG
                if (L.e.kind >= 103) { // weights only
                    d[q].s = 1.f;
                    d[q].z = 0;
                    continue;
                }
#endif
                d[q].s = M.scales[(size_t)o * groups + g];
                d[q].z = M.qzeros[(size_t)(o >> 3) * groups + g];
            }
        }
    };

    // prime the pipe before anything else: these loads do not depend on x
    RowData pipe[P][NM];
#pragma unroll
    for (int u = 0; u < P; u++) fetch(u, pipe[u]);

    // stage x for the whole block, then take this lane's chunk into registers
    float ssq = 0.f;
#pragma unroll
    for (int q = 0; q < NM; q++) {
        const Q4Mat &M = L.m[mi + q];
        const float p = stage_input<NW>(M.x + (size_t)b * in, M.wn, in, lds + q * xstride,
                                        lds + q * xstride + C * kChunkPad, tid);
        if (q == 0) ssq = p;
    }
    const bool norm = L.m[mi].wn != nullptr;
    if (norm) {
        ssq = wave_sum(ssq);
        if (lane == 0) red[wave] = ssq;
    }
    __syncthreads();
    float ss = 1.0f;
    if (norm) { // rmsnorm scale, src/models.rs:55-60
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < NW; i++) t += red[i];
        t /= (float)in;
        t += L.eps;
        ss = 1.0f / sqrtf(t);
    }
    float x[NM][32];
    float sx[NM];
#pragma unroll
    for (int q = 0; q < NM; q++) {
        const float *xs = lds + q * xstride;
        if (has_chunk) {
            const float4 *p = reinterpret_cast<const float4 *>(&xs[c * kChunkPad]);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const float4 v = p[i];
                x[q][4 * i + 0] = v.x;
                x[q][4 * i + 1] = v.y;
                x[q][4 * i + 2] = v.z;
                x[q][4 * i + 3] = v.w;
            }
            sx[q] = xs[C * kChunkPad + c];
        } else {
#pragma unroll
            for (int i = 0; i < 32; i++) x[q][i] = 0.f;
            sx[q] = 0.f;
        }
    }

    const int n_rows = row1 - row0;
    const int n_tiles = (n_rows + TR - 1) / TR;
    int buf = 0;
    for (int tile = 0; tile < n_tiles; tile++) {
#pragma unroll
        for (int u = 0; u < P; u++) {
            const int i = tile * P + u;
            const int o = row0 + stream + i * S;
            float pr[NM];
#pragma unroll
            for (int q = 0; q < NM; q++) {
                float v = 0.f;
                if (has_chunk && o < row1) {
#ifdef L2_Q4_DEBUG
                    const uint4 ww = pipe[u][q].w;
                    const float p = (L.e.kind >= 101) ? __builtin_bit_cast(float, (ww.x ^ ww.y ^ ww.z ^ ww.w) & 0x3fffffffu) + x[q][u]
                                                      : chunk_dot(ww, x[q]);
#else
                    const float p = chunk_dot(pipe[u][q].w, x[q]);
#endif
                    const int zn = (pipe[u][q].z >> (4 * (o & 7))) & 15;
                    const float z1 = (float)(zn + 1);
                    v = pipe[u][q].s * fmaf(p, 512.0f, -z1 * sx[q]);
                }
                pr[q] = v;
            }
            fetch(i + P, pipe[u]); // refill this slot: row i + P
#pragma unroll
            for (int q = 0; q < NM; q++) {
                float v = pr[q];
                v += dpp_xchg<0xB1>(v);
                v += dpp_xchg<0x4E>(v);
                v += dpp_xchg<0x141>(v);
                v += dpp_xchg<0x140>(v);
                if ((lane & 15) == 0) part[buf][u * S + stream][q][kslice * 4 + (lane >> 4)] = v;
            }
        }
#ifdef L2_Q4_DEBUG
        if (L.e.kind == 104) continue; // no reduction barrier, no epilogue
#endif
        __syncthreads();
        if (tid < TR) {
            const int o = row0 + tile * TR + tid;
            if (o < row1) {
                float sum[NM];
#pragma unroll
                for (int q = 0; q < NM; q++) {
                    float a = 0.f;
#pragma unroll
                    for (int k = 0; k < PW; k++) a += part[buf][tid][q][k];
                    sum[q] = a;
                }
                const Q4Epi &E = L.e;
                const size_t row = (size_t)b * n_out;
                float v = sum[0] * ss;
                if (PAIR) { // silu(w1 x) * (w3 x), src/models.rs:92-98
                    const float u2 = sum[NM - 1] * ss;
                    v = v * (1.0f / (1.0f + expf(-v)));
                    v = v * u2;
                } else if (E.kind == Q4_EPI_RESIDUAL) {
                    v = E.res[row + o] + v;
                }
                if (E.kind != Q4_EPI_SCATTER_ONLY) L.m[mi].y[row + o] = v;
                for (int t = 0; t < E.n_scatter; t++) E.sc_out[t][row + E.sc_idx[t][o]] = v;
            }
        }
        buf ^= 1;
    }
}

int cu_count() {
    static int n = 0;
    if (n == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
            n = prop.multiProcessorCount;
        if (n <= 0) n = 256;
    }
    return n;
}

template <int G, int NWK, int S, bool PAIR>
int launch_s(Q4Launch &L, hipStream_t stream) {
    constexpr int NW = NWK * S;
    constexpr int TR = (PAIR ? Q4S_P / 2 : Q4S_P) * S;
    const int C = L.in / 32;
    const size_t lds = (size_t)(C * kChunkPad + C) * sizeof(float) * (PAIR ? 2 : 1);
    if (lds + 8 * 1024 > 160 * 1024) return l2_fail(L2_ERR_ARG, "q4 matvec: in=%d needs %zu B of LDS", L.in, lds);
    // Blocks: a whole number of rounds over the CUs, as many blocks per CU as
    // 16 waves and the LDS allow; every block gets the same number of rows.
    int per_cu = 16 / NW;
    if (per_cu < 1) per_cu = 1;
    const int by_lds = (int)((150 * 1024) / (lds + 4 * 1024));
    if (per_cu > by_lds) per_cu = by_lds < 1 ? 1 : by_lds;
    long rows = 0;
    for (int i = 0; i < (PAIR ? 1 : L.n_mats); i++) rows += L.m[i].out;
    const long slots = (long)cu_count() * per_cu;
    int rpb = (int)((rows + slots - 1) / slots);
    if (rpb < TR) rpb = TR;
    int total = 0;
    for (;;) { // several matrices round up separately: keep the grid within one round
        total = 0;
        for (int i = 0; i < (PAIR ? 1 : L.n_mats); i++) total += (L.m[i].out + rpb - 1) / rpb;
        if (total <= slots || rpb >= rows) break;
        rpb++;
    }
    L.rows_per_block = rpb;
    for (int i = 0; i < L.n_mats; i++) L.m[i].row_blocks = (L.m[i].out + rpb - 1) / rpb;
    auto kern = q4_stream_kernel<G, NWK, S, PAIR>;
    if (lds > 48 * 1024) {
        static size_t raised = 0; // per instantiation
        if (lds > raised) {
            L2_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            raised = lds;
        }
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
int launch_sg(Q4Launch &L, hipStream_t stream) {
    const int nwk = (L.in / 32 + 63) / 64;
    if (!L.pair) {
        switch (nwk) {
            case 1: return launch_s<G, 1, 4, false>(L, stream);
            case 2: return launch_s<G, 2, 4, false>(L, stream);
            case 3: return launch_s<G, 3, 4, false>(L, stream);
            case 4: return launch_s<G, 4, 4, false>(L, stream);
            case 5: case 6: return launch_s<G, 6, 2, false>(L, stream);
            case 7: return launch_s<G, 7, 2, false>(L, stream);
            case 8: return launch_s<G, 8, 2, false>(L, stream);
            case 9: case 10: case 11: case 12: case 13: case 14: return launch_s<G, 14, 1, false>(L, stream);
        }
    } else {
        switch (nwk) {
            case 1: return launch_s<G, 1, 4, true>(L, stream);
            case 2: return launch_s<G, 2, 4, true>(L, stream);
            case 3: return launch_s<G, 3, 2, true>(L, stream);
            case 4: return launch_s<G, 4, 2, true>(L, stream);
        }
    }
    return l2_fail(L2_ERR_ARG, "q4 matvec (streaming): in=%d pair=%d has no kernel", L.in, L.pair);
}

} // namespace

int q4_stream_launch(Q4Launch &L, hipStream_t stream) {
#ifdef L2_Q4_DEBUG
    static const int dbg = getenv("L2_Q4_DBG") ? atoi(getenv("L2_Q4_DBG")) : 0;
    if (dbg) L.e.kind = dbg;
#endif
    switch (L.group_size) {
        case 32: return launch_sg<32>(L, stream);
        case 64: return launch_sg<64>(L, stream);
        case 128: return launch_sg<128>(L, stream);
    }
    return l2_fail(L2_ERR_ARG, "q4 matvec: group size %d (32, 64 or 128)", L.group_size);
}

bool q4_stream_supports(const Q4Launch &L) {
    const int nwk = (L.in / 32 + 63) / 64;
    return L.pair ? nwk <= 4 : nwk <= 14;
}
