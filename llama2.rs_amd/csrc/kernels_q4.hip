// GPTQ 4-bit dequant matvec for gfx950 (wave64).
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
// Nibbles are turned into floats by v_cvt_f32_ubyteN on words masked with
// 0x0F0F0F0F (even nibbles) and 0xF0F0F0F0 (odd nibbles, scaled by 16, undone
// exactly afterwards), so one nibble costs one convert and one FMA.  All
// accumulation is fp32; the reduction order is fixed (no atomics), so results
// are bit-stable from run to run.
#include "l2_internal.h"

namespace {

constexpr int kChunkPad = 36; // floats per staged chunk of 32

template <int CTRL>
__device__ __forceinline__ float dpp_xchg(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
    return __builtin_bit_cast(float, r);
}

// Sum over the 64 lanes of a wave; every lane gets the result.
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_xchg<0xB1>(v);  // quad_perm [1,0,3,2]
    v += dpp_xchg<0x4E>(v);  // quad_perm [2,3,0,1]
    v += dpp_xchg<0x141>(v); // row_half_mirror
    v += dpp_xchg<0x140>(v); // row_mirror
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}

// 32 nibbles of one row against 32 inputs.  lo collects even nibbles, hi the
// odd ones times 16.
__device__ __forceinline__ void chunk_dot(const uint4 w, const float (&x)[32], float &lo, float &hi) {
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int d = 0; d < 4; d++) {
        const uint32_t l = words[d] & 0x0F0F0F0Fu;
        const uint32_t h = words[d] & 0xF0F0F0F0u;
        lo = fmaf((float)(l & 0xFFu), x[8 * d + 0], lo);
        hi = fmaf((float)(h & 0xFFu), x[8 * d + 1], hi);
        lo = fmaf((float)((l >> 8) & 0xFFu), x[8 * d + 2], lo);
        hi = fmaf((float)((h >> 8) & 0xFFu), x[8 * d + 3], hi);
        lo = fmaf((float)((l >> 16) & 0xFFu), x[8 * d + 4], lo);
        hi = fmaf((float)((h >> 16) & 0xFFu), x[8 * d + 5], hi);
        lo = fmaf((float)(l >> 24), x[8 * d + 6], lo);
        hi = fmaf((float)(h >> 24), x[8 * d + 7], hi);
    }
}

// G: group size, R: rows per wave, NW: waves per block.
template <int G, int R, int NW>
__global__ __launch_bounds__(NW * 64) void q4_matvec_kernel(const Q4Launch L) {
    extern __shared__ float lds[];
    const int in = L.in;
    const int C = in >> 5;             // chunks per row
    float *xs = lds;                   // [C][36]
    float *xsum = lds + C * kChunkPad; // [C]

    // which matrix, which rows
    int rb = blockIdx.x;
    int mi = 0;
    while (mi + 1 < L.n_mats && rb >= L.m[mi].row_blocks) {
        rb -= L.m[mi].row_blocks;
        mi++;
    }
    const Q4Mat &M = L.m[mi];
    const int b = blockIdx.y;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int o0 = (rb * NW + wave) * R; // first row of this wave; multiple of R
    const bool active = o0 < M.out;
    const int groups = L.groups;

    // First chunk's weights are requested before anything else so that the HBM
    // latency overlaps with staging x.
    uint4 wcur[R];
    float scur[R];
    int32_t zcur = 0;
    int c = lane;
    constexpr int CPG = G / 32; // chunks per group
    if (active && c < C) {
        const int g = c / CPG;
        zcur = M.qzeros[(size_t)(o0 >> 3) * groups + g];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const int o = min(o0 + r, M.out - 1);
            wcur[r] = M.qweight[(size_t)o * C + c];
            scur[r] = M.scales[(size_t)o * groups + g];
        }
    }

    // stage x (already in g_index order) into padded chunks
    {
        const float4 *xin = reinterpret_cast<const float4 *>(M.x + (size_t)b * in);
        for (int j4 = tid; j4 < (in >> 2); j4 += NW * 64) {
            const float4 v = xin[j4];
            const int j = j4 << 2;
            *reinterpret_cast<float4 *>(&xs[(j >> 5) * kChunkPad + (j & 31)]) = v;
        }
    }
    __syncthreads();
    for (int cc = tid; cc < C; cc += NW * 64) {
        const float4 *p = reinterpret_cast<const float4 *>(&xs[cc * kChunkPad]);
        float s = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4 v = p[i];
            s += (v.x + v.y) + (v.z + v.w);
        }
        xsum[cc] = s;
    }
    __syncthreads();
    if (!active) return;

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.f;

    while (c < C) {
        // request the next chunk's weights before computing on this one
        const int cn = c + 64;
        uint4 wnext[R];
        float snext[R];
        int32_t znext = 0;
        if (cn < C) {
            const int g = cn / CPG;
            znext = M.qzeros[(size_t)(o0 >> 3) * groups + g];
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int o = min(o0 + r, M.out - 1);
                wnext[r] = M.qweight[(size_t)o * C + cn];
                snext[r] = M.scales[(size_t)o * groups + g];
            }
        }
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
        const float sx = xsum[c];
#pragma unroll
        for (int r = 0; r < R; r++) {
            float lo = 0.f, hi = 0.f;
            chunk_dot(wcur[r], x, lo, hi);
            const int zn = (zcur >> (4 * ((o0 + r) & 7))) & 15;
            const float z1 = (float)(zn + 1);
            float t = fmaf(hi, 0.0625f, lo);
            t = fmaf(-z1, sx, t);
            acc[r] = fmaf(scur[r], t, acc[r]);
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
            wcur[r] = wnext[r];
            scur[r] = snext[r];
        }
        zcur = znext;
        c = cn;
    }

#pragma unroll
    for (int r = 0; r < R; r++) {
        const float v = wave_sum(acc[r]);
        const int o = o0 + r;
        if (lane == 0 && o < M.out) {
            float out = v;
            if (L.epi == Q4_EPI_RESIDUAL) out = M.res[(size_t)b * M.y_stride + o] + v;
            const int dst = M.scatter ? M.scatter[o] : o;
            M.y[(size_t)b * M.y_stride + dst] = out;
        }
    }
}

template <int G, int R, int NW>
int launch_t(Q4Launch &L, hipStream_t stream) {
    int total = 0;
    for (int i = 0; i < L.n_mats; i++) {
        L.m[i].row_blocks = (L.m[i].out + NW * R - 1) / (NW * R);
        total += L.m[i].row_blocks;
    }
    const int C = L.in / 32;
    const size_t lds = (size_t)(C * kChunkPad + C) * sizeof(float);
    auto kern = q4_matvec_kernel<G, R, NW>;
    if (lds > 64 * 1024) {
        static bool raised = false; // per instantiation
        if (!raised) {
            L2_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
            raised = true;
        }
    }
    if (lds > 160 * 1024) return l2_fail(L2_ERR_ARG, "q4 matvec: in=%d needs %zu B of LDS", L.in, lds);
    dim3 grid(total, L.batch), block(NW * 64);
    hipLaunchKernelGGL(kern, grid, block, lds, stream, L);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

template <int G>
int launch_g(Q4Launch &L, hipStream_t stream, int R, int NW) {
#define Q4_CASE(r, nw) \
    if (R == r && NW == nw) return launch_t<G, r, nw>(L, stream);
    Q4_CASE(2, 4) Q4_CASE(4, 4) Q4_CASE(8, 4)
    Q4_CASE(2, 8) Q4_CASE(4, 8) Q4_CASE(8, 8)
    Q4_CASE(2, 16) Q4_CASE(4, 16) Q4_CASE(8, 16)
#undef Q4_CASE
    return l2_fail(L2_ERR_ARG, "q4 matvec: no kernel for R=%d NW=%d", R, NW);
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
    long rows = 0;
    for (int i = 0; i < L.n_mats; i++) {
        if (L.m[i].out % 8 != 0) return l2_fail(L2_ERR_ARG, "q4 matvec: out=%d not a multiple of 8", L.m[i].out);
        rows += L.m[i].out;
    }
    // Rows per wave: enough waves to cover 256 CUs several times over, more
    // rows per wave (less LDS traffic per weight byte) once there are plenty.
    static const int forced_r = env_int("L2_Q4_R", 0);
    static const int forced_nw = env_int("L2_Q4_NW", 0);
    const int C = L.in / 32;
    int R = rows >= 32768 ? 8 : rows >= 8192 ? 4 : 2;
    // Waves per block: big inputs need most of a CU's LDS for x, so one block
    // must bring enough waves by itself.
    const size_t lds = (size_t)(C * kChunkPad + C) * 4;
    int NW = lds > 80 * 1024 ? 16 : lds > 40 * 1024 ? 8 : 4;
    if (forced_r) R = forced_r;
    if (forced_nw) NW = forced_nw;
    if (NW == 16 && R > 4) R = 4; // 1024-thread blocks leave 128 VGPRs per lane
    switch (L.group_size) {
        case 32: return launch_g<32>(L, stream, R, NW);
        case 64: return launch_g<64>(L, stream, R, NW);
        case 128: return launch_g<128>(L, stream, R, NW);
    }
    return l2_fail(L2_ERR_ARG, "q4 matvec: group size %d (32, 64 or 128)", L.group_size);
}
