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
//
// Integer form (MODE 1, selected with L2_Q4_IMPL=idot; the fp32 form is the default).  The vector ALU is
// the co-bottleneck of the fp32 form (one FMA, one convert-equivalent and 3/8 of a mask per nibble).  The
// integer form quantises x once per block after staging, chunk by chunk, to 24-bit fixed point against a
// power-of-two step (delta = 2^(e-22), |x| < 2^e within the chunk) and stores it as six planes of balanced
// base-16 digits (-8..7), 8 digits per word in the nibble order of the weights.  A weight word XOR 0x88888888
// is the 8 signed nibbles n - 8, so v_dot8_i32_i4 multiplies one weight word with one digit word: 24
// instructions per 32 weights instead of ~76, exact integer sums, and
//   sum_k (n_k - z1) x_k = delta * (I - (z1 - 8) * sum_k q_k),  I = sum_d 16^d a_d.
// The quantisation error (2^-23 of the chunk maximum per element) is of the size of fp32 rounding.  Its
// quantisation prologue costs more than the shorter loop saves on the shapes measured, hence not the default.
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "q4_common.h"

namespace {

using namespace q4;

constexpr int kPlaneWords = 28; // per chunk: 6 planes x 4 words, delta, sum of q, 2 pad

template <int CTRL>
__device__ __forceinline__ int dpp_xchg_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

// Quantise a staged vector (xs[c*36 + i], c < C, i < 32) in place into digit
// planes: word (c, d, j) at ((uint32_t*)xs)[c*28 + d*4 + j]; delta and sum(q)
// as floats at [c*28 + 24], [c*28 + 25].  Thread -> (chunk, word of 8 elements);
// the 4 threads of a chunk are adjacent lanes.  Outputs only ever land on
// inputs of lower chunks, which are consumed in earlier passes.
template <int NT>
__device__ __forceinline__ void quantize_in_place(float *xs, int C, int tid) {
    uint32_t *xw = reinterpret_cast<uint32_t *>(xs);
    const int n_words = C * 4;
    for (int base = 0; base < n_words; base += NT) {
        const int wi = base + tid;
        const bool ok = wi < n_words;
        const int c = wi >> 2, j = wi & 3;
        float v[8];
        if (ok) {
            const float4 a = *reinterpret_cast<const float4 *>(&xs[c * kChunkPad + j * 8]);
            const float4 b = *reinterpret_cast<const float4 *>(&xs[c * kChunkPad + j * 8 + 4]);
            v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
        } else {
#pragma unroll
            for (int e = 0; e < 8; e++) v[e] = 0.f;
        }
        float am = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) am = fmaxf(am, fabsf(v[e]));
        am = fmaxf(am, dpp_xchg<0xB1>(am));
        am = fmaxf(am, dpp_xchg<0x4E>(am));
        // am < 2^(eb-126): step 2^(eb-148) keeps |x/step| < 2^22
        int eb = (int)((__builtin_bit_cast(uint32_t, am) >> 23) & 0xFFu);
        eb = eb < 22 ? 22 : eb;
        const float inv = __builtin_bit_cast(float, (uint32_t)(275 - eb) << 23);
        const float delta = __builtin_bit_cast(float, (uint32_t)(eb - 21) << 23);
        uint32_t u[8];
        int sq = 0;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const int q = (int)rintf(v[e] * inv);
            sq += q;
            u[e] = (uint32_t)(q + 0x888888);
        }
        sq += dpp_xchg_i<0xB1>(sq);
        sq += dpp_xchg_i<0x4E>(sq);
        uint32_t pw[6];
#pragma unroll
        for (int d = 0; d < 6; d++) {
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 8; e++) w |= ((u[e] >> (4 * d)) & 15u) << (4 * e);
            pw[d] = w ^ 0x88888888u; // unsigned digit - 8 as a signed nibble
        }
        __syncthreads(); // every input of this pass is in registers
        if (ok) {
#pragma unroll
            for (int d = 0; d < 6; d++) xw[c * kPlaneWords + d * 4 + j] = pw[d];
            if (j == 0) {
                xs[c * kPlaneWords + 24] = delta;
                xs[c * kPlaneWords + 25] = (float)sq;
            }
        }
        __syncthreads();
    }
}

// sum_k (n_k - 8) q_k over one chunk: 4 weight words against 6 digit planes.
__device__ __forceinline__ float chunk_idot(const uint4 w, const int (&xp)[24]) {
    const int w0 = (int)(w.x ^ 0x88888888u), w1 = (int)(w.y ^ 0x88888888u), w2 = (int)(w.z ^ 0x88888888u),
              w3 = (int)(w.w ^ 0x88888888u);
    int a[6];
#pragma unroll
    for (int d = 0; d < 6; d++) {
        int t = __builtin_amdgcn_sdot8(w0, xp[d * 4 + 0], 0, false);
        t = __builtin_amdgcn_sdot8(w1, xp[d * 4 + 1], t, false);
        t = __builtin_amdgcn_sdot8(w2, xp[d * 4 + 2], t, false);
        a[d] = __builtin_amdgcn_sdot8(w3, xp[d * 4 + 3], t, false);
    }
    const int lo = (((a[2] << 4) + a[1]) << 4) + a[0];
    const int hi = (((a[5] << 4) + a[4]) << 4) + a[3];
    return fmaf((float)hi, 4096.0f, (float)lo);
}

// A load of weights: read once per token and never again before some 40 GB of other weights have gone by,
// so it is marked non-temporal (no point in keeping the line in L2 or in the memory-side cache, where it
// would only push out what is re-read: x, the scales' neighbours, the next kernel's operands).  Measured on
// the 70B shapes: w1|w3 51.0 -> 45.8 us, w2 28.7 -> 25.7 us per launch.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
template <class T>
__device__ __forceinline__ T ld_at(const void *base, uint32_t byte_offset) {
    const char *p = reinterpret_cast<const char *>(base) + byte_offset;
    if constexpr (sizeof(T) == 16)
        return __builtin_bit_cast(T, __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p)));
    else
        return __builtin_nontemporal_load(reinterpret_cast<const T *>(p));
}

__device__ __forceinline__ void st_at(float *base, uint32_t byte_offset, float v) {
    *reinterpret_cast<float *>(reinterpret_cast<char *>(base) + byte_offset) = v;
}

// A uniform value, required in scalar registers where this is written: the load behind it is issued and
// waited for here rather than where the value is first used.  The value itself is not redefined (an asm
// output would hide from the compiler that a pointer is a kernel argument, i.e. global memory).
template <class T>
__device__ __forceinline__ T pin_s(T v) {
    asm volatile("" ::"s"(v));
    return v;
}

// The operands of one matrix of a launch, in scalar registers.
struct MatOps {
    const uint4 *qweight;
    const int32_t *qzeros;
    const float *scales;
    const float *x;
    const int32_t *gidx;
    const float *wn;
    float *y;
    int out;
};

__device__ __forceinline__ MatOps mat_ops(const Q4Mat &M) {
    MatOps o;
    o.qweight = pin_s(M.qweight);
    o.qzeros = pin_s(M.qzeros);
    o.scales = pin_s(M.scales);
    o.x = pin_s(M.x);
    o.gidx = pin_s(M.gidx);
    o.wn = pin_s(M.wn);
    o.y = pin_s(M.y);
    o.out = pin_s(M.out);
    return o;
}

struct RowData {
    uint4 w;
    float s;
    int32_t z;
};

// MODE 0: fp32 inner loop, x staged through LDS (rmsnorm prologue, several matrices, row pairs).
// MODE 1: integer-dot inner loop, x staged and quantised in LDS.
// MODE 2: fp32 inner loop, one matrix without rmsnorm: every wave loads its own slice of x (coalesced)
//         and turns it into the per-lane chunks through LDS of its own; no barrier before the first row.
// GATHER (MODE 0, one matrix, no rmsnorm): x arrives in its natural order and the kernel applies the act-order
//         permutation itself, x[g_index[j]] (src/gptq.rs:99-122), for a caller with no producer to do it: x and the
//         inverse of g_index are requested together and every element is written straight to its place in the
//         staged chunks (the scatter a producer's epilogue would have done); the chunk sums are taken by the lanes.
template <int G, int NWK, int S, bool PAIR, int MODE, int P, bool GATHER = false>
__global__ __launch_bounds__(NWK *S * 64) void q4_stream_kernel(const Q4Launch L) {
    constexpr bool IDOT = MODE == 1, DIRECT = MODE == 2;
    static_assert(!GATHER || (MODE == 0 && !PAIR), "the gathering form takes one matrix through the block-wide staging");
    static_assert(!(DIRECT && PAIR), "the direct form takes one matrix");
    constexpr int NM = PAIR ? 2 : 1;
    constexpr int NW = NWK * S;
    // P rows (row pairs) are in flight per stream
    constexpr int TR = P * S;       // rows per reduction tile
    constexpr int PW = NWK * 4;     // partials per row
    constexpr int CPG = G / 32;     // chunks per group
    extern __shared__ float lds[];
    __shared__ float red[NW];
    __shared__ float part[2][TR][NM][PW];

    // Every scalar operand the prologue needs is asked for here, at once, and pinned in SGPRs: a kernel's
    // arguments are cold in the scalar cache, a load that misses takes some 0.3 us, and loads the compiler
    // places where their values are first used follow each other (the matrix of this block, then its
    // pointers, then the row geometry: three round trips in front of the first weight load).
    const int in = pin_s(L.in);
    const int n_mats = pin_s(L.n_mats);
    const int groups = pin_s(L.groups);
    const int rows_per_block = pin_s(L.rows_per_block);
    const float eps = pin_s(L.eps);
    // epilogue operands, uniform for the block
    const int epi_kind = pin_s(L.e.kind);
    const int n_scatter = pin_s(L.e.n_scatter);
    const float *__restrict__ res = pin_s(L.e.res);
    const int32_t *__restrict__ sc_idx[3] = {pin_s(L.e.sc_idx[0]), pin_s(L.e.sc_idx[1]), pin_s(L.e.sc_idx[2])};
    float *__restrict__ sc_out[3] = {pin_s(L.e.sc_out[0]), pin_s(L.e.sc_out[1]), pin_s(L.e.sc_out[2])};
    MatOps mat[NM];
    int rb = blockIdx.x;
    if constexpr (PAIR) {
        mat[0] = mat_ops(L.m[0]);
        mat[1] = mat_ops(L.m[1]);
    } else {
        const MatOps m0 = mat_ops(L.m[0]), m1 = mat_ops(L.m[1]), m2 = mat_ops(L.m[2]);
        const int rb0 = pin_s(L.m[0].row_blocks), rb1 = pin_s(L.m[1].row_blocks);
        mat[0] = m0;
        if (n_mats > 1 && rb >= rb0) {
            rb -= rb0;
            mat[0] = m1;
            if (n_mats > 2 && rb >= rb1) {
                rb -= rb1;
                mat[0] = m2;
            }
        }
    }
    const int C = in >> 5;
    const int xstride = C * kChunkPad + C;

    const int b = blockIdx.y;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    // the wave's number as a scalar: the row a wave works on, and with it the row's part of every address and
    // the shift that extracts its zero point, are then scalar arithmetic, off the vector ALU
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kslice = wave % NWK;
    const int stream = wave / NWK;
    const int n_out = mat[0].out;
    const int row0 = rb * rows_per_block;
    const int row1 = min(row0 + rows_per_block, n_out);
    const int c = kslice * 64 + lane; // this lane's chunk, for good
    const bool has_chunk = c < C;

    // Row i of this stream is row0 + stream + i * S. Loads are unconditional so
    // that the loop body stays one basic block and every wait names only the
    // oldest row in flight: rows past the end re-read the block's last row and
    // lanes past the last chunk re-read the last chunk (their x is zero).
    const int cc = has_chunk ? c : C - 1;
    const int g = cc / CPG;
    const int last = row1 - 1;
    const uint4 *__restrict__ wq[NM];
    const float *__restrict__ sc[NM];
    const int32_t *__restrict__ zq[NM];
#pragma unroll
    for (int q = 0; q < NM; q++) {
        wq[q] = mat[q].qweight;
        sc[q] = mat[q].scales;
        zq[q] = mat[q].qzeros;
    }
    const uint32_t cc16 = (uint32_t)cc << 4, g4 = (uint32_t)g << 2; // the lane's part of the byte offsets
    auto fetch = [&](int i, RowData(&d)[NM]) {
        const int o = min(row0 + stream + i * S, last); // uniform: the row's part of an address is scalar work
#pragma unroll
        for (int q = 0; q < NM; q++) {
            d[q].w = ld_at<uint4>(reinterpret_cast<const char *>(wq[q]) + ((uint32_t)(o * C) << 4), cc16);
            d[q].s = ld_at<float>(reinterpret_cast<const char *>(sc[q]) + ((uint32_t)(o * groups) << 2), g4);
            d[q].z = ld_at<int32_t>(reinterpret_cast<const char *>(zq[q]) + ((uint32_t)((o >> 3) * groups) << 2), g4);
        }
    };

    // x first, then the first rows of the weights: loads return in order, and
    // the staging of x (a cache hit) must not queue behind rows that come from HBM.
    StageRegs xr[DIRECT ? 1 : NM];
    float4 xd[DIRECT ? 8 : 1];
    int4 gi[GATHER ? kStageBatch : 1];
    if constexpr (GATHER) { // the first batch covers the whole vector (checked by the launcher)
        const int n4 = in >> 2;
        const int4 *g4 = reinterpret_cast<const int4 *>(mat[0].gidx);
#pragma unroll
        for (int u = 0; u < kStageBatch; u++) {
            const int j4 = u * (NW * 64) + tid;
            gi[u] = j4 < n4 ? g4[j4] : make_int4(0, 0, 0, 0);
        }
    }
    if constexpr (DIRECT) {
        // this wave's 64 chunks of x, 1 KB per load instruction (whole cache lines); past the end the last
        // 16 bytes are re-read and zeroed below
        const float4 *xp = reinterpret_cast<const float4 *>(mat[0].x + (size_t)b * in);
        const int n4 = in >> 2;
#pragma unroll
        for (int i = 0; i < 8; i++) xd[i] = xp[min(kslice * 512 + i * 64 + lane, n4 - 1)];
    } else {
#pragma unroll
        for (int q = 0; q < NM; q++)
            stage_issue<NW>(mat[q].x + (size_t)b * in, mat[q].wn, in, 0, tid, xr[q]);
        // No wave of the block asks for weights before every wave has asked for its piece of x: a CU returns
        // loads in the order it received them, and a piece of x (a cache hit) requested behind another wave's
        // first rows (HBM) would hold up the staging of the whole block until those rows are in.
        if constexpr (NW > 1) __builtin_amdgcn_s_barrier();
    }
    __builtin_amdgcn_sched_barrier(0);
    RowData pipe[P][NM];
#pragma unroll
    for (int u = 0; u < P; u++) fetch(u, pipe[u]);
    __builtin_amdgcn_sched_barrier(0);

    // this lane's slice of x, for good: 32 floats, or 24 digit words + step + sum of q
    float x[NM][IDOT ? 1 : 32];
    int xp[NM][IDOT ? 24 : 1];
    float sx[NM];     // fp32 form: sum of the chunk's x; integer form: sum of its q
    float xdelta[NM]; // integer form: the chunk's step
    float ss = 1.0f;
    const bool norm = !DIRECT && mat[0].wn != nullptr;
    if constexpr (DIRECT) {
        // Turned through a region of LDS of the wave's own, from "lane l holds floats 4l..4l+3 of every 256"
        // to "lane l holds its chunk's 32": no block barrier (a wave's LDS accesses execute in order).
        float *xw = lds + wave * (64 * kChunkPad);
        const int n4 = in >> 2;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int j4 = i * 64 + lane; // float4 index within the wave's slice
            const float4 v = kslice * 512 + j4 < n4 ? xd[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            *reinterpret_cast<float4 *>(&xw[(j4 >> 3) * kChunkPad + (j4 & 7) * 4]) = v;
        }
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float4 v = *reinterpret_cast<const float4 *>(&xw[lane * kChunkPad + 4 * i]);
            x[0][4 * i + 0] = v.x;
            x[0][4 * i + 1] = v.y;
            x[0][4 * i + 2] = v.z;
            x[0][4 * i + 3] = v.w;
            t += (v.x + v.y) + (v.z + v.w);
        }
        sx[0] = t;
        xdelta[0] = 0.f;
    } else {
        // stage x for the whole block, then take this lane's chunk into registers
        float ssq = 0.f;
#pragma unroll
        for (int q = 0; q < NM; q++) {
            const MatOps &M = mat[q];
            float *xs = lds + q * xstride;
            float p = 0.f;
            if constexpr (GATHER) {
                const int n4 = in >> 2;
#pragma unroll
                for (int u = 0; u < kStageBatch; u++) {
                    const int j4 = u * (NW * 64) + tid;
                    if (j4 < n4) { // element 4 j4 + e of x is input gi[u].e of the sorted rows
                        xs[(gi[u].x >> 5) * kChunkPad + (gi[u].x & 31)] = xr[q].v[u].x;
                        xs[(gi[u].y >> 5) * kChunkPad + (gi[u].y & 31)] = xr[q].v[u].y;
                        xs[(gi[u].z >> 5) * kChunkPad + (gi[u].z & 31)] = xr[q].v[u].z;
                        xs[(gi[u].w >> 5) * kChunkPad + (gi[u].w & 31)] = xr[q].v[u].w;
                    }
                }
            } else {
                p = stage_consume<NW>(M.wn != nullptr, in, 0, tid, xr[q], xs, xs + C * kChunkPad, 0.f);
                p = stage_rest<NW>(M.x + (size_t)b * in, M.wn, in, xs, xs + C * kChunkPad, tid, p);
            }
            if (q == 0) ssq = p;
        }
        if (norm) {
            ssq = wave_sum(ssq);
            if (lane == 0) red[wave] = ssq;
        }
        __syncthreads();
        if (norm) { // rmsnorm scale, src/models.rs:55-60
            float t = 0.f;
#pragma unroll
            for (int i = 0; i < NW; i++) t += red[i];
            t /= (float)in;
            t += eps;
            ss = 1.0f / sqrtf(t);
        }
        if constexpr (IDOT) {
#pragma unroll
            for (int q = 0; q < NM; q++) quantize_in_place<NW * 64>(lds + q * xstride, C, tid);
        }
#pragma unroll
        for (int q = 0; q < NM; q++) {
            const float *xs = lds + q * xstride;
            xdelta[q] = 0.f;
            sx[q] = 0.f;
            if constexpr (IDOT) {
                if (has_chunk) {
                    const uint4 *p = reinterpret_cast<const uint4 *>(&xs[c * kPlaneWords]);
#pragma unroll
                    for (int i = 0; i < 6; i++) {
                        const uint4 v = p[i];
                        xp[q][4 * i + 0] = (int)v.x;
                        xp[q][4 * i + 1] = (int)v.y;
                        xp[q][4 * i + 2] = (int)v.z;
                        xp[q][4 * i + 3] = (int)v.w;
                    }
                    xdelta[q] = xs[c * kPlaneWords + 24];
                    sx[q] = xs[c * kPlaneWords + 25];
                } else {
#pragma unroll
                    for (int i = 0; i < 24; i++) xp[q][i] = 0;
                }
            } else {
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
                    if constexpr (GATHER) {
                        // the chunk's sum in the association the block-wide staging uses (fours, then the tree of
                        // its three cross-lane adds), so that both forms of the operator give the same bits
                        float s4[8];
#pragma unroll
                        for (int k = 0; k < 8; k++)
                            s4[k] = (x[q][4 * k] + x[q][4 * k + 1]) + (x[q][4 * k + 2] + x[q][4 * k + 3]);
                        sx[q] = ((s4[0] + s4[1]) + (s4[2] + s4[3])) + ((s4[7] + s4[6]) + (s4[5] + s4[4]));
                    } else {
                        sx[q] = xs[C * kChunkPad + c];
                    }
                } else {
#pragma unroll
                    for (int i = 0; i < 32; i++) x[q][i] = 0.f;
                }
            }
        }
    }

    float nsx[NM];
#pragma unroll
    for (int q = 0; q < NM; q++) nsx[q] = -sx[q];
    const int n_rows = row1 - row0;
    // Steps of the longest stream; whole tiles of P steps run in the loop, what is left runs once after it,
    // straight-line and without refills, so that the loop body stays one block (and its waits exact).
    const int n_steps = (n_rows + S - 1) / S;
    const int n_full = n_steps / P;
    const int n_rem = n_steps - n_full * P;
    int buf = 0;
    // Enter the loop with no load outstanding (the primed rows arrived while x
    // was staged). The compiler's wait counts inside the loop are then those of
    // the steady state alone: vmcnt leaves the P - 1 younger rows in flight.
    // Otherwise the issue order of the prologue leaks into the loop's waits.
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0), expcnt and lgkmcnt untouched
    const size_t out_base = (size_t)b * n_out;
    float *__restrict__ const yout = mat[0].y;
    // what the epilogue lanes prefetch; the scales (at least one word per row) stand in for absent operands
    const bool has_res = !PAIR && epi_kind == Q4_EPI_RESIDUAL;
    const float *__restrict__ res_p = has_res ? res + out_base : sc[0];
    const int32_t *__restrict__ idx_p[3];
#pragma unroll
    for (int t = 0; t < 3; t++) idx_p[t] = t < n_scatter ? sc_idx[t] : reinterpret_cast<const int32_t *>(sc[0]);

    // one row (row pair) of this stream: dequantised dot product of the lane's chunk -> pr
    auto row_dot = [&](int o, const RowData(&d)[NM], float(&pr)[NM]) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < NM; q++) {
            const int zn = (int)(((uint32_t)d[q].z >> (4 * (o & 7))) & 15u);
            if constexpr (IDOT) {
                const float f = chunk_idot(d[q].w, xp[q]);
                pr[q] = (d[q].s * xdelta[q]) * fmaf(-(float)(zn - 7), sx[q], f);
            } else {
                const float p = chunk_dot(d[q].w, x[q]);
                // -(zn + 1) sx as one FMA on the converted nibble (the same real number, rounded once either way)
                pr[q] = d[q].s * fmaf(p, 512.0f, fmaf((float)zn, nsx[q], nsx[q]));
            }
        }
    };
    // 64 partials -> 4 (one per 16-lane row) -> the tile's slot for this row
    auto row_fold = [&](int u, const float(&pr)[NM]) __attribute__((always_inline)) {
#pragma unroll
        for (int q = 0; q < NM; q++) {
            float v = pr[q];
            v += dpp_xchg<0xB1>(v);
            v += dpp_xchg<0x4E>(v);
            v += dpp_xchg<0x141>(v);
            v += dpp_xchg<0x140>(v);
            if ((lane & 15) == 0) part[buf][u * S + stream][q][kslice * 4 + (lane >> 4)] = v;
        }
    };
    // one thread per row of the tile: fixed-order sum of the partials, then the epilogue
    auto tile_finish = [&](int eo, float res_v, const uint32_t(&sidx)[3]) __attribute__((always_inline)) {
        float sum[NM];
#pragma unroll
        for (int q = 0; q < NM; q++) {
            float a = 0.f;
#pragma unroll
            for (int k = 0; k < PW; k++) a += part[buf][tid][q][k];
            sum[q] = a;
        }
        float v = sum[0] * ss;
        if (PAIR) { // silu(w1 x) * (w3 x), src/models.rs:92-98
            const float u2 = sum[NM - 1] * ss;
            v = v * (1.0f / (1.0f + expf(-v)));
            v = v * u2;
        } else if (epi_kind == Q4_EPI_RESIDUAL) {
            v = res_v + v;
        }
        if (epi_kind != Q4_EPI_SCATTER_ONLY) yout[out_base + eo] = v;
#pragma unroll
        for (int t = 0; t < 3; t++)
            if (t < n_scatter) st_at(sc_out[t], ((uint32_t)out_base + sidx[t]) << 2, v); // 32-bit offset: nothing widens the loaded index
    };

    for (int tile = 0; tile < n_full; tile++) {
        // The lanes that finish this tile's rows fetch what the epilogue reads
        // (residual, scatter indices) now: by the time it is needed, P rows of
        // younger loads stand behind it and the wait leaves those in flight.
        const int eo = row0 + tile * TR + tid;
        const bool epi = tid < TR && eo < row1;
        float res_v = 0.f;
        uint32_t sidx[3] = {0, 0, 0};
        if (epi) { // no branch per operand: an unused one reads a valid dummy
            res_v = res_p[eo];
#pragma unroll
            for (int t = 0; t < 3; t++) sidx[t] = (uint32_t)idx_p[t][eo];
        }
#pragma unroll
        for (int u = 0; u < P; u++) {
            const int i = tile * P + u;
            float pr[NM];
            row_dot(row0 + stream + i * S, pipe[u], pr);
            // Refill this slot with row i + P, after its last use and not before:
            // a load hoisted above the row's arithmetic makes the compiler copy
            // live registers of the other slots, and each copy waits on its load.
            // The empty statements pin the row's result before the loads and
            // the loads before what follows.
            if constexpr (NM == 2) asm volatile("" : "+v"(pr[0]), "+v"(pr[NM - 1])::"memory");
            else asm volatile("" : "+v"(pr[0])::"memory");
            __builtin_amdgcn_sched_barrier(0);
            fetch(i + P, pipe[u]);
            __builtin_amdgcn_sched_barrier(0);
            row_fold(u, pr);
        }
        __syncthreads();
        if (epi) tile_finish(eo, res_v, sidx);
        buf ^= 1;
    }
    if (n_rem > 0) { // the rows already in the pipe: no refill, nothing younger to leave in flight
        const int eo = row0 + n_full * TR + tid;
        const bool epi = tid < TR && eo < row1;
        float res_v = 0.f;
        uint32_t sidx[3] = {0, 0, 0};
        if (epi) {
            res_v = res_p[eo];
#pragma unroll
            for (int t = 0; t < 3; t++) sidx[t] = (uint32_t)idx_p[t][eo];
        }
#pragma unroll
        for (int u = 0; u < P - 1; u++) {
            if (u < n_rem) {
                float pr[NM];
                row_dot(row0 + stream + (n_full * P + u) * S, pipe[u], pr);
                row_fold(u, pr);
            }
        }
        __syncthreads();
        if (epi) tile_finish(eo, res_v, sidx);
    }
}

// Rows per block for a block of NW waves and tiles of TR rows: a whole number of rounds over the CUs, as
// many blocks per CU as 16 waves and the LDS allow (one for a row pair); every block gets the same number of
// rows; several matrices round up separately and the grid stays within one round.
static int plan_rows(const Q4Launch &L, int NW, int TR, size_t lds, bool pair, int *total_out) {
    int per_cu = 16 / NW;
    if (pair) per_cu = 1; // w1|w3: one block per CU measured faster than two (7B: 13.1 -> 12.4 us, 722 -> 733 tok/s)
    if (per_cu < 1) per_cu = 1;
    const int by_lds = (int)((150 * 1024) / (lds + 4 * 1024));
    if (per_cu > by_lds) per_cu = by_lds < 1 ? 1 : by_lds;
    long rows = 0;
    const int nm = pair ? 1 : L.n_mats;
    for (int i = 0; i < nm; i++) rows += L.m[i].out;
    const long slots = (long)cu_count() * per_cu;
    int rpb = (int)((rows + slots - 1) / slots);
    if (rpb < TR) rpb = TR;
    int total = 0;
    for (;;) {
        total = 0;
        for (int i = 0; i < nm; i++) total += (L.m[i].out + rpb - 1) / rpb;
        if (total <= slots || rpb >= rows) break;
        rpb++;
    }
    if (total_out) *total_out = total;
    return rpb;
}

// Wave-rows of arithmetic per CU for a candidate shape: what the choice between shapes minimises.
static long plan_cost(const Q4Launch &L, int NWK, int S, int P, bool pair) {
    const int C = L.in / 32;
    const size_t lds = (size_t)(C * kChunkPad + C) * sizeof(float) * (pair ? 2 : 1);
    const int NW = NWK * S, TR = P * S;
    int per_cu = 16 / NW;
    if (pair) per_cu = 1; // w1|w3: one block per CU measured faster than two (7B: 13.1 -> 12.4 us, 722 -> 733 tok/s)
    if (per_cu < 1) per_cu = 1;
    const int by_lds = (int)((150 * 1024) / (lds + 4 * 1024));
    if (per_cu > by_lds) per_cu = by_lds < 1 ? 1 : by_lds;
    const int rpb = plan_rows(L, NW, TR, lds, pair, nullptr);
    const long tiles = (rpb + TR - 1) / TR;
    return (long)per_cu * NW * tiles * P;
}

template <int G, int NWK, int S, bool PAIR, int MODE, int P = (PAIR ? 2 : 4), bool GATHER = false>
int launch_s(Q4Launch &L, hipStream_t stream) {
    constexpr int NW = NWK * S;
    constexpr int TR = P * S;
    const int C = L.in / 32;
    const size_t lds = MODE == 2 ? (size_t)NW * 64 * kChunkPad * sizeof(float)
                                 : (size_t)(C * kChunkPad + C) * sizeof(float) * (PAIR ? 2 : 1);
    if (GATHER && L.in > NW * 64 * 4 * kStageBatch)
        return l2_fail(L2_ERR_ARG, "q4 matvec (gathering): in=%d is more than one staging batch of %d waves", L.in, NW);
    if (lds + 8 * 1024 > 160 * 1024) return l2_fail(L2_ERR_ARG, "q4 matvec: in=%d needs %zu B of LDS", L.in, lds);
    int total = 0;
    const int rpb = plan_rows(L, NW, TR, lds, PAIR, &total);
    L.rows_per_block = rpb;
    for (int i = 0; i < L.n_mats; i++) L.m[i].row_blocks = (L.m[i].out + rpb - 1) / rpb;
    auto kern = q4_stream_kernel<G, NWK, S, PAIR, MODE, P, GATHER>;
    if (g_q4_name.armed) {
        g_q4_name.armed = false;
        snprintf(g_q4_name.buf, (size_t)g_q4_name.cap, "q4_stream_kernel<%d, %d, %d, %s, %d, %d, %s>", G, NWK, S,
                 PAIR ? "true" : "false", MODE, P, GATHER ? "true" : "false");
        g_q4_name.grid = total, g_q4_name.block = NW * 64, g_q4_name.rows_per_block = rpb, g_q4_name.lds = lds;
        return L2_OK;
    }
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

// Rows in flight per stream (P) were measured per shape on whole decode steps.  Where the rows of a block are
// few (4096 and 11008 inputs: 4 to 8 rows per stream), fewer loads primed in front of x let x arrive sooner,
// and every instruction of the kernel waits for x: two rows at 4096 inputs (7B +1.2 %), three at 11008 (+0.9 %)
// and at 13824 through the per-wave form (13B +0.7 %); priming all rows of the block is 15-20 % slower.
template <int G, int MODE>
int launch_sg(Q4Launch &L, hipStream_t stream) {
    const int nwk = (L.in / 32 + 63) / 64;
    if constexpr (MODE == 2) { // only the shapes q4_stream_launch sends here
        if (!L.pair) switch (nwk) {
            case 3:
                if (plan_cost(L, 3, 5, 4, false) < plan_cost(L, 3, 4, 4, false)) return launch_s<G, 3, 5, false, MODE>(L, stream);
                return launch_s<G, 3, 4, false, MODE>(L, stream);
            case 7: return launch_s<G, 7, 2, false, MODE, 3>(L, stream);
            case 9: case 10: case 11: case 12: case 13: case 14: return launch_s<G, 14, 1, false, MODE>(L, stream);
        }
    } else if (MODE == 0 && !L.pair && L.n_mats == 1 && L.m[0].gidx) {
        if constexpr (MODE == 0) switch (nwk) { // the gathering form, where one staging batch covers the vector
            case 1: return launch_s<G, 1, 4, false, 0, 4, true>(L, stream);
            case 2: return launch_s<G, 2, 4, false, 0, 2, true>(L, stream);
            case 3: return launch_s<G, 3, 4, false, 0, 4, true>(L, stream);
            case 4: return launch_s<G, 4, 4, false, 0, 2, true>(L, stream);
        }
    } else if (!L.pair) {
        switch (nwk) {
            case 1: return launch_s<G, 1, 4, false, MODE>(L, stream);
            case 2: return launch_s<G, 2, 4, false, MODE, 2>(L, stream);
            case 3: // 5120: 20 rows per block are one tile of 5 streams, 60 or so are four tiles either way
                if (plan_cost(L, 3, 5, 4, false) < plan_cost(L, 3, 4, 4, false)) return launch_s<G, 3, 5, false, MODE>(L, stream);
                return launch_s<G, 3, 4, false, MODE>(L, stream);
            case 4: return launch_s<G, 4, 4, false, MODE, 2>(L, stream); // 8192: rows of 4 KB; two in flight per stream measured faster than four (q|k|v 13.4 -> 12.2 us, wo 12.1 -> 10.9)
            case 5: case 6: return launch_s<G, 6, 2, false, MODE, 3>(L, stream);
            case 7: return launch_s<G, 7, 2, false, MODE, 5>(L, stream); // 13824 -> 5120: 20 rows per block in two tiles
            case 8: return launch_s<G, 8, 2, false, MODE>(L, stream);
            case 9: case 10: case 11: case 12: case 13: case 14: return launch_s<G, 14, 1, false, MODE>(L, stream);
        }
    } else {
        switch (nwk) {
            case 1: return launch_s<G, 1, 4, true, MODE>(L, stream);
            case 2: return launch_s<G, 2, 4, true, MODE>(L, stream);
            case 3: return launch_s<G, 3, 5, true, MODE>(L, stream);
            case 4: return launch_s<G, 4, 2, true, MODE>(L, stream);
        }
    }
    return l2_fail(L2_ERR_ARG, "q4 matvec (streaming): in=%d pair=%d has no kernel", L.in, L.pair);
}

} // namespace

int q4_stream_launch(Q4Launch &L, hipStream_t stream) {
    // L2_Q4_IMPL=idot selects the integer-dot form of the inner loop; the default is the fp32 form.
    static const bool fp32_form = []() {
        const char *v = getenv("L2_Q4_IMPL");
        return !(v && !strcmp(v, "idot"));
    }();
    // One matrix and no rmsnorm in front: x can reach the registers through LDS of each wave's own instead
    // of a block-wide staging with a barrier.  Measured per input width (cadence of the launch, block-wide
    // against per-wave): 28672: 30.3 -> 28.6 us; 13824: 14.2 -> 13.2; 5120: 9.0 -> 7.7; but 11008: 9.0 -> 9.5,
    // 8192: 11.6 -> 12.3, 4096 equal within the model.  The per-wave form is taken where it won: 3 and 7 waves
    // per row, and inputs too long to stage block-wide beside a second block.
    const int nwk = (L.in / 32 + 63) / 64;
    const bool direct = fp32_form && !L.pair && L.n_mats == 1 && L.m[0].wn == nullptr && L.m[0].gidx == nullptr &&
                        (L.in > 16384 || nwk == 3 || nwk == 7);
    if (direct) {
        switch (L.group_size) {
            case 32: return launch_sg<32, 2>(L, stream);
            case 64: return launch_sg<64, 2>(L, stream);
            case 128: return launch_sg<128, 2>(L, stream);
        }
    } else if (fp32_form) {
        switch (L.group_size) {
            case 32: return launch_sg<32, 0>(L, stream);
            case 64: return launch_sg<64, 0>(L, stream);
            case 128: return launch_sg<128, 0>(L, stream);
        }
    } else {
        switch (L.group_size) {
            case 32: return launch_sg<32, 1>(L, stream);
            case 64: return launch_sg<64, 1>(L, stream);
            case 128: return launch_sg<128, 1>(L, stream);
        }
    }
    return l2_fail(L2_ERR_ARG, "q4 matvec: group size %d (32, 64 or 128)", L.group_size);
}

static bool fp32_stream_form() {
    static const bool yes = []() {
        const char *v = getenv("L2_Q4_IMPL");
        return !(v && (!strcmp(v, "idot") || !strcmp(v, "tile")));
    }();
    return yes;
}

bool q4_gathers_in_kernel(const Q4Launch &L) {
    const int nwk = (L.in / 32 + 63) / 64;
    return fp32_stream_form() && !L.pair && L.n_mats == 1 && L.m[0].wn == nullptr && nwk <= 4 && L.in % 4 == 0 &&
           q4_stream_supports(L);
}

bool q4_stream_supports(const Q4Launch &L) {
    const int nwk = (L.in / 32 + 63) / 64;
    // the kernel addresses a matrix with 32-bit byte offsets and 24-bit row numbers
    for (int i = 0; i < L.n_mats; i++)
        if (L.m[i].out >= (1 << 24) || (size_t)L.m[i].out * (size_t)(L.in / 8) * 4 >= ((size_t)1 << 32)) return false;
    return L.pair ? nwk <= 4 : nwk <= 14;
}
