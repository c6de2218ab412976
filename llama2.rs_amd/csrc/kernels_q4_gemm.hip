// Batched-prefill form of the GPTQ 4-bit linear layer for gfx950: dequantise
// tiles of the packed weights to fp16 in registers and feed them to the matrix
// cores (v_mfma_f32_32x32x16_f16), fp32 accumulate.
//
//   Y[t][o] = sum_k W[o][k] * X[t][k],   W[o][k] = scales[o][k/G] * (nib(qweight[o],k) - z1[o][k/G])
//
// for a chunk of T tokens whose inputs the caller has already brought into this
// layer's g_index order, multiplied by the norm weight where one applies, and
// rounded to fp16 (prep_f16_kernel).  This is the one place in the token loop
// that is a dense contraction, hence the one place that uses MFMA; the decode
// matvec stays on the vector ALU in fp32.
//
// Tiling.  A block is 4 waves; a wave owns one tile of 32 output rows and all NB
// blocks of 32 tokens (the dequantised weights are reused NB times), so a block
// covers 128 rows x 32*NB tokens.  With only 128 tokens per chunk that leaves
// few blocks, so K is also cut into KS slices across grid.z; each slice writes
// its fp32 partial tile to a workspace and q4_gemm_reduce_kernel adds the
// slices in a fixed order and runs the epilogue.  K advances
// 64 at a time: lane (r = l%32, h = l/32) loads the 16 bytes qweight[o][K/8+4h ..
// +4) of its row -- four packed words, each of which is exactly the 8 k-values
// one MFMA step wants from this lane.  The X slice [tokens][64] is staged in LDS
// (rows padded to 72 halves so that 16-byte reads of 32 lanes are conflict-free),
// double-buffered.
//
// Dequant.  (w >> 4i) & 0x000F000F | 0x64006400 is the fp16 pair (1024+n_i,
// 1024+n_{i+4}); subtracting 1024+z1 is exact.  The pairs come out as
// (n0,n4),(n1,n5),(n2,n6),(n3,n7), so X is stored with the same interleave
// inside every 8 consecutive k.  For G >= 64 the matrix cores see the exact
// integers n - z1 and the fp32 scale is applied to the fp32 partial sum of each
// group (one FMA per accumulator element and group), so the only rounding on
// the weight side is none at all; for G = 32 a K step of 64 straddles two
// groups, and the weights are multiplied by fp16(scale) before the MFMA.
#include "l2_internal.h"
#include <algorithm>

namespace {

typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kXPad = 8; // halves of padding per staged token row (K step + 8: 16-byte reads stay conflict-free)

union A8 {
    h8 v;
    h2 p[4];
    uint32_t u[4];
};

// (x & mask) | magic in one instruction; the compiler splits it into v_and + v_or because both constants
// would be literals.  mask lives in a VGPR, magic in an SGPR (one scalar operand per VALU instruction).
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask_v, uint32_t magic_s) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(mask_v), "s"(magic_s));
    return r;
}

struct DequantConsts {
    uint32_t mask_lo, mask_hi; // 0x000F000F, 0x00F000F0 (VGPRs)
    uint32_t magic;            // 0x64006400: fp16 1024 in both halves (SGPR)
    h2 neg_off;                // -(1024 + z1)
    h2 neg_off16;              // -(64 + z1)
    h2 sixteenth;              // 1/16
};

// One packed word of 8 nibbles -> 8 fp16 values n - z1 (exact), times `scale` if SCALED, in the pair
// order (0,4,1,5,2,6,3,7).  Nibbles 0 and 4 (and 2, 6 after one shift by 8) land in the low mantissa bits
// of the fp16 pair: 1024 + n.  Nibbles 1 and 5 (3, 7) are taken where they stand, four bits higher:
// 1024 + 16 n, and one packed FMA with 1/16 brings them to 64 + n, both exact.  9 instructions per word.
template <bool SCALED>
__device__ __forceinline__ h8 dequant8(uint32_t w, const DequantConsts &c, h2 scale) {
    A8 a;
    const uint32_t w8 = w >> 8;
    h2 v0 = __builtin_bit_cast(h2, and_or(w, c.mask_lo, c.magic)) + c.neg_off;
    h2 v1 = __builtin_elementwise_fma(__builtin_bit_cast(h2, and_or(w, c.mask_hi, c.magic)), c.sixteenth, c.neg_off16);
    h2 v2 = __builtin_bit_cast(h2, and_or(w8, c.mask_lo, c.magic)) + c.neg_off;
    h2 v3 = __builtin_elementwise_fma(__builtin_bit_cast(h2, and_or(w8, c.mask_hi, c.magic)), c.sixteenth, c.neg_off16);
    a.p[0] = SCALED ? v0 * scale : v0;
    a.p[1] = SCALED ? v1 * scale : v1;
    a.p[2] = SCALED ? v2 * scale : v2;
    a.p[3] = SCALED ? v3 * scale : v3;
    return a.v;
}

template <class T>
__device__ __forceinline__ T ld_at(const void *base, uint32_t byte_offset) {
    return *reinterpret_cast<const T *>(reinterpret_cast<const char *>(base) + byte_offset);
}

// Software pipeline of the K loop.  The weights of a K step are loaded WR steps ahead, its activation
// tile XP steps ahead, the scales and zero points of PW groups once per PW steps, all unconditionally
// (steps past the end of the block's K slice re-read its last step), into rings of registers indexed
// statically by the position in the loop body, which is unrolled PW times.  Loads return in order, so a
// wait for the oldest ring slot leaves the younger ones in flight; within a step the activation tile is
// requested before the weights, because the end of the step waits for it (it comes from the L2) and would
// otherwise wait for the weights requested before it as well.  Shallow rings on purpose: at K steps of 128,
// depths of 4 and 2 instead of 2 and 1 cost 34 more registers and were 3 % slower.
constexpr int kGemmPW = 4;
// ring depths in K steps: 256 k ahead for the weights, 128 k for the activation tile
constexpr int gemm_wr(int kstep) { return 256 / kstep; }
constexpr int gemm_xp(int kstep) { return 128 / kstep; }

template <int G, int NB, int KSTEP>
__global__ __launch_bounds__(256, NB > 2 ? 2 : 1) void q4_gemm_kernel(const Q4Launch L, const XhList xh_list, const float *__restrict__ ss,
                                                      float *__restrict__ ws, int KS, int partials) {
    constexpr int PW = kGemmPW, XP = gemm_xp(KSTEP), WR = gemm_wr(KSTEP);
    static_assert(PW % WR == 0 && PW % XP == 0, "ring slots are indexed by the position in the unrolled body");
    constexpr int W = KSTEP / 64;        // sub-steps of 64 k per K step
    constexpr int kXRow = KSTEP + kXPad; // halves per staged token row
    static_assert(KSTEP == 64 || G >= KSTEP, "a longer K step stays inside one group");
    constexpr int TN = 32 * NB;
    constexpr bool SA = G >= 64; // scale after the group's partial sum
    extern __shared__ _Float16 xs[]; // [2][TN][kXRow]
    __shared__ float gsc[2][kGemmPW][128]; // fp32 scales of the block's 128 rows, PW groups at a time
    __shared__ int32_t zsc[2][kGemmPW][16]; // their packed zero points: one word per 8 rows and group
    const int in = L.in;
    const int n_k = in / KSTEP; // K iterations

    int rb = blockIdx.x;
    int mi = 0;
    while (mi + 1 < L.n_mats && rb >= L.m[mi].row_blocks) {
        rb -= L.m[mi].row_blocks;
        mi++;
    }
    const Q4Mat &M = L.m[mi];
    const _Float16 *xh = reinterpret_cast<const _Float16 *>(xh_list.p[mi]); // [B][in] fp16, pair-interleaved
    const int n_out = M.out;
    const int groups = L.groups;
    const int B = L.batch;
    const int t0 = blockIdx.y * TN;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int C4 = in >> 5; // uint4 per weight row

    const int o_lane = rb * 128 + wave * 32 + r;
    const int orow = min(o_lane, n_out - 1);
    // scale-after form: the thread fetches the scales of row `grow` for two of every PW groups
    const int grow = min(rb * 128 + (tid & 127), n_out - 1);
    const int ghalf = tid >> 7;

    f16v acc[NB];  // running result
    f16v accg[NB]; // partial sum of the current group (SA only): every K step starts it from zero
#pragma unroll
    for (int nb = 0; nb < NB; nb++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[nb][i] = 0.f;
    constexpr int KPG = G / KSTEP > 0 ? G / KSTEP : 1; // K iterations per group
    // this block's slice of K, in whole groups
    const int ks = blockIdx.z;
    const int n_grp = n_k / KPG;
    // slices start on an even group: the scales are fetched as aligned pairs
    const int kit0 = ((int)((long)n_grp * ks / KS) & ~1) * KPG;
    const int kit1 = ks + 1 == KS ? n_k : ((int)((long)n_grp * (ks + 1) / KS) & ~1) * KPG;
    const int n_it = kit1 - kit0;

    struct WStage {
        uint4 w[W];
        int32_t z;
        float s;  // this lane's row, scaled form only
    };
    const void *qw_base = M.qweight;
    const void *qz_base = M.qzeros;
    const void *sc_base = M.scales;
    auto fetch_w = [&](int kit, WStage &d) {
        const int kc = min(kit, kit1 - 1);
        const int g = (kc * KSTEP + 32 * h) / G;
#pragma unroll
        for (int sw = 0; sw < W; sw++)
            d.w[sw] = ld_at<uint4>(qw_base, (uint32_t)(orow * C4 + kc * (2 * W) + 2 * sw + h) << 4);
        if constexpr (SA) {
            d.z = 0, d.s = 0.f; // scale-after form: zero points and scales travel by the block, PW groups at a time
        } else {
            d.z = ld_at<int32_t>(qz_base, (uint32_t)((orow >> 3) * groups + g) << 2);
            d.s = ld_at<float>(sc_base, (uint32_t)(orow * groups + g) << 2);
        }
    };
    // Scale-after form: one 8-byte load per thread and PW K steps (a K step is a group there) instead of
    // one scattered 4-byte load per thread and step.  Block j of PW groups starts at group kit0 + PW * j;
    // pairs past the row's last group re-read its last pair (their steps are never run).
    static_assert(!SA || KPG == 1, "scale-after form: a K step is one group");
    auto fetch_gs = [&](int j) {
        const int ge = min(kit0 + PW * j + 2 * ghalf, groups - 2);
        return ld_at<float2>(sc_base, (uint32_t)(grow * groups + ge) << 2);
    };
    auto store_gs = [&](int j, const float2 v) {
        gsc[j & 1][2 * ghalf][tid & 127] = v.x;
        gsc[j & 1][2 * ghalf + 1][tid & 127] = v.y;
    };
    // zero points of the same PW groups: 16 row groups x PW words per block; every wave fetches the same 64
    // words (no load under a branch), lane -> (row group lane / 4, group lane % 4)
    const int zrg = min(rb * 16 + (lane >> 2), (n_out - 1) >> 3);
    auto fetch_zs = [&](int j) {
        const int ge = min(kit0 + PW * j + (lane & 3), groups - 1);
        return ld_at<int32_t>(qz_base, (uint32_t)(zrg * groups + ge) << 2);
    };
    auto store_zs = [&](int j, const int32_t v) { zsc[j & 1][lane & 3][lane >> 2] = v; };
    // staging map: thread -> (token, 16-byte segment) x (TN*8/256) pieces
    constexpr int SEGS = KSTEP / 8; // 16-byte segments per token and K step
    constexpr int PIECES = TN * SEGS / 256;
    struct XStage {
        uint4 v[PIECES];
    };
    uint32_t xoff[PIECES]; // byte offset of this thread's pieces within a K step
#pragma unroll
    for (int p = 0; p < PIECES; p++) {
        const int idx = p * 256 + tid;
        const int t = idx / SEGS, seg = idx % SEGS;
        xoff[p] = ((uint32_t)min(t0 + t, B - 1) * (uint32_t)in + seg * 8) * 2u;
    }
    auto fetch_x = [&](int kit, XStage &d) {
        const uint32_t kb = (uint32_t)min(kit, kit1 - 1) * (uint32_t)(KSTEP * 2);
#pragma unroll
        for (int p = 0; p < PIECES; p++) d.v[p] = ld_at<uint4>(xh, xoff[p] + kb);
    };
    auto store_x = [&](int buf, const XStage &d) {
#pragma unroll
        for (int p = 0; p < PIECES; p++) {
            const int idx = p * 256 + tid;
            const int t = idx / SEGS, seg = idx % SEGS;
            *reinterpret_cast<uint4 *>(xs + ((size_t)buf * TN + t) * kXRow + seg * 8) = d.v[p];
        }
    };

    XStage xr[XP];
    WStage wr[WR];
    float2 gs2 = make_float2(0.f, 0.f);
    int32_t zs2 = 0;
    if constexpr (SA) gs2 = fetch_gs(0), zs2 = fetch_zs(0);
#pragma unroll
    for (int j = 0; j < XP; j++) fetch_x(kit0 + j, xr[j]);
#pragma unroll
    for (int j = 0; j < WR; j++) fetch_w(kit0 + j, wr[j]);
    __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0): the loop's waits then reflect its own order only
    store_x(0, xr[0]);
    if constexpr (SA) store_gs(0, gs2), store_zs(0, zs2);
    __syncthreads();

    // One K step; u = step % PW indexes the register rings (a compile-time constant where it is called).
    auto k_step = [&](const int stepi, const int u) __attribute__((always_inline)) {
        {
            const int base = stepi - u;
            const int kit = kit0 + stepi;
            const int buf = u & 1; // PW is even: the parity of the step
            // this step's weights -> registers of their own, then refill the slot
            const int zword = SA ? zsc[(stepi / PW) & 1][u][(wave * 32 + r) >> 3] : wr[u % WR].z;
            const int zn = (zword >> (4 * (orow & 7))) & 15;
            DequantConsts dc;
            dc.mask_lo = 0x000F000Fu, dc.mask_hi = 0x00F000F0u, dc.magic = 0x64006400u;
            const _Float16 off = (_Float16)(-(1024.0f + (float)(zn + 1)));
            const _Float16 off16 = (_Float16)(-(64.0f + (float)(zn + 1)));
            dc.neg_off = h2{off, off};
            dc.neg_off16 = h2{off16, off16};
            dc.sixteenth = h2{(_Float16)0.0625f, (_Float16)0.0625f};
            const _Float16 s1 = (_Float16)wr[u % WR].s;
            const h2 s16 = h2{s1, s1};
            uint32_t wd[W][4];
#pragma unroll
            for (int sw = 0; sw < W; sw++) {
                wd[sw][0] = wr[u % WR].w[sw].x, wd[sw][1] = wr[u % WR].w[sw].y, wd[sw][2] = wr[u % WR].w[sw].z, wd[sw][3] = wr[u % WR].w[sw].w;
                asm volatile("" : "+v"(wd[sw][0]), "+v"(wd[sw][1]), "+v"(wd[sw][2]), "+v"(wd[sw][3])::"memory");
            }
            // The ring slot stays in its own registers up to here (the copies above live elsewhere), so the
            // refill can land in them: otherwise the copy takes the slot's registers over, the refill goes to
            // fresh ones and is copied back at the loop's end, behind a wait for the load just issued.
#pragma unroll
            for (int sw = 0; sw < W; sw++)
                asm volatile("" : "+v"(wr[u % WR].w[sw].x), "+v"(wr[u % WR].w[sw].y), "+v"(wr[u % WR].w[sw].z), "+v"(wr[u % WR].w[sw].w));
            if constexpr (!SA) asm volatile("" : "+v"(wr[u % WR].z));
            __builtin_amdgcn_sched_barrier(0);
            // The refills of this step (ring slot u of the weights, slot u % XP of the activations, once per
            // round the next PW groups' scales and zero points) are issued one at a time between the MFMA
            // steps below: a global load takes the wave hundreds of cycles to issue when the address unit is
            // busy, and issued in one burst here those cycles stood in front of the first MFMA.
            const int kc_w = min(kit + WR, kit1 - 1);
            const uint32_t kb_x = (uint32_t)min(kit + XP, kit1 - 1) * (uint32_t)(KSTEP * 2);
            constexpr int NL = W + 1 + PIECES + 1;
            auto refill = [&](const int i) __attribute__((always_inline)) {
                if (i < PIECES) { // the activations first: the end of the step waits for them, not for what follows
                    xr[u % XP].v[i] = ld_at<uint4>(xh, xoff[i] + kb_x);
                } else if (i < PIECES + W) {
                    wr[u % WR].w[i - PIECES] =
                        ld_at<uint4>(qw_base, (uint32_t)(orow * C4 + kc_w * (2 * W) + 2 * (i - PIECES) + h) << 4);
                } else if (i == PIECES + W) {
                    if constexpr (!SA) {
                        const int g = (kc_w * KSTEP + 32 * h) / G;
                        wr[u % WR].z = ld_at<int32_t>(qz_base, (uint32_t)((orow >> 3) * groups + g) << 2);
                        wr[u % WR].s = ld_at<float>(sc_base, (uint32_t)(orow * groups + g) << 2);
                    }
                } else if (SA && u == 0) {
                    gs2 = fetch_gs(base / PW + 1), zs2 = fetch_zs(base / PW + 1);
                }
            };
            const _Float16 *xb = xs + (size_t)buf * TN * kXRow;
            // W * 4 steps of 16 k.  The operands of step i + 1 (two LDS reads per token tile, the
            // dequantised weights) are produced while the MFMAs of step i run: without this the
            // LDS latency stands in front of every MFMA.
            constexpr int NSTEP = W * 4;
            h8 aq[2], bq[2][NB];
            auto produce = [&](int step, int slot) {
                const int sw = step >> 2, j = step & 3;
#pragma unroll
                for (int nb = 0; nb < NB; nb++)
                    bq[slot][nb] = *reinterpret_cast<const h8 *>(xb + (size_t)(nb * 32 + r) * kXRow +
                                                                 (sw * 8 + 4 * h + j) * 8);
                aq[slot] = dequant8<!SA>(wd[sw][j], dc, s16);
            };
            produce(0, 0);
            // The wave that has its MFMAs to issue goes first on its SIMD; the other wave there is in its fold, its
            // tile store or at its barrier (q|k|v at 512 tokens 68 -> 64 us, the other launches 1-4 %).
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int step = 0; step < NSTEP; step++) {
#pragma unroll
                for (int i = step * NL / NSTEP; i < (step + 1) * NL / NSTEP; i++) refill(i);
                if (step + 1 < NSTEP) produce(step + 1, (step + 1) & 1);
#pragma unroll
                for (int nb = 0; nb < NB; nb++) {
                    if (SA) // a K step is one group: its first MFMA starts from zero, so the fold below clears nothing
                        accg[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aq[step & 1], bq[step & 1][nb],
                                                                          step == 0 ? f16v{} : accg[nb], 0, 0, 0);
                    else
                        acc[nb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(aq[step & 1], bq[step & 1][nb], acc[nb], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_s_setprio(0);
            if (SA && (u + 1) % KPG == 0) {
                // end of a group: fold its partial sum into the result with the fp32 scale of each row
                const int gb = (base / PW) & 1;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const float4 sv = *reinterpret_cast<const float4 *>(&gsc[gb][u][wave * 32 + q * 8 + h * 4]);
                    const float svv[4] = {sv.x, sv.y, sv.z, sv.w};
#pragma unroll
                    for (int nb = 0; nb < NB; nb++)
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            acc[nb][4 * q + e] = fmaf(svv[e], accg[nb][4 * q + e], acc[nb][4 * q + e]);
                }
                if (u == PW - 1) store_gs(base / PW + 1, gs2), store_zs(base / PW + 1, zs2); // fetched at the round's first step
            }
            // the next step's activation tile was fetched XP - 1 steps ago
            store_x(buf ^ 1, xr[(u + 1) % XP]);
            __syncthreads();
        }
    };
    // Whole rounds of PW steps in the loop, the remaining steps straight-line after it: an exit from the
    // middle of the unrolled body makes the compiler copy ring registers at the loop's end, and every copy
    // waits for its load, which drains the prefetch once per round.
    const int n_full = n_it / PW, n_rem = n_it - n_full * PW;
    for (int bi = 0; bi < n_full; bi++) {
#pragma unroll
        for (int u = 0; u < PW; u++) k_step(bi * PW + u, u);
    }
#pragma unroll
    for (int u = 0; u < PW - 1; u++)
        if (u < n_rem) k_step(n_full * PW + u, u);

    // C layout: lane (col n = l%32 -> token, h = l/32), register i -> row (i/4)*8 + h*4 + i%4.
    // Stored as it stands, every store instruction would touch 64 separate 16-byte pieces; instead each
    // wave turns its 32 rows x 32 tokens through LDS (the activation buffers are free now) so that a
    // store instruction writes 8 tokens x 128 contiguous bytes.
    const Q4Epi &E = L.e;
    // workspace of matrix mi starts after those of the matrices before it
    size_t ws_base = 0;
    for (int i = 0; i < mi; i++) ws_base += (size_t)KS * B * L.m[i].out;
    const int obase = rb * 128 + wave * 32;
    constexpr int kTRow = 36; // floats per staged token row: 32 + 4 pad (16-byte reads of 8 lanes per token)
    float *tile = reinterpret_cast<float *>(xs) + wave * 32 * kTRow; // 4.5 KB per wave
    const int tl = lane >> 3, oc = (lane & 7) * 4; // read-back map: token within a pass of 8, 4 rows
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
#pragma unroll
        for (int q = 0; q < 4; q++)
            *reinterpret_cast<float4 *>(&tile[r * kTRow + q * 8 + h * 4]) =
                make_float4(acc[nb][4 * q + 0], acc[nb][4 * q + 1], acc[nb][4 * q + 2], acc[nb][4 * q + 3]);
        // the wave reads what the wave wrote: no block barrier, the LDS queue of a wave is in order
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            const int tt = pass * 8 + tl;
            float4 v = *reinterpret_cast<const float4 *>(&tile[tt * kTRow + oc]);
            const int t = t0 + nb * 32 + tt;
            const int o = obase + oc;
            if (t >= B || o >= n_out) continue;
            const size_t row = (size_t)t * n_out;
            if (KS > 1 || partials) { // partial tile of this K slice
                *reinterpret_cast<float4 *>(ws + ws_base + ((size_t)ks * B + t) * n_out + o) = v;
                continue;
            }
            const float scale_t = ss ? ss[t] : 1.0f;
            v.x *= scale_t, v.y *= scale_t, v.z *= scale_t, v.w *= scale_t;
            if (E.kind == Q4_EPI_RESIDUAL) {
                const float4 rr = *reinterpret_cast<const float4 *>(E.res + row + o);
                v.x += rr.x;
                v.y += rr.y;
                v.z += rr.z;
                v.w += rr.w;
            }
            if (E.kind != Q4_EPI_SCATTER_ONLY) *reinterpret_cast<float4 *>(M.y + row + o) = v;
            const float vals[4] = {v.x, v.y, v.z, v.w};
            for (int c = 0; c < E.n_scatter; c++)
#pragma unroll
                for (int e = 0; e < 4; e++) E.sc_out[c][row + E.sc_idx[c][o + e]] = vals[e];
        }
    }
}

// Adds the KS partial tiles of a split-K GEMM in slice order and runs the epilogue; a thread owns four
// consecutive outputs of one token (every `out` is a multiple of 32).
// grid: (ceil(sum_out / 1024), B); the matrices of the launch are laid end to end.
__global__ __launch_bounds__(256) void q4_gemm_reduce_kernel(const Q4Launch L, const float *__restrict__ ss,
                                                             const float *__restrict__ ws, int KS) {
    const int t = blockIdx.y;
    int o = (blockIdx.x * 256 + threadIdx.x) * 4;
    int mi = 0;
    size_t ws_base = 0;
    const int B = L.batch;
    while (mi + 1 < L.n_mats && o >= L.m[mi].out) {
        o -= L.m[mi].out;
        ws_base += (size_t)KS * B * L.m[mi].out;
        mi++;
    }
    const Q4Mat &M = L.m[mi];
    if (o >= M.out) return;
    const float *p = ws + ws_base + (size_t)t * M.out + o;
    const size_t slice = (size_t)B * M.out;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int ks = 0; ks < KS; ks++) {
        const float4 a = *reinterpret_cast<const float4 *>(p + ks * slice);
        v.x += a.x, v.y += a.y, v.z += a.z, v.w += a.w;
    }
    if (ss) {
        const float sc = ss[t];
        v.x *= sc, v.y *= sc, v.z *= sc, v.w *= sc;
    }
    const Q4Epi &E = L.e;
    const size_t row = (size_t)t * M.out;
    if (E.kind == Q4_EPI_RESIDUAL) {
        const float4 r = *reinterpret_cast<const float4 *>(E.res + row + o);
        v.x += r.x, v.y += r.y, v.z += r.z, v.w += r.w;
    }
    if (E.kind != Q4_EPI_SCATTER_ONLY) *reinterpret_cast<float4 *>(M.y + row + o) = v;
    const float vals[4] = {v.x, v.y, v.z, v.w};
    for (int c = 0; c < E.n_scatter; c++) {
        const int4 idx = *reinterpret_cast<const int4 *>(E.sc_idx[c] + o);
        const int id[4] = {idx.x, idx.y, idx.z, idx.w};
#pragma unroll
        for (int e = 0; e < 4; e++) E.sc_out[c][row + id[e]] = vals[e];
    }
}

// What follows a residual projection (wo, w2) of a chunk, in one kernel instead of three: add the KS partial
// tiles in slice order and the residual (src/models.rs:263-264, 283-285), store the new residual stream,
// take its rms scale (src/models.rs:55-60), and hand fp16 copies times the norm weight to up to three
// consumers, each in its own act-order and in the pair-interleaved order the GEMM reads.
// One block of 1024 threads per token, four outputs per thread and trip; every load of a trip (residual,
// partial tiles, the consumers' indices, the norm weight) goes out before the first use.
__global__ __launch_bounds__(1024) void gemm_residual_norm_prep_kernel(const ResNormPrep A) {
    __shared__ float red[16];
    extern __shared__ _Float16 perm_h[]; // [consumer][out]: the token's row in each consumer's order
    const int t = blockIdx.x, tid = threadIdx.x;
    const int n4 = A.out >> 2;
    const size_t row = (size_t)t * A.out;
    const size_t slice = (size_t)A.B * A.out;
    float sq = 0.f;
    for (int i4 = tid; i4 < n4; i4 += 1024) {
        const float *p = A.ws + row + 4 * i4;
        float4 v = *reinterpret_cast<const float4 *>(A.res + row + 4 * i4);
        float4 part[8];
#pragma unroll
        for (int ks = 0; ks < 8; ks++) part[ks] = *reinterpret_cast<const float4 *>(p + min(ks, A.KS - 1) * slice);
        int4 idx[3];
#pragma unroll
        for (int c = 0; c < 3; c++)
            idx[c] = *reinterpret_cast<const int4 *>((c < A.n ? A.inv[c] : A.inv[0]) + 4 * i4);
        const float4 g = *reinterpret_cast<const float4 *>(A.wn + 4 * i4); // one norm weight for all consumers
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int ks = 0; ks < 8; ks++)
            if (ks < A.KS) a.x += part[ks].x, a.y += part[ks].y, a.z += part[ks].z, a.w += part[ks].w;
        v.x += a.x, v.y += a.y, v.z += a.z, v.w += a.w;
        *reinterpret_cast<float4 *>(A.x + row + 4 * i4) = v;
        sq = fmaf(v.x, v.x, sq), sq = fmaf(v.y, v.y, sq), sq = fmaf(v.z, v.z, sq), sq = fmaf(v.w, v.w, sq);
        const _Float16 vals[4] = {(_Float16)(v.x * g.x), (_Float16)(v.y * g.y), (_Float16)(v.z * g.z), (_Float16)(v.w * g.w)};
#pragma unroll
        for (int c = 0; c < 3; c++) {
            if (c >= A.n) continue;
            const int id[4] = {idx[c].x, idx[c].y, idx[c].z, idx[c].w};
            // the permutation happens in LDS: the global stores below are whole 16-byte pieces
#pragma unroll
            for (int e = 0; e < 4; e++) perm_h[c * A.out + h16_slot(id[e])] = vals[e];
        }
    }
    for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off);
    if ((tid & 63) == 0) red[tid >> 6] = sq;
    __syncthreads();
    if (tid == 0) {
        float s = 0.f;
        for (int w = 0; w < 16; w++) s += red[w];
        s /= (float)A.out;
        s += A.eps;
        A.ss[t] = 1.0f / sqrtf(s);
    }
    const int n8 = A.out >> 3;
    for (int i = tid; i < A.n * n8; i += 1024) {
        const int c = i / n8, j8 = i - c * n8;
        reinterpret_cast<uint4 *>(reinterpret_cast<_Float16 *>(A.out_h[c]) + row)[j8] =
            reinterpret_cast<const uint4 *>(perm_h + (size_t)c * A.out)[j8];
    }
}

// What follows the q|k|v projection of a chunk, in one kernel instead of two: add the KS partial tiles of
// the three matrices in slice order, apply the token's rms scale, rotate q and k (src/models.rs:100-129: the
// second half of a head uses the first half's ROTATED value), write q back and k and v into the cache rows
// of the tokens' positions (:236-249).  One block per token; thread -> (head, i < 64).
__global__ __launch_bounds__(1024) void gemm_rope_kv_kernel(const RopeKvArgs A) {
    constexpr int HS = 128, HALF = 64;
    const int b = blockIdx.x;
    const int dim = A.n_heads * HS, kv_dim = A.n_kv_heads * HS;
    const int p = A.pos[b];
    const float ss = A.ss[b];
    const float *ct = A.cos_t + (size_t)p * HALF, *st = A.sin_t + (size_t)p * HALF;
    const float *wq = A.ws + (size_t)b * dim;
    const float *wk = A.ws + (size_t)A.KS * A.B * dim + (size_t)b * kv_dim;
    const float *wv = wk + (size_t)A.KS * A.B * kv_dim;
    const size_t sq = (size_t)A.B * dim, sk = (size_t)A.B * kv_dim;
    float *kc = A.kcache + (size_t)p * kv_dim, *vc = A.vcache + (size_t)p * kv_dim;
    for (int idx = threadIdx.x; idx < A.n_heads * HALF; idx += 1024) {
        const int h = idx >> 6, i = idx & 63;
        const float c = ct[i], s = st[i];
        float qa = 0.f, qb = 0.f, ka = 0.f, kb = 0.f;
        const bool has_k = h < A.n_kv_heads;
        for (int ks = 0; ks < A.KS; ks++) {
            qa += wq[ks * sq + h * HS + i];
            qb += wq[ks * sq + h * HS + i + HALF];
            if (has_k) {
                ka += wk[ks * sk + h * HS + i];
                kb += wk[ks * sk + h * HS + i + HALF];
            }
        }
        qa *= ss, qb *= ss;
        const float first = qa * c - qb * s;
        A.q[(size_t)b * dim + h * HS + i] = first;
        A.q[(size_t)b * dim + h * HS + i + HALF] = qb * c + first * s;
        if (has_k) {
            ka *= ss, kb *= ss;
            const float kf = ka * c - kb * s;
            kc[h * HS + i] = kf;
            kc[h * HS + i + HALF] = kb * c + kf * s;
        }
    }
    for (int i = threadIdx.x; i < kv_dim; i += 1024) {
        float v = 0.f;
        for (int ks = 0; ks < A.KS; ks++) v += wv[ks * sk + i];
        vc[i] = v * ss;
    }
}

// fp32 [B][n] (already in the consumer's g_index order) -> fp16 [B][n], times the
// norm weight if given, with the (0,4,1,5,2,6,3,7) interleave inside every 8.
__global__ void prep_f16_kernel(const PrepList P, int n) {
    _Float16 *out = reinterpret_cast<_Float16 *>(P.out[blockIdx.z]);
    const float *x = P.x[blockIdx.z];
    const float *wn = P.wn[blockIdx.z];
    const int b = blockIdx.y;
    const int j8 = blockIdx.x * blockDim.x + threadIdx.x; // group of 8
    if (j8 * 8 >= n) return;
    const float4 a = reinterpret_cast<const float4 *>(x + (size_t)b * n)[j8 * 2];
    const float4 c = reinterpret_cast<const float4 *>(x + (size_t)b * n)[j8 * 2 + 1];
    float v[8] = {a.x, a.y, a.z, a.w, c.x, c.y, c.z, c.w};
    if (wn) {
        const float4 g0 = reinterpret_cast<const float4 *>(wn)[j8 * 2];
        const float4 g1 = reinterpret_cast<const float4 *>(wn)[j8 * 2 + 1];
        const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] *= g[i];
    }
    A8 o;
    o.p[0] = h2{(_Float16)v[0], (_Float16)v[4]};
    o.p[1] = h2{(_Float16)v[1], (_Float16)v[5]};
    o.p[2] = h2{(_Float16)v[2], (_Float16)v[6]};
    o.p[3] = h2{(_Float16)v[3], (_Float16)v[7]};
    reinterpret_cast<uint4 *>(out + (size_t)b * n)[j8] = make_uint4(o.u[0], o.u[1], o.u[2], o.u[3]);
}

// ss[b] = 1 / sqrt(mean(x[b]^2) + eps)   (src/models.rs:55-60)
__global__ __launch_bounds__(256) void rms_scale_kernel(float *ss, const float *x, float eps, int dim) {
    __shared__ float red[4];
    const int b = blockIdx.x;
    float s = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        const float v = x[(size_t)b * dim + i];
        s = fmaf(v, v, s);
    }
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        float t = red[0] + red[1] + red[2] + red[3];
        t /= (float)dim;
        t += eps;
        ss[b] = 1.0f / sqrtf(t);
    }
}

// silu gate (src/models.rs:92-98) for a chunk: out[b][scatter[i]] = silu(a[b][i]) * c[b][i]
__global__ void silu_scatter_kernel(float *out, const float *a, const float *c, const int32_t *scatter, int n) {
    const int b = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = a[(size_t)b * n + i];
    s = s * (1.0f / (1.0f + expf(-s)));
    s = s * c[(size_t)b * n + i];
    out[(size_t)b * n + (scatter ? scatter[i] : i)] = s;
}

// The same gate handing fp16 to the next GEMM: one block per token permutes the token's row in LDS (the
// consumer's act-order, pair-interleaved), so that the global stores are whole 16-byte pieces.
__global__ __launch_bounds__(1024) void silu_scatter_f16_kernel(_Float16 *__restrict__ out_h, const float *__restrict__ a,
                                                                const float *__restrict__ c,
                                                                const int32_t *__restrict__ scatter, int n) {
    extern __shared__ _Float16 perm_row[]; // [n]
    const size_t row = (size_t)blockIdx.x * n;
    const int tid = threadIdx.x;
    for (int i4 = tid; i4 < (n >> 2); i4 += 1024) {
        const float4 x = *reinterpret_cast<const float4 *>(a + row + 4 * i4);
        const float4 y = *reinterpret_cast<const float4 *>(c + row + 4 * i4);
        const int4 id = *reinterpret_cast<const int4 *>(scatter + 4 * i4);
        const float xs[4] = {x.x, x.y, x.z, x.w}, ys[4] = {y.x, y.y, y.z, y.w};
        const int ids[4] = {id.x, id.y, id.z, id.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            float s = xs[e];
            s = s * (1.0f / (1.0f + expf(-s)));
            perm_row[h16_slot(ids[e])] = (_Float16)(s * ys[e]);
        }
    }
    __syncthreads();
    for (int j8 = tid; j8 < (n >> 3); j8 += 1024)
        reinterpret_cast<uint4 *>(out_h + row)[j8] = reinterpret_cast<const uint4 *>(perm_row)[j8];
}

template <int G>
int launch_gemm_g(Q4Launch &L, const XhList &xh, const float *ss, float *ws, size_t ws_floats, hipStream_t st,
                  int *ks_out) {
    int total = 0;
    long rows = 0;
    for (int i = 0; i < L.n_mats; i++) {
        L.m[i].row_blocks = (L.m[i].out + 127) / 128;
        total += L.m[i].row_blocks;
        rows += L.m[i].out;
    }
    const int B = L.batch;
    // Up to 255 tokens a wave takes 64 of them: with 128 a chunk of 128 tokens is too few blocks for the chip
    // (w1|w3 of 7B: 172 blocks on 256 CUs; the launches of a 128-token chunk are 7 % slower that way).  From
    // 256 tokens on a wave takes 128 (within 256 registers: two blocks per CU): every weight is dequantised
    // once per 128 tokens instead of twice, and there are blocks enough whatever the tile (w1|w3 of 7B at 512
    // tokens: 115 against 129 us).
    const int NB = (G >= 64 && B >= 256) ? 4 : B > 32 ? 2 : 1;
    const int TN = 32 * NB;
    const int t_tiles = (B + TN - 1) / TN;
    // K slices: as many as keep the grid within one round of 2 blocks per CU, whole groups per slice, at most 4.
    // (Up to 8 fill the chip when a launch runs alone, but every slice is a partial tile that the consumer reads
    // back, and with two chunks of a prompt in flight the other chunk's kernels take the free slots: at most 4
    // measured 34.4 k against 32.7 k tok/s on the 7B prompt, 19.9 k against 19.5 k on 13B, no change on 70B, and
    // 25.1 k against 24.6 k with a single chunk in flight.)
    // K step: 128 where a group is at least that long (half the block barriers per k), else 64
    constexpr int KSTEP = G >= 128 ? 128 : 64;
    const int n_grp = (L.in / KSTEP) / (G / KSTEP > 0 ? G / KSTEP : 1);
    int KS = (2 * cu_count()) / (total * t_tiles); // all blocks resident at once: two per CU
    if (KS > 4) KS = 4;
    if (KS > n_grp / 2) KS = n_grp / 2; // slices start on even groups
    if (KS < 1) KS = 1;
    while (KS > 1 && (size_t)KS * B * rows > ws_floats) KS--;
    dim3 grid(total, t_tiles, KS), block(256);
    // the activation buffers, or the four output staging tiles of the epilogue (32 x 36 floats per wave)
    const size_t lds = std::max((size_t)2 * TN * (KSTEP + kXPad) * sizeof(_Float16), (size_t)4 * 32 * 36 * sizeof(float));
    switch (NB) {
        case 1: hipLaunchKernelGGL((q4_gemm_kernel<G, 1, KSTEP>), grid, block, lds, st, L, xh, ss, ws, KS, ks_out != nullptr); break;
        case 2: hipLaunchKernelGGL((q4_gemm_kernel<G, 2, KSTEP>), grid, block, lds, st, L, xh, ss, ws, KS, ks_out != nullptr); break;
        case 4:
            if constexpr (G >= 64) {
                static LdsLimit limit(48 * 1024);
                L2_TRY(limit.ensure(reinterpret_cast<const void *>(q4_gemm_kernel<G, 4, KSTEP>), lds));
                hipLaunchKernelGGL((q4_gemm_kernel<G, 4, KSTEP>), grid, block, lds, st, L, xh, ss, ws, KS, ks_out != nullptr);
                break;
            }
            [[fallthrough]];
        default: return l2_fail(L2_ERR_ARG, "q4 gemm: token tile");
    }
    L2_HIP(hipGetLastError());
    if (ks_out) { // the caller's own kernel adds the partial tiles
        *ks_out = KS;
        return L2_OK;
    }
    if (KS > 1) {
        hipLaunchKernelGGL(q4_gemm_reduce_kernel, dim3((unsigned)((rows + 1023) / 1024), B), dim3(256), 0, st, L, ss, ws, KS);
        L2_HIP(hipGetLastError());
    }
    return L2_OK;
}

} // namespace

int q4_gemm_launch(Q4Launch &L, const XhList &xh_list_dev, const float *ss, float *ws, size_t ws_floats,
                   hipStream_t st, int *ks_out) {
    if (L.n_mats < 1 || L.n_mats > 3) return l2_fail(L2_ERR_ARG, "q4 gemm: n_mats=%d", L.n_mats);
    if (L.in % 128 != 0 || L.in % L.group_size != 0) return l2_fail(L2_ERR_ARG, "q4 gemm: in=%d must be a multiple of 128", L.in);
    if (L.group_size >= 64 && (L.in / L.group_size) % 2 != 0)
        return l2_fail(L2_ERR_ARG, "q4 gemm: in=%d is an odd number of groups of %d", L.in, L.group_size);
    for (int i = 0; i < L.n_mats; i++)
        if (L.m[i].out % 32 != 0) return l2_fail(L2_ERR_ARG, "q4 gemm: out=%d must be a multiple of 32", L.m[i].out);
    if (L.pair) return l2_fail(L2_ERR_ARG, "q4 gemm: pair launches are not supported");
    switch (L.group_size) {
        case 32: return launch_gemm_g<32>(L, xh_list_dev, ss, ws, ws_floats, st, ks_out);
        case 64: return launch_gemm_g<64>(L, xh_list_dev, ss, ws, ws_floats, st, ks_out);
        case 128: return launch_gemm_g<128>(L, xh_list_dev, ss, ws, ws_floats, st, ks_out);
    }
    return l2_fail(L2_ERR_ARG, "q4 gemm: group size %d", L.group_size);
}

bool q4_gemm_supports(int in, int out, int group_size) {
    if (in % 128 != 0 || out % 32 != 0 || group_size <= 0 || in % group_size != 0) return false;
    // groups of 64 and 128: the group scales are fetched as aligned pairs
    return group_size < 64 || (in / group_size) % 2 == 0;
}

int prep_f16_multi_launch(const PrepList &P, int n, int B, hipStream_t st) {
    if (n % 8 || P.n_mats < 1 || P.n_mats > 3) return l2_fail(L2_ERR_ARG, "prep: n=%d, %d vectors", n, P.n_mats);
    hipLaunchKernelGGL(prep_f16_kernel, dim3((n / 8 + 255) / 256, B, P.n_mats), dim3(256), 0, st, P, n);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int prep_f16_launch(void *out_f16, const float *x, const float *wn, int n, int B, hipStream_t st) {
    PrepList P{};
    P.out[0] = out_f16, P.x[0] = x, P.wn[0] = wn, P.n_mats = 1;
    return prep_f16_multi_launch(P, n, B, st);
}

int rms_scale_launch(float *ss, const float *x, float eps, int dim, int B, hipStream_t st) {
    hipLaunchKernelGGL(rms_scale_kernel, dim3(B), dim3(256), 0, st, ss, x, eps, dim);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int silu_scatter_launch(float *out, void *out_f16, const float *a, const float *c, const int32_t *scatter, int n,
                        int B, hipStream_t st) {
    if (out_f16) {
        if (!scatter || n % 8 || (size_t)n * 2 > 60 * 1024)
            return l2_fail(L2_ERR_ARG, "silu gate (fp16): n=%d needs a permutation and at most 60 KB of LDS", n);
        static LdsLimit limit(48 * 1024);
        L2_TRY(limit.ensure(reinterpret_cast<const void *>(silu_scatter_f16_kernel), (size_t)n * 2));
        hipLaunchKernelGGL(silu_scatter_f16_kernel, dim3(B), dim3(1024), (size_t)n * 2, st, (_Float16 *)out_f16, a, c, scatter, n);
    } else {
        hipLaunchKernelGGL(silu_scatter_kernel, dim3((n + 255) / 256, B), dim3(256), 0, st, out, a, c, scatter, n);
    }
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int gemm_residual_norm_prep_launch(const ResNormPrep &A, hipStream_t st) {
    if (A.KS < 1 || A.KS > 8 || A.out % 4 || A.n < 0 || A.n > 3)
        return l2_fail(L2_ERR_ARG, "residual epilogue: %d slices, %d outputs, %d consumers", A.KS, A.out, A.n);
    if (A.n == 0) return l2_fail(L2_ERR_ARG, "residual epilogue: no consumer");
    const size_t lds = (size_t)A.n * A.out * sizeof(_Float16);
    if (A.out % 8 || lds > 60 * 1024) return l2_fail(L2_ERR_ARG, "residual epilogue: %d outputs x %d consumers", A.out, A.n);
    static LdsLimit limit(48 * 1024);
    L2_TRY(limit.ensure(reinterpret_cast<const void *>(gemm_residual_norm_prep_kernel), lds));
    hipLaunchKernelGGL(gemm_residual_norm_prep_kernel, dim3(A.B), dim3(1024), lds, st, A);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int gemm_rope_kv_launch(const RopeKvArgs &A, hipStream_t st) {
    if (A.KS < 1 || A.KS > 8 || A.B < 1 || A.n_heads < A.n_kv_heads)
        return l2_fail(L2_ERR_ARG, "q|k|v epilogue: %d slices, %d tokens", A.KS, A.B);
    hipLaunchKernelGGL(gemm_rope_kv_kernel, dim3(A.B), dim3(1024), 0, st, A);
    L2_HIP(hipGetLastError());
    return L2_OK;
}
