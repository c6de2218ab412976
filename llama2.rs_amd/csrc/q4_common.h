// Device helpers shared by the q4 matvec kernels (gfx950, wave64).
#pragma once

#include "l2_internal.h"

namespace q4 {

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

typedef float v2f __attribute__((ext_vector_type(2)));

// 32 nibbles of one row against 32 inputs: returns 2^-9 * sum_k n_k x_k.
//
// A nibble n parked in the low half of a byte, 0000nnnn, read as an OCP FP8
// E4M3 number is exactly n * 2^-9 (subnormal for n < 8, exponent 1 above, the
// same step on both sides), so v_cvt_pk_f32_fp8 turns two nibbles into two
// floats in one instruction.  Even nibbles come from w & 0x0F0F0F0F, odd ones
// from (w >> 4) & 0x0F0F0F0F.  The power of two is undone exactly by the
// caller.
__device__ __forceinline__ float chunk_dot(const uint4 w, const float (&x)[32]) {
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int d = 0; d < 4; d++) {
        const uint32_t l = words[d] & 0x0F0F0F0Fu;
        const uint32_t h = (words[d] >> 4) & 0x0F0F0F0Fu;
        const v2f l01 = __builtin_amdgcn_cvt_pk_f32_fp8(l, false); // nibbles 0, 2
        const v2f l23 = __builtin_amdgcn_cvt_pk_f32_fp8(l, true);  // nibbles 4, 6
        const v2f h01 = __builtin_amdgcn_cvt_pk_f32_fp8(h, false); // nibbles 1, 3
        const v2f h23 = __builtin_amdgcn_cvt_pk_f32_fp8(h, true);  // nibbles 5, 7
        a0 = fmaf(l01.x, x[8 * d + 0], a0);
        a1 = fmaf(h01.x, x[8 * d + 1], a1);
        a0 = fmaf(l01.y, x[8 * d + 2], a0);
        a1 = fmaf(h01.y, x[8 * d + 3], a1);
        a0 = fmaf(l23.x, x[8 * d + 4], a0);
        a1 = fmaf(h23.x, x[8 * d + 5], a1);
        a0 = fmaf(l23.y, x[8 * d + 6], a0);
        a1 = fmaf(h23.y, x[8 * d + 7], a1);
    }
    return a0 + a1;
}

// Stage one input vector into padded chunks + chunk sums; returns this
// thread's share of sum(x^2) (of the raw input, before the norm weight).
constexpr int kStageBatch = 4; // float4 loads of x (and of the norm weight) in flight per thread

struct StageRegs {
    float4 v[kStageBatch], g[kStageBatch];
};

// Issue the loads of batch `base` (in float4 units) into registers.
template <int NW>
__device__ __forceinline__ void stage_issue(const float *__restrict__ xin_f, const float *__restrict__ wn_f,
                                            int in, int base, int tid, StageRegs &r) {
    const float4 *xin = reinterpret_cast<const float4 *>(xin_f);
    const float4 *wn = reinterpret_cast<const float4 *>(wn_f);
    const int n4 = in >> 2;
    constexpr int T = NW * 64;
#pragma unroll
    for (int u = 0; u < kStageBatch; u++) {
        const int j4 = base + u * T + tid;
        r.v[u] = j4 < n4 ? xin[j4] : make_float4(0.f, 0.f, 0.f, 0.f);
        r.g[u] = (wn_f && j4 < n4) ? wn[j4] : make_float4(1.f, 1.f, 1.f, 1.f);
    }
}

// Consume a batch: norm weight, sum of squares, chunk sums, LDS.
template <int NW>
__device__ __forceinline__ float stage_consume(bool norm, int in, int base, int tid, StageRegs &r, float *xs,
                                               float *xsum, float ssq) {
    const int n4 = in >> 2;
    constexpr int T = NW * 64;
#pragma unroll
    for (int u = 0; u < kStageBatch; u++) {
        const int j4 = base + u * T + tid;
        float4 v = r.v[u];
        if (norm) {
            ssq = fmaf(v.x, v.x, ssq);
            ssq = fmaf(v.y, v.y, ssq);
            ssq = fmaf(v.z, v.z, ssq);
            ssq = fmaf(v.w, v.w, ssq);
            v.x *= r.g[u].x;
            v.y *= r.g[u].y;
            v.z *= r.g[u].z;
            v.w *= r.g[u].w;
        }
        // the 8 consecutive lanes that hold one chunk add up its sum
        float s = (v.x + v.y) + (v.z + v.w);
        s += dpp_xchg<0xB1>(s);  // lanes ^1
        s += dpp_xchg<0x4E>(s);  // lanes ^2
        s += dpp_xchg<0x141>(s); // 7 - lane within each 8: the other quad
        if (j4 < n4) {
            const int j = j4 << 2;
            *reinterpret_cast<float4 *>(&xs[(j >> 5) * kChunkPad + (j & 31)]) = v;
            if ((tid & 7) == 0) xsum[j >> 5] = s;
        }
    }
    return ssq;
}

// Whatever the first batch did not cover.
template <int NW>
__device__ __forceinline__ float stage_rest(const float *__restrict__ xin_f, const float *__restrict__ wn_f, int in,
                                            float *xs, float *xsum, int tid, float ssq) {
    const int n4 = in >> 2;
    constexpr int T = NW * 64;
    for (int base = T * kStageBatch; base < n4; base += T * kStageBatch) {
        StageRegs r;
        stage_issue<NW>(xin_f, wn_f, in, base, tid, r);
        ssq = stage_consume<NW>(wn_f != nullptr, in, base, tid, r, xs, xsum, ssq);
    }
    return ssq;
}

template <int NW>
__device__ __forceinline__ float stage_input(const float *__restrict__ xin_f, const float *__restrict__ wn_f,
                                             int in, float *xs, float *xsum, int tid) {
    StageRegs r;
    stage_issue<NW>(xin_f, wn_f, in, 0, tid, r);
    const float ssq = stage_consume<NW>(wn_f != nullptr, in, 0, tid, r, xs, xsum, 0.f);
    return stage_rest<NW>(xin_f, wn_f, in, xs, xsum, tid, ssq);
}

} // namespace q4
