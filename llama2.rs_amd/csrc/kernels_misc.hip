// The per-token kernels around the q4 matvec: embedding gather, RoPE + KV-cache
// write for prefill chunks, the fp32 classifier with RMSNorm in front
// and the argmax behind, and the greedy loop's token hand-over.  gfx950, wave64.
//
// This file is compiled with -ffp-contract=off: wherever the reference rounds
// a product before adding (Rust never fuses), so does this code; FMAs appear
// only where written as fmaf().
//
// "scatter" arguments are inverse act-order permutations: a producer writes
// element i of its result to slot inv[i] of the buffer the next QLinear reads,
// which is that layer's x[g_index[j]] gather (src/gptq.rs:110-114) done once
// at the source instead of once per consumer block.
#include "l2_internal.h"

namespace {

template <int CTRL>
__device__ __forceinline__ float dpp_xchg(float v) {
    int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true);
    return __builtin_bit_cast(float, r);
}

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

// Block-wide sum / max for blocks of up to 1024 threads; `red` holds 16 floats.
__device__ __forceinline__ float block_sum(float v, float *red) {
    v = wave_sum(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float s = 0.f;
    for (int i = 0; i < nw; i++) s += red[i];
    return s;
}

__device__ __forceinline__ float block_max(float v, float *red) {
    v = wave_max(v);
    const int wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float s = red[0];
    for (int i = 1; i < nw; i++) s = fmaxf(s, red[i]);
    return s;
}

// x[b] = token_embedding_table[token[b]]  (src/models.rs:189-191), also written
// in the input order of the first layer's q, k and v projections.  Starts a
// forward pass, so it also clears the running argmax.
__global__ void embed_kernel(float *x, const float *emb, const int32_t *tokens, int dim, ScatterTargets t,
                             unsigned long long *amax) {
    const int b = blockIdx.y;
    const float *src = emb + (size_t)tokens[b] * dim;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < dim) {
        const float v = src[i];
        x[(size_t)b * dim + i] = v;
        for (int c = 0; c < t.n; c++) t.out[c][(size_t)b * dim + t.inv[c][i]] = v;
    }
    if (amax && b == 0 && i == 0) amax[0] = 0ull;
}

// out[b][j] = x[b][g_index[j]]  (src/gptq.rs:110-114), for callers that hand the
// operator an input in natural order.
__global__ void gather_kernel(float *out, const float *x, const int32_t *g_index, int n) {
    const int b = blockIdx.y;
    const int j = blockIdx.x * blockDim.x + threadIdx.x;
    if (j < n) out[(size_t)b * n + j] = x[(size_t)b * n + g_index[j]];
}

// rope (src/models.rs:100-129) on q in place and on k while it is copied into
// the cache, v copied beside it (:236-249).  The second half of a head uses the
// first half's ROTATED value, as the reference's in-place loop does.
// One block per (batch column); thread -> (head, i < half).
__global__ void rope_kv_kernel(float *q, const float *k, const float *v, const int32_t *pos,
                               const float *cos_t, const float *sin_t, float *kcache, float *vcache,
                               int n_heads, int n_kv_heads, int head_size) {
    const int b = blockIdx.x;
    const int half = head_size >> 1;
    const int dim = n_heads * head_size, kv_dim = n_kv_heads * head_size;
    const int p = pos[b];
    const float *ct = cos_t + (size_t)p * half;
    const float *st = sin_t + (size_t)p * half;
    float *qb = q + (size_t)b * dim;
    const float *kb = k + (size_t)b * kv_dim;
    const float *vb = v + (size_t)b * kv_dim;
    float *kc = kcache + (size_t)p * kv_dim;
    float *vc = vcache + (size_t)p * kv_dim;
    for (int idx = threadIdx.x; idx < n_heads * half; idx += blockDim.x) {
        const int h = idx / half, i = idx - h * half;
        const float c = ct[i], s = st[i];
        float *qh = qb + h * head_size;
        const float a = qh[i], bb = qh[i + half];
        const float first = a * c - bb * s;
        const float second = bb * c + first * s;
        qh[i] = first;
        qh[i + half] = second;
        if (h < n_kv_heads) {
            const float *kh = kb + h * head_size;
            const float ka = kh[i], kb2 = kh[i + half];
            const float kf = ka * c - kb2 * s;
            const float ks = kb2 * c + kf * s;
            kc[h * head_size + i] = kf;
            kc[h * head_size + i + half] = ks;
        }
    }
    for (int i = threadIdx.x; i < kv_dim; i += blockDim.x) vc[i] = vb[i];
}


// Order-preserving key for (value, index): larger value wins, equal values ->
// larger index wins, which is util::argmax's last-index rule (src/util.rs:39-46).
__device__ __forceinline__ unsigned long long amax_key(float v, int idx) {
    if (v == 0.0f) v = 0.0f; // -0.0 and +0.0 compare equal in the reference
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return ((unsigned long long)u << 32) | (uint32_t)idx;
}

// Linear::matvec (src/model.rs:22-31): the classifier of every model and every
// projection of the model without quantisation.  One wave per row, x staged in
// LDS.  With wn set, x is first normalised as rmsnorm does (src/models.rs:53-66):
// the block stages wn[i]*x[i] and scales each output by ss = 1/sqrt(mean(x^2) +
// eps).  Epilogue, all optional: the SiLU gate out = silu(gate[o]) * out
// (src/models.rs:92-98, gate = the w1 output when this is w3), the residual
// add out = res[o] + out (:47-51), and the fold of (value, index) into a 64-bit
// maximum, one atomic per wave.  blockIdx.y is the batch column.
//
// A wave takes R rows at a time and issues all R * KI loads of 16 bytes per
// lane (32 in all) before the first FMA, every load unconditional: columns past
// the end re-read the row's last 16 bytes against a zero of x, rows past the
// end re-read the last row.  Inputs longer than 32 * 64 float4 take several
// such passes over a row (R = 1) into the same accumulator.
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int KI> // float4 per lane, row and pass
__global__ __launch_bounds__(256) void dense_matvec_kernel(const DenseArgs A) {
    constexpr int R = 32 / KI >= 1 ? 32 / KI : 1;
    extern __shared__ float xs[]; // n_pass * KI * 64 float4, zero beyond in
    __shared__ float red[16];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // uniform: row addresses stay scalar
    const int in = A.in, out = A.out;
    const int n4 = in >> 2;
    const int n_pass = A.n_pass;
    const int padded = n_pass * KI * 64;
    const size_t bcol = blockIdx.y;
    const float *__restrict__ x = A.x + bcol * in;
    const float *__restrict__ wn = A.wn;
    const float4 *__restrict__ w4 = reinterpret_cast<const float4 *>(A.w);
    const float4 *__restrict__ xs4 = reinterpret_cast<const float4 *>(xs);

    float ssq = 0.f;
    for (int base = 0; base < padded; base += 256) {
        const int i = base + tid;
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (i < n4) {
            v = reinterpret_cast<const float4 *>(x)[i];
            if (wn) {
                const float4 g = reinterpret_cast<const float4 *>(wn)[i];
                ssq = fmaf(v.x, v.x, ssq);
                ssq = fmaf(v.y, v.y, ssq);
                ssq = fmaf(v.z, v.z, ssq);
                ssq = fmaf(v.w, v.w, ssq);
                v.x *= g.x;
                v.y *= g.y;
                v.z *= g.z;
                v.w *= g.w;
            }
        }
        if (i < padded) reinterpret_cast<float4 *>(xs)[i] = v;
    }
    float ss = 1.0f;
    if (wn) {
        ssq = block_sum(ssq, red);
        ssq /= (float)in;
        ssq += A.eps;
        ss = 1.0f / sqrtf(ssq);
    }
    __syncthreads();

    const int waves_total = gridDim.x * 4;
    const int o_first = (blockIdx.x * 4 + wave) * R;
    float4 wv[R][KI];
    auto load_tile = [&](int o, int pass) {
#pragma unroll
        for (int k = 0; k < R; k++) {
            // 32-bit byte offsets from the one base (the launcher checks that the matrix stays below 4 GiB)
            const uint32_t row = (uint32_t)min(o + k, out - 1) * ((uint32_t)n4 << 4);
#pragma unroll
            for (int i = 0; i < KI; i++) {
                const uint32_t col = (uint32_t)min((pass * KI + i) * 64 + lane, n4 - 1) << 4;
                // read once per token: non-temporal, so that the rows do not displace what is re-read
                wv[k][i] = __builtin_bit_cast(float4, __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(
                                                          reinterpret_cast<const char *>(w4) + (row + col))));
            }
        }
    };
    unsigned long long key = 0ull;
    float *__restrict__ y = A.y + bcol * out;
    const float *__restrict__ res = A.res ? A.res + bcol * out : nullptr;
    const float *__restrict__ gate = A.gate ? A.gate + bcol * out : nullptr;
    for (int o = o_first; o < out; o += waves_total * R) {
        float a[R];
#pragma unroll
        for (int k = 0; k < R; k++) a[k] = 0.f;
        for (int pass = 0; pass < n_pass; pass++) {
            __builtin_amdgcn_sched_barrier(0); // a pass's loads stay behind the pass before it: one set of registers
            load_tile(o, pass);
            __builtin_amdgcn_sched_barrier(0); // every load of the pass before its first FMA
#pragma unroll
            for (int i = 0; i < KI; i++) {
                const float4 xx = xs4[(pass * KI + i) * 64 + lane];
#pragma unroll
                for (int k = 0; k < R; k++) {
                    a[k] = fmaf(wv[k][i].x, xx.x, a[k]);
                    a[k] = fmaf(wv[k][i].y, xx.y, a[k]);
                    a[k] = fmaf(wv[k][i].z, xx.z, a[k]);
                    a[k] = fmaf(wv[k][i].w, xx.w, a[k]);
                }
            }
        }
#pragma unroll
        for (int k = 0; k < R; k++) {
            float v = wave_sum(a[k]) * ss;
            if (lane == 0 && o + k < out) {
                if (gate) {
                    const float g = gate[o + k];
                    v = (g * (1.0f / (1.0f + expf(-g)))) * v;
                }
                if (res) v = res[o + k] + v;
                y[o + k] = v;
                const unsigned long long kk = amax_key(v, o + k);
                key = kk > key ? kk : key;
            }
        }
    }
    if (lane == 0 && A.amax && key) atomicMax(A.amax, key);
}

// Greedy hand-over (src/inference.rs:154-162, 185-189): next is the forced
// prompt token while pos < n_prompt, else the argmax; it is recorded, fed back
// as the next input token, and the position advances -- all without the host.
__global__ void next_token_kernel(const unsigned long long *amax, const int32_t *prompt, int n_prompt,
                                  int32_t *dpos, int32_t *out_ids, int pos0, int32_t *tok,
                                  const int32_t *loop_params) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        if (loop_params) {
            n_prompt = loop_params[0];
            pos0 = loop_params[1];
        }
        const int pos = dpos[0];
        const int32_t next = pos < n_prompt ? prompt[pos] : (int32_t)(amax[0] & 0xFFFFFFFFull);
        if (out_ids) out_ids[pos - pos0] = next;
        tok[0] = next;
        dpos[0] = pos + 1;
    }
}

__global__ void set_i32_kernel(int32_t *p, int32_t a, int32_t *q, int32_t b) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        p[0] = a;
        if (q) q[0] = b;
    }
}

__global__ void fill_pattern_kernel(float *p, size_t n, uint64_t seed) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t z = seed + 0x9E3779B97F4A7C15ull * (i + 1);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    p[i] = (float)((double)(z >> 11) * (1.0 / 9007199254740992.0) * 2.0 - 1.0);
}

} // namespace

int embed_launch(float *x, const float *emb, const int32_t *tokens, int dim, int B, const ScatterTargets &t,
                 unsigned long long *amax_key, hipStream_t st) {
    if (t.n < 0 || t.n > 3) return l2_fail(L2_ERR_ARG, "embed: %d targets", t.n);
    hipLaunchKernelGGL(embed_kernel, dim3((dim + 255) / 256, B), dim3(256), 0, st, x, emb, tokens, dim, t, amax_key);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int gather_launch(float *out, const float *x, const int32_t *g_index, int n, int B, hipStream_t st) {
    hipLaunchKernelGGL(gather_kernel, dim3((n + 255) / 256, B), dim3(256), 0, st, out, x, g_index, n);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int rope_kv_launch(float *q, const float *k, const float *v, const int32_t *pos, const float *cos_t,
                   const float *sin_t, float *kcache_l, float *vcache_l, int n_heads, int n_kv_heads,
                   int head_size, int B, hipStream_t st) {
    hipLaunchKernelGGL(rope_kv_kernel, dim3(B), dim3(1024), 0, st, q, k, v, pos, cos_t, sin_t, kcache_l,
                       vcache_l, n_heads, n_kv_heads, head_size);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int dense_launch(const DenseArgs &a0, hipStream_t st) {
    DenseArgs a = a0;
    if (a.in < 4 || a.in % 4 || a.in > 32768 || a.out < 1 || a.batch < 1 ||
        (size_t)a.in * a.out * 4 >= ((size_t)1 << 32))
        return l2_fail(L2_ERR_ARG, "dense matvec: in=%d out=%d batch=%d", a.in, a.out, a.batch);
    if (a.amax && a.batch != 1) return l2_fail(L2_ERR_ARG, "dense matvec: the running maximum takes one column");
    const int ki = (a.in / 4 + 63) / 64; // float4 per lane and row
    const int KI = ki <= 4 ? 4 : ki <= 8 ? 8 : ki <= 16 ? 16 : ki <= 20 ? 20 : 32;
    const int R = 32 / KI >= 1 ? 32 / KI : 1;
    a.n_pass = (ki + KI - 1) / KI;
    // One column (the classifier of a decode step): one block per CU -- 7B 93 -> 85 us, 13B 112 -> 103, 70B 172 ->
    // 161 against three per CU, which the registers would allow and which stays the rule for several columns.
    // Fewer when the rows run out.
    const int per_cu = a.batch == 1 ? 1 : 3;
    int blocks = (per_cu * cu_count() + a.batch - 1) / a.batch;
    const int need = (a.out + 4 * R - 1) / (4 * R);
    if (blocks > need) blocks = need;
    const size_t lds = (size_t)a.n_pass * KI * 64 * 16;
    dim3 grid(blocks, a.batch), block(256);
    if (lds > 48 * 1024) { // only rows of more than one pass, which run with KI = 32
        if (KI != 32) return l2_fail(L2_ERR_ARG, "dense matvec: in=%d out=%d needs %zu B of LDS with %d loads per pass", a.in, a.out, lds, KI);
        static LdsLimit limit;
        L2_TRY(limit.ensure(reinterpret_cast<const void *>(dense_matvec_kernel<32>), lds));
    }
    switch (KI) {
        case 4: hipLaunchKernelGGL(dense_matvec_kernel<4>, grid, block, lds, st, a); break;
        case 8: hipLaunchKernelGGL(dense_matvec_kernel<8>, grid, block, lds, st, a); break;
        case 16: hipLaunchKernelGGL(dense_matvec_kernel<16>, grid, block, lds, st, a); break;
        case 20: hipLaunchKernelGGL(dense_matvec_kernel<20>, grid, block, lds, st, a); break;
        default: hipLaunchKernelGGL(dense_matvec_kernel<32>, grid, block, lds, st, a); break;
    }
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int dense_matvec_launch(float *y, const float *w, const float *x, const float *wn, float eps, int in, int out,
                        unsigned long long *amax_key, hipStream_t st) {
    DenseArgs a{};
    a.y = y, a.w = w, a.x = x, a.wn = wn, a.eps = eps, a.in = in, a.out = out, a.amax = amax_key, a.batch = 1;
    return dense_launch(a, st);
}

int next_token_launch(const unsigned long long *amax_key, const int32_t *prompt, int n_prompt,
                      int32_t *dpos, int32_t *out_ids, int pos0, int32_t *tok, hipStream_t st,
                      const int32_t *loop_params) {
    hipLaunchKernelGGL(next_token_kernel, dim3(1), dim3(64), 0, st, amax_key, prompt, n_prompt, dpos,
                       out_ids, pos0, tok, loop_params);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int set_i32_launch(int32_t *p, int32_t a, int32_t *q, int32_t b, hipStream_t st) {
    hipLaunchKernelGGL(set_i32_kernel, dim3(1), dim3(64), 0, st, p, a, q, b);
    L2_HIP(hipGetLastError());
    return L2_OK;
}

int fill_pattern_launch(float *p, size_t n, uint64_t seed, hipStream_t st) {
    hipLaunchKernelGGL(fill_pattern_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p, n, seed);
    L2_HIP(hipGetLastError());
    return L2_OK;
}
