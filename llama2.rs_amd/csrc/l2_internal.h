// Internal declarations shared by the host code and the kernel launchers.
// Not part of the C ABI (that is include/llama2_hip.h).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stddef.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <string>
#include <type_traits>
#include <vector>

#include "../../include/llama2_hip.h"
#include "../../include/llama2_hip_bench.h"

// Compute units of the current device (256 on MI355X); asked once.
inline int cu_count() {
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

// ---- error plumbing -------------------------------------------------------
int l2_fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define L2_HIP(call)                                                                     \
    do {                                                                                 \
        hipError_t e_ = (call);                                                          \
        if (e_ != hipSuccess)                                                            \
            return l2_fail(L2_ERR_HIP, "%s: %s (%s:%d)", #call, hipGetErrorString(e_),   \
                           __FILE__, __LINE__);                                          \
    } while (0)

#define L2_TRY(call)            \
    do {                        \
        int rc_ = (call);       \
        if (rc_ != L2_OK) return rc_; \
    } while (0)

// A kernel's dynamic-LDS limit (hipFuncAttributeMaxDynamicSharedMemorySize), raised when a launch needs more than it
// was last raised to.  One of these per kernel (a function-local static at the launch site).  The attribute belongs to
// the kernel as loaded on ONE device, so what was raised is kept per device; model handles on different host threads
// share the launch sites, so the slow path is behind a mutex and the fast path reads an atomic.
struct LdsLimit {
    static constexpr int kMaxDevices = 64;
    std::atomic<size_t> raised[kMaxDevices];
    std::mutex mu;
    explicit LdsLimit(size_t initial = 0) {
        for (auto &r : raised) r.store(initial, std::memory_order_relaxed);
    }
    int ensure(const void *kernel, size_t bytes) {
        int dev = 0;
        L2_HIP(hipGetDevice(&dev));
        if (dev < 0 || dev >= kMaxDevices) return l2_fail(L2_ERR_HIP, "device %d: more devices than the launch tables hold", dev);
        if (bytes <= raised[dev].load(std::memory_order_acquire)) return L2_OK;
        std::lock_guard<std::mutex> lock(mu);
        if (bytes <= raised[dev].load(std::memory_order_relaxed)) return L2_OK;
        L2_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
        raised[dev].store(bytes, std::memory_order_release);
        return L2_OK;
    }
};

// Position at which the prefill ladder 64/32/16/8/4/2 (src/inference.rs:78-127) leaves off.
int l2_prefill_ladder_end(int n_prompt);

// ---- device views ---------------------------------------------------------

// One QLinear resident in device memory, `.bin` layout (src/gptq.rs:68-84),
// plus the inverse of g_index so that a producer can write its output straight
// into the order this layer reads it in.
struct DevQLinear {
    const uint4 *qweight = nullptr;   // [out][in/32] chunks of 32 nibbles
    const int32_t *qzeros = nullptr;  // [out/8][groups]
    const float *scales = nullptr;    // [out][groups]
    const int32_t *g_index = nullptr; // [in]
    const int32_t *inv_index = nullptr; // [in], inv_index[g_index[j]] = j
    int in = 0, out = 0, groups = 0, group_size = 0;
    const float *dense = nullptr;     // the model without quantisation: Linear<IN,OUT>.w [out][in]; the rest null
};

// ---- q4 matvec launch description ------------------------------------------

enum {
    Q4_EPI_STORE = 0,       // y[b][o] = v (+ scatter targets)
    Q4_EPI_RESIDUAL = 1,    // v += res[b][o]; y[b][o] = v (+ scatter targets)
    Q4_EPI_SCATTER_ONLY = 2 // scatter targets only
};

struct Q4Mat {
    const uint4 *qweight;
    const int32_t *qzeros;
    const float *scales;
    const float *x;  // input already in this layer's g_index order: [B][in] (in its natural order if gidx is set)
    const int32_t *gidx; // null, or the INVERSE of this layer's g_index: x is in its natural order and the kernel puts
                         // x[b][i] where input gidx[i] of the sorted rows is read (one matrix, no rmsnorm)
    const float *wn; // rmsnorm weights in the same order, or null: x is used as it is
    float *y;        // [B][out]
    int out;
    int row_blocks;  // blocks of grid.x that belong to this matrix
};

struct Q4Epi {
    int kind;
    const float *res;          // Q4_EPI_RESIDUAL: [B][out] (may alias y)
    int n_scatter;             // 0..3
    const int32_t *sc_idx[3];  // inverse act-order permutation of a following layer
    float *sc_out[3];          // [B][out]: sc_out[t][b][sc_idx[t][o]] = v
};

struct Q4Launch {
    Q4Mat m[3];
    Q4Epi e;
    int n_mats;
    int in;      // shared by all matrices of one launch
    int groups;
    int group_size;
    int batch;
    int pair;    // 1: m[0], m[1] are w1, w3; v = silu(m0 row) * (m1 row)
    float eps;   // rmsnorm epsilon, used when wn is set
    int rows_per_block; // filled by the streaming launcher
};
// The launch description travels by value as the kernel's one argument: it must stay far inside the 4 KB a
// dispatch packet's argument block holds, and be plain data that a byte copy reproduces.
static_assert(sizeof(Q4Launch) <= 1024, "Q4Launch is passed by value as a kernel argument");
static_assert(std::is_trivially_copyable<Q4Launch>::value && std::is_standard_layout<Q4Launch>::value,
              "Q4Launch is copied byte for byte into the dispatch's argument block");

// When armed (profiling runs only), the next q4 launch goes out through
// hipExtLaunchKernel with these events, which then carry the dispatch's own
// begin and end timestamps rather than those of marker packets around it.
struct Q4ProfHook {
    hipEvent_t start = nullptr, stop = nullptr;
    bool armed = false;
};
extern thread_local Q4ProfHook g_q4_prof;

// When armed, the next q4 launch is not launched: the launcher writes the name of the kernel it would run
// (as a profiler prints it, template arguments included) into buf and disarms the hook.
struct Q4NameHook {
    char *buf = nullptr;
    int cap = 0;
    bool armed = false;
    int grid = 0, block = 0, rows_per_block = 0; // what the launch would have been
    size_t lds = 0;
};
extern thread_local Q4NameHook g_q4_name;

// Launch the fp32 dequant matvec for up to 3 matrices that share `in`
// (wq|wk|wv), or a (w1, w3) pair.  Fills row_blocks itself.
int q4_matvec_launch(Q4Launch &L, hipStream_t stream);
// The two forms of the kernel behind q4_matvec_launch.
int q4_stream_launch(Q4Launch &L, hipStream_t stream);
bool q4_stream_supports(const Q4Launch &L);
// Whether q4_matvec_launch would apply the act-order permutation itself for this launch if m[0].gidx were set (one
// matrix, no rmsnorm, the default fp32 streaming form, rows of at most four waves); otherwise the caller gathers.
bool q4_gathers_in_kernel(const Q4Launch &L);

// ---- prefill chunks through the matrix cores ---------------------------------

struct XhList {
    const void *p[3]; // per matrix of the launch: fp16 [B][in], g_index order, pair-interleaved (prep_f16_launch)
};
// Y = X W^T for a chunk of L.batch tokens; ss (per token, may be null) scales the rows of Y.
// Epilogues as in the matvec (no pair launches).  ws: workspace of ws_floats floats for split-K partial
// tiles (the launcher uses as many K slices as fit).
// ks_out given: the kernel leaves its K slices as partial tiles [KS][B][out] in ws (also when KS is 1), no
// reduction is launched, and *ks_out says how many there are.
int q4_gemm_launch(Q4Launch &L, const XhList &xh, const float *ss, float *ws, size_t ws_floats, hipStream_t st,
                   int *ks_out = nullptr);

struct ResNormPrep {
    const float *ws;   // partial tiles [KS][B][out] of one matrix
    int KS, B, out;
    const float *res;  // [B][out] residual stream in
    float *x;          // [B][out] residual stream out (may be res)
    float *ss;         // [B] rms scale of the new residual stream
    float eps;
    int n;             // consumers (1..3)
    const int32_t *inv[3]; // inverse act-order permutation of each consumer
    const float *wn;       // [out] norm weight of the consumers' rmsnorm, in the order of the residual stream
    void *out_h[3];        // [B][out] fp16, pair-interleaved, in each consumer's order
};
int gemm_residual_norm_prep_launch(const ResNormPrep &A, hipStream_t st);

struct RopeKvArgs {
    const float *ws;   // partial tiles of q, k, v laid end to end: [KS][B][dim], [KS][B][kv_dim], [KS][B][kv_dim]
    int KS, B;
    const float *ss;   // [B] rms scale of the layer's input
    const int32_t *pos;
    const float *cos_t, *sin_t;
    float *q;          // [B][dim] out
    float *kcache, *vcache; // the layer's cache: rows [pos][kv_dim]
    int n_heads, n_kv_heads; // head size 128
};
int gemm_rope_kv_launch(const RopeKvArgs &A, hipStream_t st);
bool q4_gemm_supports(int in, int out, int group_size);
// out_f16[b][j'] = fp16(x[b][j] * (wn ? wn[j] : 1)), j' = j with the order (0,4,1,5,2,6,3,7) inside every 8.
int prep_f16_launch(void *out_f16, const float *x, const float *wn, int n, int B, hipStream_t st);
// The same for up to three vectors of one length in one launch (q|k|v, w1|w3 inputs).
struct PrepList {
    void *out[3];
    const float *x[3];
    const float *wn[3];
    int n_mats;
};
int prep_f16_multi_launch(const PrepList &P, int n, int B, hipStream_t st);
int rms_scale_launch(float *ss, const float *x, float eps, int dim, int B, hipStream_t st);
// out[b][scatter[i]] = silu(a[b][i]) * c[b][i]; with out_f16 set the result goes there instead, as fp16 in
// the pair-interleaved order the GEMM reads (no separate conversion pass).
int silu_scatter_launch(float *out, void *out_f16, const float *a, const float *c, const int32_t *scatter, int n,
                        int B, hipStream_t st);
// Slot of element j of a vector in the fp16 pair-interleaved order: (0,4,1,5,2,6,3,7) inside every 8.
__host__ __device__ inline int h16_slot(int j) {
    const int e = j & 7;
    return (j & ~7) | (e < 4 ? 2 * e : 2 * (e - 4) + 1);
}

// ---- the other per-token kernels -------------------------------------------

struct ScatterTargets {
    const int32_t *inv[3];
    float *out[3];
    int n;
};

// x[b] = emb[tokens[b]], also delivered through t; clears the running argmax.
int embed_launch(float *x, const float *emb, const int32_t *tokens, int dim, int B, const ScatterTargets &t,
                 unsigned long long *amax_key, hipStream_t st);
int gather_launch(float *out, const float *x, const int32_t *g_index, int n, int B, hipStream_t st);
int rope_kv_launch(float *q, const float *k, const float *v, const int32_t *pos, const float *cos_t,
                   const float *sin_t, float *kcache_l, float *vcache_l, int n_heads, int n_kv_heads,
                   int head_size, int B, hipStream_t st);
// Batched attention over an already written cache: out[b][scatter[i]] for query b at pos[b].
int attention_launch(float *out, void *out_f16, const float *q, const float *kcache_l, const float *vcache_l,
                     const int32_t *pos, const int32_t *scatter, int n_heads, int n_kv_heads,
                     int head_size, int max_pos, int B, hipStream_t st);

// Decode attention (one query) with RoPE and the cache write folded in.
struct AttnDecode {
    const float *q;      // [dim]    raw query of this step
    const float *k_new;  // [kv_dim] raw key
    const float *v_new;  // [kv_dim] value
    float *kcache, *vcache;          // this layer: [max_seq][kv_dim]
    const float *cos_t, *sin_t;      // [max_seq][head_size/2]
    int pos;                         // position of this step (the host knows it; no device read in front of the loads)
    const int32_t *dpos;             // if set, the position is read from here instead (a captured step serves many positions)
    float *out;                      // [dim], written through scatter
    const int32_t *scatter;
    float *part;                     // split workspace: [n_heads][max_splits][130]
    int n_heads, n_kv_heads;
    int ts;                          // timesteps per split (multiple of 64)
    int n_splits;                    // grid.y; 1 = no combine pass
    int max_splits;
};
int attention_decode_launch(const AttnDecode &a, hipStream_t st);

// logits = wcls (rmsnorm(x, wn)); folds (value, index) into amax_key when set.
// wn == nullptr: plain Linear::matvec of x.
int dense_matvec_launch(float *y, const float *w, const float *x, const float *wn, float eps, int in, int out,
                        unsigned long long *amax_key, hipStream_t st);
// The general form: y[b] = epilogue(w (rmsnorm?)(x[b])) for `batch` columns (see dense_matvec_kernel).
struct DenseArgs {
    float *y;            // [batch][out]
    const float *w;      // [out][in]
    const float *x;      // [batch][in]
    const float *wn;     // [in] or null: rmsnorm weight applied to x, with eps
    float eps;
    int in, out, batch;
    unsigned long long *amax; // null, or the running (value, index) maximum (batch == 1)
    const float *res;    // null, or [batch][out] added to the result (may alias y)
    const float *gate;   // null, or [batch][out]: result = silu(gate) * result
    int n_pass;          // set by the launcher
};
int dense_launch(const DenseArgs &a, hipStream_t st);
// pos = dpos[0]; next = pos < n_prompt ? prompt[pos] : index(amax_key);
// out_ids[pos - pos0] = next; tok[0] = next; dpos[0] = pos + 1.
// With loop_params (device: {n_prompt, pos0}) those two come from there, so that one captured launch serves any loop.
int next_token_launch(const unsigned long long *amax_key, const int32_t *prompt, int n_prompt,
                      int32_t *dpos, int32_t *out_ids, int pos0, int32_t *tok, hipStream_t st,
                      const int32_t *loop_params = nullptr);
// p[0] = a; if (q) q[0] = b.  Scalars travel as kernel arguments, never as
// asynchronous copies from the caller's stack.
int set_i32_launch(int32_t *p, int32_t a, int32_t *q, int32_t b, hipStream_t st);
int fill_pattern_launch(float *p, size_t n, uint64_t seed, hipStream_t st);
