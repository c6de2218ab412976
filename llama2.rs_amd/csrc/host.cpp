// Host side of the C ABI: checkpoint loading and upload (LlamaModel::from_file,
// src/lib.rs:45-104), RunState (src/models.rs:29-42), the layer schedule of
// transformer<B> (src/models.rs:178-298) and the greedy loop of generate
// (src/inference.rs:16-193), driving the HIP kernels.  Nothing here computes on
// the CPU except the one-time RoPE angle table and the synthetic-image
// generator.
#include <map>
#include <fcntl.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <mutex>
#include <numeric>
#include <thread>

#include "l2_internal.h"

// ---------------------------------------------------------------------------
// errors

static thread_local char g_err[512] = "";
thread_local Q4ProfHook g_q4_prof;
thread_local Q4NameHook g_q4_name;

int l2_fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char *l2_last_error(void) { return g_err; }

// ---------------------------------------------------------------------------
// dims, presets, sizes

static int64_t div_up(int64_t x, int64_t y) { return x / y + (x % y == 0 ? 0 : 1); }

static size_t qlinear_bytes(int in, int out, int g) {
    if (g == 0) return (size_t)out * in * 4; // dense Linear<IN,OUT> (src/model.rs:11-15)
    const size_t groups = (size_t)div_up(in, g);
    return (size_t)out * (in / 8) * 4 + (size_t)(out / 8) * groups * 4 + (size_t)out * groups * 4 +
           (size_t)in * 4;
}

static int check_dims(const l2_dims *d) {
    if (!d) return l2_fail(L2_ERR_ARG, "dims is null");
    if (d->dim <= 0 || d->hidden_dim <= 0 || d->n_layers <= 0 || d->n_heads <= 0 ||
        d->n_kv_heads <= 0 || d->vocab_size <= 0 || d->seq_len <= 0)
        return l2_fail(L2_ERR_ARG, "dims: non-positive field");
    // 0 is the build without quantisation (GROUPSIZE of src/constants.rs:58-61): every projection dense
    if (d->group_size != 0 && d->group_size != 32 && d->group_size != 64 && d->group_size != 128)
        return l2_fail(L2_ERR_ARG, "dims: group_size %d (32, 64, 128, or 0 for the model without quantisation)",
                       d->group_size);
    if (d->dim % d->n_heads || d->n_heads % d->n_kv_heads)
        return l2_fail(L2_ERR_ARG, "dims: heads do not divide");
    if (d->dim / d->n_heads != 128)
        return l2_fail(L2_ERR_ARG, "dims: head size %d (the kernels are built for 128)", d->dim / d->n_heads);
    if ((d->group_size && (d->dim % d->group_size || d->hidden_dim % d->group_size)) || d->dim % 32 ||
        d->hidden_dim % 32)
        return l2_fail(L2_ERR_ARG, "dims: dim and hidden_dim must be multiples of 32 and of the group size");
    return L2_OK;
}

extern "C" int l2_preset(const char *model_size, int group_size, l2_dims *out) {
    if (!model_size || !out) return l2_fail(L2_ERR_ARG, "l2_preset: null argument");
    l2_dims d;
    // src/constants.rs:7-41
    if (!strcmp(model_size, "7B"))
        d = {4096, 11008, 32, 32, 32, 32000, 2048, group_size};
    else if (!strcmp(model_size, "13B"))
        d = {5120, 13824, 40, 40, 40, 32000, 2048, group_size};
    else if (!strcmp(model_size, "70B"))
        d = {8192, 28672, 80, 64, 8, 32000, 2048, group_size};
    else
        return l2_fail(L2_ERR_ARG, "l2_preset: model size '%s' (7B, 13B or 70B)", model_size);
    L2_TRY(check_dims(&d));
    *out = d;
    return L2_OK;
}

extern "C" size_t l2_weights_bytes(const l2_dims *d) {
    if (!d || d->n_heads <= 0) return 0;
    const int hs = d->dim / d->n_heads;
    const int kv_dim = d->n_kv_heads * hs;
    const size_t L = (size_t)d->n_layers;
    const int G = d->group_size;
    size_t n = 4;
    n += (size_t)d->vocab_size * d->dim * 4;
    n += L * d->dim * 4;
    n += L * (2 * qlinear_bytes(d->dim, d->dim, G) + 2 * qlinear_bytes(d->dim, kv_dim, G));
    n += L * d->dim * 4;
    n += L * (2 * qlinear_bytes(d->dim, d->hidden_dim, G) + qlinear_bytes(d->hidden_dim, d->dim, G));
    n += (size_t)d->dim * 4;
    n += (size_t)d->seq_len * (hs / 2) * 4 * 2;
    n += (size_t)d->vocab_size * d->dim * 4;
    return n;
}

// ---------------------------------------------------------------------------
// synthetic image

namespace {

struct Rng { // splitmix64
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed) {}
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }
    float normal(float sigma) {
        double u1 = uniform(), u2 = uniform();
        if (u1 < 1e-300) u1 = 1e-300;
        return (float)(sigma * sqrt(-2.0 * log(u1)) * cos(6.283185307179586 * u2));
    }
};

// One tensor-sized job of the generator; jobs are independent so that threads
// can take them in any order and still produce the same bytes.
struct SynthJob {
    char *dst;
    size_t n; // elements
    int kind; // 0 random words, 1 scales, 2 normal(0.02), 3 g_index, 4 freq cos, 5 freq sin
    uint64_t seed;
    int a, b; // g_index: in, group_size; freq: seq_len, half
};

void run_job(const SynthJob &j) {
    Rng r(j.seed);
    switch (j.kind) {
        case 0: {
            uint32_t *p = (uint32_t *)j.dst;
            size_t i = 0;
            for (; i + 1 < j.n; i += 2) {
                const uint64_t v = r.next();
                p[i] = (uint32_t)v;
                p[i + 1] = (uint32_t)(v >> 32);
            }
            if (i < j.n) p[i] = (uint32_t)r.next();
            break;
        }
        case 1: {
            float *p = (float *)j.dst;
            for (size_t i = 0; i < j.n; i++) p[i] = (float)(0.002 + 0.018 * r.uniform());
            break;
        }
        case 2: {
            float *p = (float *)j.dst;
            for (size_t i = 0; i < j.n; i++) p[i] = r.normal(0.02f);
            break;
        }
        case 3: {
            // g_idx = shuffled i / group_size; g_index = stable argsort(g_idx)
            // (export.py:52,65)
            const int in = j.a, G = j.b;
            std::vector<int32_t> gidx(in);
            for (int i = 0; i < in; i++) gidx[i] = i / G;
            for (int i = in - 1; i > 0; i--) {
                const int k = (int)(r.next() % (uint64_t)(i + 1));
                std::swap(gidx[i], gidx[k]);
            }
            const int groups = (in + G - 1) / G;
            std::vector<int32_t> start(groups + 1, 0);
            for (int i = 0; i < in; i++) start[gidx[i] + 1]++;
            for (int g = 0; g < groups; g++) start[g + 1] += start[g];
            int32_t *p = (int32_t *)j.dst;
            for (int i = 0; i < in; i++) p[start[gidx[i]]++] = i;
            break;
        }
        case 4:
        case 5: {
            float *p = (float *)j.dst;
            const int half = j.b;
            for (int t = 0; t < j.a; t++)
                for (int i = 0; i < half; i++) {
                    const float f = 1.0f / powf(10000.0f, (float)(2 * i) / (float)(2 * half));
                    const float ang = (float)t * f;
                    p[(size_t)t * half + i] = j.kind == 4 ? cosf(ang) : sinf(ang);
                }
            break;
        }
    }
}

// Walk the image in struct order (src/gptq.rs:34-84), calling f(kind, ptr, elems, in, out).
struct Walker {
    const l2_dims &d;
    char *p;
    std::vector<SynthJob> jobs;
    uint64_t seed;
    uint64_t counter = 0;
    void add(int kind, size_t n, int a = 0, int b = 0) {
        // big tensors are cut into slices so that the threads stay balanced
        const size_t slice = (kind == 3 || kind == 4 || kind == 5) ? n : ((size_t)1 << 22);
        for (size_t off = 0; off < n; off += slice) {
            const size_t m = std::min(slice, n - off);
            jobs.push_back({p + off * 4, m, kind, seed * 0x100000001B3ull + (++counter) * 0x9E3779B97F4A7C15ull, a, b});
        }
        p += n * 4;
    }
    void qlinears(int in, int out) {
        const int G = d.group_size;
        if (G == 0) { // dense projections, N(0, 0.02) like the embedding
            for (int l = 0; l < d.n_layers; l++) add(2, (size_t)out * in);
            return;
        }
        const size_t groups = (size_t)div_up(in, G);
        for (int l = 0; l < d.n_layers; l++) {
            add(0, (size_t)out * (in / 8));
            add(0, (size_t)(out / 8) * groups);
            add(1, (size_t)out * groups);
            add(3, (size_t)in, in, G);
        }
    }
};

} // namespace

extern "C" int l2_synth_image(const l2_dims *d, uint64_t seed, void *buf, size_t nbytes) {
    L2_TRY(check_dims(d));
    if (!buf) return l2_fail(L2_ERR_ARG, "l2_synth_image: null buffer");
    if (nbytes != l2_weights_bytes(d))
        return l2_fail(L2_ERR_ARG, "l2_synth_image: buffer is %zu bytes, image is %zu", nbytes, l2_weights_bytes(d));
    const int hs = d->dim / d->n_heads, kv_dim = d->n_kv_heads * hs;
    Walker w{*d, (char *)buf, {}, seed};
    const float eps = 1e-5f;
    memcpy(w.p, &eps, 4);
    w.p += 4;
    w.add(2, (size_t)d->vocab_size * d->dim);
    w.add(2, (size_t)d->n_layers * d->dim);
    w.qlinears(d->dim, d->dim);
    w.qlinears(d->dim, kv_dim);
    w.qlinears(d->dim, kv_dim);
    w.qlinears(d->dim, d->dim);
    w.add(2, (size_t)d->n_layers * d->dim);
    w.qlinears(d->dim, d->hidden_dim);
    w.qlinears(d->hidden_dim, d->dim);
    w.qlinears(d->dim, d->hidden_dim);
    w.add(2, (size_t)d->dim);
    w.add(4, (size_t)d->seq_len * (hs / 2), d->seq_len, hs / 2);
    w.add(5, (size_t)d->seq_len * (hs / 2), d->seq_len, hs / 2);
    w.add(2, (size_t)d->vocab_size * d->dim);
    if ((size_t)(w.p - (char *)buf) != nbytes) return l2_fail(L2_ERR_ARG, "l2_synth_image: internal size mismatch");
    unsigned nt = std::thread::hardware_concurrency();
    if (nt == 0) nt = 1;
    if (nt > 16) nt = 16;
    std::vector<std::thread> th;
    for (unsigned t = 0; t < nt; t++)
        th.emplace_back([&, t]() {
            for (size_t i = t; i < w.jobs.size(); i += nt) run_job(w.jobs[i]);
        });
    for (auto &t : th) t.join();
    return L2_OK;
}

// ---------------------------------------------------------------------------
// model

struct l2_model {
    l2_dims d{};
    l2_config cfg{};
    int max_seq = 0;
    int head_size = 0, kv_dim = 0;
    float rms_eps = 0.f;
    int prefill_mode = L2_PREFILL_FP32;
    hipStream_t stream = nullptr;

    char *dimage = nullptr; // device copy of the weights image (shifted to 128-byte alignment)
    const float *tok_emb = nullptr, *rms_att = nullptr, *rms_ffn = nullptr, *rms_final = nullptr,
                *wcls = nullptr;
    std::vector<DevQLinear> q[7]; // indexed by L2_WQ..L2_W3, then layer
    int32_t *dinv = nullptr;      // all inverse permutations
    float *rope_cos = nullptr, *rope_sin = nullptr; // [max_seq][head_size/2]

    float *dwn = nullptr;         // norm weights in consumer order: [L][5][dim] (q, k, v, w1, w3)
    float *attn_part = nullptr;   // split-KV workspace [n_heads][kMaxSplits][130]

    // forward scratch, sized for cap_B batch columns.  xq/xk/xv and x1/x3 hold
    // the raw residual stream in the input order of the named projection.
    int cap_B = 0;
    float *x = nullptr, *xq = nullptr, *xk = nullptr, *xv = nullptr, *qv = nullptr, *kv = nullptr,
          *vv = nullptr, *attg = nullptr, *x1 = nullptr, *x3 = nullptr, *hg = nullptr, *hd = nullptr,
          *logits = nullptr;
    // extra scratch of the MFMA prefill path (cap_B_mfma columns): fp16 inputs, w1/w3 outputs, row scales
    int cap_B_mfma = 0;
    void *h16a = nullptr, *h16b = nullptr, *h16c = nullptr; // fp16 [B][max(dim, hidden)]
    float *hb = nullptr, *hb2 = nullptr, *ssb = nullptr, *gemm_ws = nullptr;
    size_t gemm_ws_floats = 0;
    int32_t *dtok = nullptr, *dpos = nullptr;
    unsigned long long *amax = nullptr;
    // l2_prefill_chunks: further streams, each with a set of chunk buffers of its own (consecutive chunks of a
    // prompt run side by side, one layer apart), the whole prompt's ids and positions, one event per layer and lane.
    // Lane 0 is the model's stream with its primary buffers; lanes 1.. use extra[lane - 1].
    static constexpr int kMaxLanes = 4; // the process has four hardware queues
    int n_lanes = 2;
    hipStream_t extra_stream[kMaxLanes - 1] = {nullptr, nullptr, nullptr};
    struct ChunkBufs {
        float *x = nullptr, *xq = nullptr, *xk = nullptr, *xv = nullptr, *qv = nullptr, *kv = nullptr, *vv = nullptr;
        void *h16a = nullptr, *h16b = nullptr, *h16c = nullptr;
        float *hb = nullptr, *hb2 = nullptr, *ssb = nullptr, *gemm_ws = nullptr;
        size_t gemm_ws_floats = 0;
        const int32_t *dtok = nullptr, *dpos = nullptr;
    };
    ChunkBufs extra[kMaxLanes - 1];
    int cap_B_extra[kMaxLanes - 1] = {0, 0, 0};
    int32_t *pf_tok = nullptr, *pf_pos = nullptr;
    int cap_pf = 0;
    std::vector<hipEvent_t> pf_ev[kMaxLanes];
    hipEvent_t pf_join = nullptr;
    int32_t *dprompt = nullptr, *dout_ids = nullptr;
    int cap_prompt = 0, cap_out = 0;
    // The decode step as a HIP graph (one per bucket of positions, kept in the state).  Off by default: a
    // replayed step takes the host out of the loop (one call per token instead of some 160), but the step is
    // bound by its kernels, not by their launches, and reading the position from device memory costs the
    // attention kernel a little (7B: 625 tok/s replayed, 629 launched).
    int32_t *dloop = nullptr;     // device {n_prompt, pos0} of the running loop, read by the captured next_token launch
    uint64_t buf_epoch = 1;       // bumped whenever a buffer a captured step points at is reallocated
    bool capturing = false;       // forward_enqueue: take the position from m->dpos, size attention for max_pos
    bool use_graph = false;
    // scratch for the operator-level entry points
    float *op_x = nullptr, *op_xg = nullptr, *op_y = nullptr;
    size_t op_cap = 0;
    // per-launch event timing, on only inside l2_decode_profile
    struct ProfRec { int cls; hipEvent_t e0, e1; };
    bool prof_on = false;
    std::vector<ProfRec> prof;
};


enum { K_EMBED = 0, K_Q4_QKV, K_ROPE_KV, K_ATTENTION, K_Q4_WO, K_Q4_W13, K_Q4_W2, K_CLASSIFIER, K_NEXT_TOKEN,
       K_NCLASS };
static const char *const kClassNames[K_NCLASS] = {"embed", "q4_qkv", "rope_kv", "attention", "q4_wo",
                                                  "q4_w13", "q4_w2", "classifier", "next_token"};
static constexpr int kMaxSplits = 64;

// Time one launch (profiling runs only).  The q4 launches of the streaming form hand their events to the
// dispatch itself; everything else is bracketed by event records on the stream.  Events of a launch that
// failed, or that nobody recorded, are destroyed here and leave no record.
template <class F>
static int timed_launch(l2_model *m, int cls, F &&launch) {
    l2_model::ProfRec r{cls, nullptr, nullptr};
    auto drop = [&]() {
        if (r.e0) (void)hipEventDestroy(r.e0);
        if (r.e1) (void)hipEventDestroy(r.e1);
    };
    hipError_t e = hipEventCreate(&r.e0);
    if (e == hipSuccess) e = hipEventCreate(&r.e1);
    if (e != hipSuccess) {
        drop();
        return l2_fail(L2_ERR_HIP, "hipEventCreate: %s", hipGetErrorString(e));
    }
    const bool q4 = m->d.group_size != 0 &&
                    (cls == K_Q4_QKV || cls == K_Q4_WO || cls == K_Q4_W13 || cls == K_Q4_W2);
    int rc = L2_OK;
    bool recorded = true;
    if (q4) {
        g_q4_prof.start = r.e0;
        g_q4_prof.stop = r.e1;
        g_q4_prof.armed = true;
        rc = launch();
        recorded = !g_q4_prof.armed; // a form of the kernel that does not take the events leaves them armed
        g_q4_prof.armed = false;
    } else {
        e = hipEventRecord(r.e0, m->stream);
        if (e == hipSuccess) rc = launch();
        if (e == hipSuccess && rc == L2_OK) e = hipEventRecord(r.e1, m->stream);
        if (e != hipSuccess && rc == L2_OK) rc = l2_fail(L2_ERR_HIP, "hipEventRecord: %s", hipGetErrorString(e));
    }
    if (rc != L2_OK || !recorded) {
        drop();
        return rc;
    }
    m->prof.push_back(r);
    return L2_OK;
}

#define LAUNCH(cls_, call)                                                   \
    do {                                                                     \
        if (m->prof_on)                                                      \
            L2_TRY(timed_launch(m, (cls_), [&]() -> int { return (call); })); \
        else                                                                 \
            L2_TRY(call);                                                    \
    } while (0)

struct StepGraph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    uint64_t epoch = 0;
};

struct l2_state {
    l2_model *m = nullptr;
    float *kcache = nullptr, *vcache = nullptr; // [L][max_seq][kv_dim]
    size_t elems = 0;
    std::map<int, StepGraph> steps; // captured decode step per upper bound of the position
};

static void step_graph_drop(StepGraph &g);

struct l2_qlinear {
    DevQLinear q;
    void *bufs[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    hipStream_t stream = nullptr;
    float *x = nullptr, *xg = nullptr, *y = nullptr;
    int cap_B = 0;
};

extern "C" int l2_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    return n;
}

static int require_device() {
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if (e != hipSuccess || n < 1) {
        (void)hipGetLastError();
        return l2_fail(L2_ERR_HIP, "no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    }
    return L2_OK;
}

template <typename T>
static int dalloc(T **p, size_t n) {
    void *v = nullptr;
    hipError_t e = hipMalloc(&v, n * sizeof(T) ? n * sizeof(T) : 16);
    if (e != hipSuccess) return l2_fail(L2_ERR_HIP, "hipMalloc(%zu bytes): %s", n * sizeof(T), hipGetErrorString(e));
    *p = (T *)v;
    return L2_OK;
}

static void dfree(void *p) {
    if (p) (void)hipFree(p);
}

static void invert_perm(const int32_t *g, int n, int32_t *inv, bool *ok) {
    std::fill(inv, inv + n, -1);
    for (int j = 0; j < n; j++) {
        const int32_t v = g[j];
        if (v < 0 || v >= n || inv[v] != -1) {
            *ok = false;
            return;
        }
        inv[v] = j;
    }
}

static constexpr size_t kImageShift = 124; // image offset 4 (first tensor) lands on a 128-byte boundary

static int model_build(const char *weights, size_t nbytes, const l2_dims *dims, int max_seq, l2_model **out) {
    L2_TRY(check_dims(dims));
    if (!weights || !out) return l2_fail(L2_ERR_ARG, "null argument");
    if (nbytes != l2_weights_bytes(dims)) // src/lib.rs:97
        return l2_fail(L2_ERR_FORMAT, "weights are %zu bytes, the struct for these dims is %zu", nbytes,
                       l2_weights_bytes(dims));
    if (max_seq <= 0) max_seq = dims->seq_len;
    {   // the attention kernels address one layer's cache with 32-bit byte offsets
        const size_t layer_bytes = (size_t)max_seq * dims->n_kv_heads * (dims->dim / dims->n_heads) * 4;
        if (layer_bytes >= ((size_t)1 << 32))
            return l2_fail(L2_ERR_RANGE, "max_seq %d: one layer of the cache would be %zu bytes (below 4 GiB)", max_seq,
                           layer_bytes);
    }
    L2_TRY(require_device());

    l2_model *m = new l2_model();
    m->use_graph = getenv("L2_STEP_GRAPH") != nullptr; // also l2_model_set_step_graph
    if (const char *v = getenv("L2_PREFILL_LANES")) { // chunks of a prompt in flight at once (l2_prefill_chunks)
        const int n = atoi(v);
        if (n >= 1 && n <= l2_model::kMaxLanes) m->n_lanes = n;
    }
    m->d = *dims;
    m->max_seq = max_seq;
    m->head_size = dims->dim / dims->n_heads;
    m->kv_dim = dims->n_kv_heads * m->head_size;
    m->cfg = {dims->dim, dims->hidden_dim, dims->n_layers, dims->n_heads, dims->n_kv_heads,
              dims->vocab_size, dims->seq_len, 0};
    auto bail = [&](int rc) {
        l2_model_close(m);
        return rc;
    };
#define M_HIP(call)                                                                              \
    do {                                                                                         \
        hipError_t e_ = (call);                                                                  \
        if (e_ != hipSuccess)                                                                    \
            return bail(l2_fail(L2_ERR_HIP, "%s: %s", #call, hipGetErrorString(e_)));            \
    } while (0)
#define M_TRY(call)                    \
    do {                               \
        int rc_ = (call);              \
        if (rc_ != L2_OK) return bail(rc_); \
    } while (0)

    M_HIP(hipStreamCreate(&m->stream));
    M_TRY(dalloc(&m->dimage, nbytes + 256));
    char *dbase = m->dimage + kImageShift;
    // one pass over the host image, in 64 MiB pieces so that a mapped file is paged in as it goes
    for (size_t off = 0; off < nbytes; off += (size_t)64 << 20) {
        const size_t n = std::min((size_t)64 << 20, nbytes - off);
        M_HIP(hipMemcpy(dbase + off, weights + off, n, hipMemcpyHostToDevice));
    }

    // views, in struct order (src/gptq.rs:34-66)
    const int L = dims->n_layers, G = dims->group_size, dim = dims->dim, hid = dims->hidden_dim;
    size_t off = 0;
    memcpy(&m->rms_eps, weights, 4);
    off += 4;
    auto f32 = [&](size_t n) {
        const float *p = (const float *)(dbase + off);
        off += n * 4;
        return p;
    };
    size_t inv_total = 0;
    struct Pending { int proj, layer; size_t host_off; int in; size_t inv_off; };
    std::vector<Pending> pend;
    auto qblock = [&](int proj, int in, int outn) {
        m->q[proj].resize(L);
        if (G == 0) { // src/model.rs:36-67: the same field order, every projection a dense matrix
            for (int l = 0; l < L; l++) {
                DevQLinear &q = m->q[proj][l];
                q.in = in;
                q.out = outn;
                q.dense = (const float *)(dbase + off);
                off += (size_t)outn * in * 4;
            }
            return;
        }
        const int groups = (int)div_up(in, G);
        for (int l = 0; l < L; l++) {
            DevQLinear &q = m->q[proj][l];
            q.in = in;
            q.out = outn;
            q.groups = groups;
            q.group_size = G;
            q.qweight = (const uint4 *)(dbase + off);
            off += (size_t)outn * (in / 8) * 4;
            q.qzeros = (const int32_t *)(dbase + off);
            off += (size_t)(outn / 8) * groups * 4;
            q.scales = (const float *)(dbase + off);
            off += (size_t)outn * groups * 4;
            q.g_index = (const int32_t *)(dbase + off);
            pend.push_back({proj, l, off, in, inv_total});
            inv_total += (size_t)in;
            off += (size_t)in * 4;
        }
    };
    m->tok_emb = f32((size_t)dims->vocab_size * dim);
    m->rms_att = f32((size_t)L * dim);
    qblock(L2_WQ, dim, dim);
    qblock(L2_WK, dim, m->kv_dim);
    qblock(L2_WV, dim, m->kv_dim);
    qblock(L2_WO, dim, dim);
    m->rms_ffn = f32((size_t)L * dim);
    qblock(L2_W1, dim, hid);
    qblock(L2_W2, hid, dim);
    qblock(L2_W3, dim, hid);
    m->rms_final = f32((size_t)dim);
    off += (size_t)dims->seq_len * (m->head_size / 2) * 4 * 2; // deprecated tables, never read (src/models.rs:193-197)
    m->wcls = f32((size_t)dims->vocab_size * dim);
    if (off != nbytes) return bail(l2_fail(L2_ERR_FORMAT, "internal: walked %zu of %zu bytes", off, nbytes));

    // inverse act-order permutations (also validates every g_index)
    if (G != 0) {
        std::vector<int32_t> inv(inv_total);
        bool ok = true;
        for (const Pending &p : pend) {
            invert_perm((const int32_t *)(weights + p.host_off), p.in, inv.data() + p.inv_off, &ok);
            if (!ok)
                return bail(l2_fail(L2_ERR_FORMAT, "g_index of projection %d, layer %d is not a permutation of 0..%d",
                                    p.proj, p.layer, p.in - 1));
        }
        M_TRY(dalloc(&m->dinv, inv_total));
        M_HIP(hipMemcpy(m->dinv, inv.data(), inv_total * 4, hipMemcpyHostToDevice));
        for (const Pending &p : pend) m->q[p.proj][p.layer].inv_index = m->dinv + p.inv_off;
    }

    M_TRY(dalloc(&m->attn_part, (size_t)dims->n_heads * kMaxSplits * 130));
    // Norm weights re-ordered for each consumer of a normalised vector, so that the
    // matvec prologue reads them linearly: wn_c[j] = w[g_index_c[j]].
    if (G != 0) {
        const size_t per_layer = (size_t)5 * dim;
        std::vector<float> wn((size_t)L * per_layer);
        const float *att_h = (const float *)(weights + ((const char *)m->rms_att - dbase));
        const float *ffn_h = (const float *)(weights + ((const char *)m->rms_ffn - dbase));
        const int projs[5] = {L2_WQ, L2_WK, L2_WV, L2_W1, L2_W3};
        for (int l = 0; l < L; l++)
            for (int c = 0; c < 5; c++) {
                const float *src = (c < 3 ? att_h : ffn_h) + (size_t)l * dim;
                const int32_t *g = (const int32_t *)(weights + ((const char *)m->q[projs[c]][l].g_index - dbase));
                float *dst = wn.data() + l * per_layer + (size_t)c * dim;
                for (int j = 0; j < dim; j++) dst[j] = src[g[j]];
            }
        M_TRY(dalloc(&m->dwn, wn.size()));
        M_HIP(hipMemcpy(m->dwn, wn.data(), wn.size() * 4, hipMemcpyHostToDevice));
    }

    // RoPE angles exactly as the reference evaluates them per element
    // (src/models.rs:107-110), computed once with the host's libm.
    {
        const int half = m->head_size / 2;
        std::vector<float> c((size_t)max_seq * half), s((size_t)max_seq * half);
        for (int i = 0; i < half; i++) {
            const float freq = 1.0f / powf(10000.0f, ((float)((2 * i) % m->head_size)) / (float)m->head_size);
            for (int p = 0; p < max_seq; p++) {
                const float val = (float)p * freq;
                c[(size_t)p * half + i] = cosf(val);
                s[(size_t)p * half + i] = sinf(val);
            }
        }
        M_TRY(dalloc(&m->rope_cos, c.size()));
        M_TRY(dalloc(&m->rope_sin, s.size()));
        M_HIP(hipMemcpy(m->rope_cos, c.data(), c.size() * 4, hipMemcpyHostToDevice));
        M_HIP(hipMemcpy(m->rope_sin, s.data(), s.size() * 4, hipMemcpyHostToDevice));
    }
    M_TRY(dalloc(&m->amax, 1));
    M_HIP(hipDeviceSynchronize());
#undef M_HIP
#undef M_TRY
    *out = m;
    return L2_OK;
}

extern "C" int l2_model_from_image(const void *weights, size_t nbytes, const l2_dims *dims, int max_seq,
                                   l2_model **out) {
    return model_build((const char *)weights, nbytes, dims, max_seq, out);
}

extern "C" int l2_model_open(const char *path, const l2_dims *expect, int max_seq, l2_model **out) {
    if (!path || !expect || !out) return l2_fail(L2_ERR_ARG, "l2_model_open: null argument");
    L2_TRY(check_dims(expect));
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return l2_fail(L2_ERR_IO, "open %s: %s", path, strerror(errno));
    struct stat st;
    if (fstat(fd, &st) != 0) {
        close(fd);
        return l2_fail(L2_ERR_IO, "stat %s: %s", path, strerror(errno));
    }
    int32_t h[7];
    if (st.st_size < 28 || pread(fd, h, 28, 0) != 28) {
        close(fd);
        return l2_fail(L2_ERR_FORMAT, "%s: shorter than the 28-byte header", path);
    }
    // Config::load + check_static (src/constants.rs:94-119)
    l2_config cfg = {h[0], h[1], h[2], h[3], h[4], h[5] < 0 ? -h[5] : h[5], h[6], h[5] > 0};
    if (cfg.dim != expect->dim || cfg.hidden_dim != expect->hidden_dim || cfg.n_layers != expect->n_layers ||
        cfg.n_heads != expect->n_heads || cfg.vocab_size != expect->vocab_size) {
        close(fd);
        return l2_fail(L2_ERR_FORMAT,
                       "%s: header (dim %d, hidden %d, layers %d, heads %d, vocab %d) does not match the "
                       "expected (%d, %d, %d, %d, %d)",
                       path, cfg.dim, cfg.hidden_dim, cfg.n_layers, cfg.n_heads, cfg.vocab_size, expect->dim,
                       expect->hidden_dim, expect->n_layers, expect->n_heads, expect->vocab_size);
    }
    const size_t want = l2_weights_bytes(expect);
    if ((size_t)st.st_size - 28 != want) { // src/lib.rs:97
        close(fd);
        return l2_fail(L2_ERR_FORMAT, "%s: %zu bytes after the header, the struct for these dims is %zu", path,
                       (size_t)st.st_size - 28, want);
    }
    // The reference maps from byte 28 (src/lib.rs:95-96); mmap offsets must be
    // page aligned, so map from 0 and step over the header.
    void *map = mmap(nullptr, (size_t)st.st_size, PROT_READ, MAP_PRIVATE, fd, 0);
    close(fd);
    if (map == MAP_FAILED) return l2_fail(L2_ERR_IO, "mmap %s: %s", path, strerror(errno));
    (void)madvise(map, (size_t)st.st_size, MADV_SEQUENTIAL);
    const int rc = model_build((const char *)map + 28, want, expect, max_seq, out);
    munmap(map, (size_t)st.st_size);
    if (rc == L2_OK) (*out)->cfg = cfg;
    return rc;
}

extern "C" void l2_model_close(l2_model *m) {
    if (!m) return;
    if (m->stream) (void)hipStreamSynchronize(m->stream);
    for (hipStream_t es : m->extra_stream)
        if (es) (void)hipStreamSynchronize(es);
    void *ptrs[] = {m->dimage, m->dinv, m->rope_cos, m->rope_sin, m->dwn, m->attn_part, m->x, m->xq, m->xk,
                    m->xv, m->qv, m->kv, m->vv, m->attg, m->x1, m->x3, m->hg, m->hd, m->logits, m->dtok, m->dpos, m->dloop,
                    m->amax, m->dprompt, m->dout_ids, m->op_x, m->op_xg, m->op_y, m->h16a, m->h16b, m->h16c,
                    m->hb, m->hb2, m->ssb, m->gemm_ws};
    for (void *p : ptrs) dfree(p);
    for (auto &a : m->extra) {
        void *bufs[] = {a.x, a.xq, a.xk, a.xv, a.qv, a.kv, a.vv, a.h16a, a.h16b, a.h16c, a.hb, a.hb2, a.ssb, a.gemm_ws};
        for (void *p : bufs) dfree(p);
    }
    dfree(m->pf_tok);
    dfree(m->pf_pos);
    for (auto &v : m->pf_ev)
        for (hipEvent_t e : v) (void)hipEventDestroy(e);
    if (m->pf_join) (void)hipEventDestroy(m->pf_join);
    for (hipStream_t es : m->extra_stream)
        if (es) (void)hipStreamDestroy(es);
    if (m->stream) (void)hipStreamDestroy(m->stream);
    delete m;
}

extern "C" int l2_model_config(const l2_model *m, l2_config *out) {
    if (!m || !out) return l2_fail(L2_ERR_ARG, "null argument");
    *out = m->cfg;
    return L2_OK;
}

extern "C" int l2_model_dims(const l2_model *m, l2_dims *out) {
    if (!m || !out) return l2_fail(L2_ERR_ARG, "null argument");
    *out = m->d;
    return L2_OK;
}

extern "C" int l2_model_max_seq(const l2_model *m) { return m ? m->max_seq : 0; }

extern "C" int l2_prefill_supported(const l2_model *m) { return m ? 1 : 0; }

extern "C" int l2_model_set_step_graph(l2_model *m, int on) {
    if (!m) return l2_fail(L2_ERR_ARG, "null model");
    m->use_graph = on != 0;
    return L2_OK;
}

extern "C" int l2_model_set_prefill_mode(l2_model *m, int mode) {
    if (!m) return l2_fail(L2_ERR_ARG, "null model");
    if (mode != L2_PREFILL_FP32 && mode != L2_PREFILL_MFMA) return l2_fail(L2_ERR_ARG, "prefill mode %d", mode);
    if (mode == L2_PREFILL_MFMA && m->d.group_size == 0)
        return l2_fail(L2_ERR_ARG, "the MFMA prefill path is the quantised model's");
    const int G = m->d.group_size;
    if (mode == L2_PREFILL_MFMA && m->head_size != 128)
        return l2_fail(L2_ERR_ARG, "the MFMA prefill path is built for heads of 128 (this model: %d)", m->head_size);
    if (mode == L2_PREFILL_MFMA && !(q4_gemm_supports(m->d.dim, m->d.dim, G) && q4_gemm_supports(m->d.hidden_dim, m->kv_dim, G) &&
                                     q4_gemm_supports(m->d.dim, m->d.hidden_dim, G)))
        return l2_fail(L2_ERR_ARG, "the MFMA prefill path needs dim and hidden_dim to be multiples of 128 (of 2 groups for "
                                   "group sizes 64 and 128) and output sizes to be multiples of 32");
    m->prefill_mode = mode;
    return L2_OK;
}

static int ensure_batch_mfma(l2_model *m, int B);

// Nothing may be running on either of the model's streams when a buffer they use is freed.
static int drain_streams(l2_model *m) {
    L2_HIP(hipStreamSynchronize(m->stream));
    for (hipStream_t es : m->extra_stream)
        if (es) L2_HIP(hipStreamSynchronize(es));
    return L2_OK;
}

static int ensure_batch(l2_model *m, int B) {
    if (B <= m->cap_B) return L2_OK;
    L2_TRY(drain_streams(m));
    m->buf_epoch++;
    float **bufs[] = {&m->x, &m->xq, &m->xk, &m->xv, &m->qv, &m->kv, &m->vv, &m->attg, &m->x1, &m->x3, &m->hg};
    for (float **b : bufs) {
        dfree(*b);
        *b = nullptr;
    }
    dfree(m->dtok);
    dfree(m->dpos);
    m->dtok = m->dpos = nullptr;
    m->cap_B = 0;
    const size_t dim = m->d.dim, hid = m->d.hidden_dim, kvd = m->kv_dim;
    L2_TRY(dalloc(&m->x, B * dim));
    L2_TRY(dalloc(&m->xq, B * dim));
    L2_TRY(dalloc(&m->xk, B * dim));
    L2_TRY(dalloc(&m->xv, B * dim));
    L2_TRY(dalloc(&m->qv, B * dim));
    L2_TRY(dalloc(&m->kv, B * kvd));
    L2_TRY(dalloc(&m->vv, B * kvd));
    L2_TRY(dalloc(&m->attg, B * dim));
    L2_TRY(dalloc(&m->x1, B * dim));
    L2_TRY(dalloc(&m->x3, B * dim));
    L2_TRY(dalloc(&m->hg, B * hid));
    if (m->d.group_size == 0) { // the dense model keeps w1's output beside the gated product
        dfree(m->hd);
        m->hd = nullptr;
        L2_TRY(dalloc(&m->hd, B * hid));
    }
    L2_TRY(dalloc(&m->dtok, (size_t)B));
    L2_TRY(dalloc(&m->dpos, (size_t)B));
    if (!m->logits) L2_TRY(dalloc(&m->logits, (size_t)m->d.vocab_size));
    if (!m->dloop) L2_TRY(dalloc(&m->dloop, (size_t)2));
    m->cap_B = B;
    return L2_OK;
}

// ---------------------------------------------------------------------------
// state

extern "C" int l2_state_new(l2_model *m, l2_state **out) {
    if (!m || !out) return l2_fail(L2_ERR_ARG, "null argument");
    l2_state *s = new l2_state();
    s->m = m;
    s->elems = (size_t)m->d.n_layers * m->max_seq * m->kv_dim;
    int rc = dalloc(&s->kcache, s->elems);
    if (rc == L2_OK) rc = dalloc(&s->vcache, s->elems);
    if (rc != L2_OK) {
        l2_state_free(s);
        return rc;
    }
    rc = l2_state_reset(s);
    if (rc != L2_OK) {
        l2_state_free(s);
        return rc;
    }
    *out = s;
    return L2_OK;
}

extern "C" void l2_state_free(l2_state *s) {
    if (!s) return;
    if (s->m && s->m->stream) (void)hipStreamSynchronize(s->m->stream);
    for (auto &kv : s->steps) step_graph_drop(kv.second);
    dfree(s->kcache);
    dfree(s->vcache);
    delete s;
}

extern "C" int l2_state_reset(l2_state *s) {
    if (!s) return l2_fail(L2_ERR_ARG, "null state");
    L2_HIP(hipMemsetAsync(s->kcache, 0, s->elems * 4, s->m->stream));
    L2_HIP(hipMemsetAsync(s->vcache, 0, s->elems * 4, s->m->stream));
    L2_HIP(hipStreamSynchronize(s->m->stream));
    return L2_OK;
}

extern "C" int l2_state_read_kv(l2_state *s, int layer, int pos0, int npos, float *k_host, float *v_host) {
    if (!s || !k_host || !v_host) return l2_fail(L2_ERR_ARG, "null argument");
    const l2_model *m = s->m;
    if (layer < 0 || layer >= m->d.n_layers || pos0 < 0 || npos < 0 || pos0 + npos > m->max_seq)
        return l2_fail(L2_ERR_RANGE, "read_kv: layer %d, positions [%d,%d)", layer, pos0, pos0 + npos);
    const size_t off = ((size_t)layer * m->max_seq + pos0) * m->kv_dim;
    L2_HIP(hipStreamSynchronize(m->stream));
    L2_HIP(hipMemcpy(k_host, s->kcache + off, (size_t)npos * m->kv_dim * 4, hipMemcpyDeviceToHost));
    L2_HIP(hipMemcpy(v_host, s->vcache + off, (size_t)npos * m->kv_dim * 4, hipMemcpyDeviceToHost));
    return L2_OK;
}

extern "C" int l2_state_write_kv(l2_state *s, int layer, int pos0, int npos, const float *k_host,
                                 const float *v_host) {
    if (!s || !k_host || !v_host) return l2_fail(L2_ERR_ARG, "null argument");
    const l2_model *m = s->m;
    if (layer < 0 || layer >= m->d.n_layers || pos0 < 0 || npos < 0 || pos0 + npos > m->max_seq)
        return l2_fail(L2_ERR_RANGE, "write_kv: layer %d, positions [%d,%d)", layer, pos0, pos0 + npos);
    const size_t off = ((size_t)layer * m->max_seq + pos0) * m->kv_dim;
    L2_HIP(hipStreamSynchronize(m->stream));
    L2_HIP(hipMemcpy(s->kcache + off, k_host, (size_t)npos * m->kv_dim * 4, hipMemcpyHostToDevice));
    L2_HIP(hipMemcpy(s->vcache + off, v_host, (size_t)npos * m->kv_dim * 4, hipMemcpyHostToDevice));
    return L2_OK;
}

extern "C" int l2_state_fill_synthetic(l2_state *s, int pos0, int npos, uint64_t seed) {
    if (!s) return l2_fail(L2_ERR_ARG, "null state");
    const l2_model *m = s->m;
    if (pos0 < 0 || npos < 0 || pos0 + npos > m->max_seq)
        return l2_fail(L2_ERR_RANGE, "fill: positions [%d,%d)", pos0, pos0 + npos);
    for (int l = 0; l < m->d.n_layers; l++) {
        const size_t off = ((size_t)l * m->max_seq + pos0) * m->kv_dim;
        const size_t n = (size_t)npos * m->kv_dim;
        L2_TRY(fill_pattern_launch(s->kcache + off, n, seed * 2654435761ull + 2 * l, m->stream));
        L2_TRY(fill_pattern_launch(s->vcache + off, n, seed * 2654435761ull + 2 * l + 1, m->stream));
    }
    L2_HIP(hipStreamSynchronize(m->stream));
    return L2_OK;
}

// ---------------------------------------------------------------------------
// operators

static Q4Mat mat_of(const DevQLinear &q, const float *x, const float *wn, float *y) {
    Q4Mat M{};
    M.qweight = q.qweight;
    M.qzeros = q.qzeros;
    M.scales = q.scales;
    M.x = x;
    M.wn = wn;
    M.y = y;
    M.out = q.out;
    return M;
}

static Q4Launch launch_of(const DevQLinear &q, int B, float eps) {
    Q4Launch L{};
    L.n_mats = 1;
    L.in = q.in;
    L.groups = q.groups;
    L.group_size = q.group_size;
    L.batch = B;
    L.eps = eps;
    L.e.kind = Q4_EPI_STORE;
    return L;
}

// y = W xg for one matrix, plain store.
static int q4_one(const DevQLinear &q, const float *xg, float *y, int B, hipStream_t st) {
    Q4Launch L = launch_of(q, B, 0.f);
    L.m[0] = mat_of(q, xg, nullptr, y);
    return q4_matvec_launch(L, st);
}

// QLinear::matvec<B> on x in its natural order (src/gptq.rs:94-176, the act-order gather of :99-122 included):
// one launch where the kernel can apply g_index itself, else a gather into xg_scratch and the matvec.
static int q4_one_natural(const DevQLinear &q, const float *x, float *xg_scratch, float *y, int B, hipStream_t st) {
    Q4Launch L = launch_of(q, B, 0.f);
    L.m[0] = mat_of(q, x, nullptr, y);
    if (q4_gathers_in_kernel(L)) {
        L.m[0].gidx = q.inv_index;
        return q4_matvec_launch(L, st);
    }
    L2_TRY(gather_launch(xg_scratch, x, q.g_index, q.in, B, st));
    return q4_one(q, xg_scratch, y, B, st);
}

static int check_qlinear_shape(int in, int out, int g) {
    if (g != 32 && g != 64 && g != 128) return l2_fail(L2_ERR_ARG, "group size %d (32, 64 or 128)", g);
    if (in <= 0 || out <= 0 || in % 32 || in % g || out % 8)
        return l2_fail(L2_ERR_ARG, "QLinear %dx%d: in must be a multiple of 32 and of the group size, out of 8", in, out);
    return L2_OK;
}

static int qlinear_scratch(l2_qlinear *q, int B);
static int scratch_ptr(float **out);

// Everything a later launch of this layer's operator would otherwise do on first use, done once here and waited
// for: the code object is loaded on this device, the kernel's dynamic-LDS limit is raised, the fixed scratch
// array's address is resolved.  A call made under stream capture afterwards only enqueues kernels.
static int qlinear_warm_up(l2_qlinear *q) {
    L2_TRY(qlinear_scratch(q, 1));
    float *fixed = nullptr;
    L2_TRY(scratch_ptr(&fixed));
    L2_HIP(hipMemsetAsync(q->x, 0, (size_t)q->q.in * 4, q->stream));
    L2_TRY(q4_one_natural(q->q, q->x, q->xg, q->y, 1, q->stream));   // the form l2_qlinear_matvec runs
    L2_TRY(gather_launch(q->xg, q->x, q->q.g_index, q->q.in, 1, q->stream));
    L2_TRY(q4_one(q->q, q->xg, q->y, 1, q->stream));                 // the form l2_qlinear_matvec_device runs
    L2_HIP(hipStreamSynchronize(q->stream));
    return L2_OK;
}

extern "C" int l2_qlinear_create(const int32_t *qweight, const int32_t *qzeros, const float *scales,
                                 const int32_t *g_index, int in, int out, int group_size, l2_qlinear **ql) {
    if (!qweight || !qzeros || !scales || !g_index || !ql) return l2_fail(L2_ERR_ARG, "null argument");
    L2_TRY(check_qlinear_shape(in, out, group_size));
    L2_TRY(require_device());
    const int groups = (int)div_up(in, group_size);
    std::vector<int32_t> inv(in);
    bool ok = true;
    invert_perm(g_index, in, inv.data(), &ok);
    if (!ok) return l2_fail(L2_ERR_FORMAT, "g_index is not a permutation of 0..%d", in - 1);
    l2_qlinear *q = new l2_qlinear();
    const size_t sizes[5] = {(size_t)out * (in / 8) * 4, (size_t)(out / 8) * groups * 4, (size_t)out * groups * 4,
                             (size_t)in * 4, (size_t)in * 4};
    const void *src[5] = {qweight, qzeros, scales, g_index, inv.data()};
    for (int i = 0; i < 5; i++) {
        hipError_t e = hipMalloc(&q->bufs[i], sizes[i]);
        if (e == hipSuccess) e = hipMemcpy(q->bufs[i], src[i], sizes[i], hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            l2_qlinear_free(q);
            return l2_fail(L2_ERR_HIP, "upload of QLinear array %d: %s", i, hipGetErrorString(e));
        }
    }
    if (hipStreamCreate(&q->stream) != hipSuccess) {
        l2_qlinear_free(q);
        return l2_fail(L2_ERR_HIP, "hipStreamCreate failed");
    }
    q->q.qweight = (const uint4 *)q->bufs[0];
    q->q.qzeros = (const int32_t *)q->bufs[1];
    q->q.scales = (const float *)q->bufs[2];
    q->q.g_index = (const int32_t *)q->bufs[3];
    q->q.inv_index = (const int32_t *)q->bufs[4];
    q->q.in = in;
    q->q.out = out;
    q->q.groups = groups;
    q->q.group_size = group_size;
    const int rc = qlinear_warm_up(q);
    if (rc != L2_OK) {
        l2_qlinear_free(q);
        return rc;
    }
    *ql = q;
    return L2_OK;
}

extern "C" void l2_qlinear_free(l2_qlinear *q) {
    if (!q) return;
    if (q->stream) (void)hipStreamSynchronize(q->stream);
    for (void *p : q->bufs) dfree(p);
    dfree(q->x);
    dfree(q->xg);
    dfree(q->y);
    if (q->stream) (void)hipStreamDestroy(q->stream);
    delete q;
}

static int qlinear_scratch(l2_qlinear *q, int B) {
    if (B <= q->cap_B) return L2_OK;
    dfree(q->x);
    dfree(q->xg);
    dfree(q->y);
    q->x = q->xg = q->y = nullptr;
    q->cap_B = 0;
    L2_TRY(dalloc(&q->x, (size_t)B * q->q.in));
    L2_TRY(dalloc(&q->xg, (size_t)B * q->q.in));
    L2_TRY(dalloc(&q->y, (size_t)B * q->q.out));
    q->cap_B = B;
    return L2_OK;
}

// x (host, natural order) -> gather through g_index -> matvec -> y (host)
static int matvec_host(const DevQLinear &q, float *dx, float *dxg, float *dy, const float *x_host, int B,
                       float *y_host, hipStream_t st) {
    L2_HIP(hipMemcpyAsync(dx, x_host, (size_t)B * q.in * 4, hipMemcpyHostToDevice, st));
    L2_TRY(q4_one_natural(q, dx, dxg, dy, B, st));
    L2_HIP(hipMemcpyAsync(y_host, dy, (size_t)B * q.out * 4, hipMemcpyDeviceToHost, st));
    L2_HIP(hipStreamSynchronize(st));
    return L2_OK;
}

extern "C" int l2_qlinear_matvec(l2_qlinear *q, const float *x_host, int B, float *y_host) {
    if (!q || !x_host || !y_host) return l2_fail(L2_ERR_ARG, "null argument");
    if (B < 1 || B > 4096) return l2_fail(L2_ERR_RANGE, "batch %d (1..4096)", B);
    L2_TRY(qlinear_scratch(q, B));
    return matvec_host(q->q, q->x, q->xg, q->y, x_host, B, y_host, q->stream);
}

// ---- the same operator for callers that cannot allocate ---------------------------------------------
// (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  The one buffer
// l2_qlinear_matvec needs beyond its input and output -- x gathered into the layer's act-order -- lives in a
// fixed device array instead of a hipMalloc'ed one.  Every GPU the library runs on holds its own copy of
// the array, at its own address, until the process ends.
static constexpr size_t kScratchFloats = L2_MATVEC_DEVICE_MAX_ELEMS; // 4 MiB
static __device__ __align__(256) float scratch[kScratchFloats];

// The array's address on the current device.  `scratch` by name is a host-side stand-in, not a device
// address; the address is asked for once per device, with that device current, and kept.
static int scratch_ptr(float **out) {
    static constexpr int kMaxDevices = 64;
    static float *ptrs[kMaxDevices] = {};
    static std::mutex mu;
    int dev = 0;
    L2_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return l2_fail(L2_ERR_HIP, "device %d: more devices than the scratch table holds", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void *p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return l2_fail(L2_ERR_HIP, "hipGetSymbolAddress(scratch) on device %d: %s", dev, hipGetErrorString(e));
        ptrs[dev] = (float *)p;
    }
    *out = ptrs[dev];
    return L2_OK;
}

extern "C" int l2_qlinear_matvec_device(l2_qlinear *q, const float *x_dev, int B, float *y_dev, void *hip_stream) {
    if (!q || !x_dev || !y_dev) return l2_fail(L2_ERR_ARG, "null argument");
    if (B < 1 || B > 4096) return l2_fail(L2_ERR_RANGE, "batch %d (1..4096)", B);
    if ((size_t)B * (size_t)q->q.in > kScratchFloats)
        return l2_fail(L2_ERR_RANGE, "B * in = %zu floats exceed the fixed scratch of %zu (no allocation is made here: "
                                     "use a smaller batch, or l2_qlinear_matvec)",
                       (size_t)B * (size_t)q->q.in, kScratchFloats);
    float *xg = nullptr;
    L2_TRY(scratch_ptr(&xg));
    hipStream_t st = (hipStream_t)hip_stream;
    // Every element of xg[0 .. B * in) is written by the gather before the matvec reads it: nothing of the
    // previous call's contents is read, so nothing needs clearing.
    L2_TRY(gather_launch(xg, x_dev, q->q.g_index, q->q.in, B, st));
    L2_TRY(q4_one(q->q, xg, y_dev, B, st));
    return L2_OK;
}

static int op_scratch(l2_model *m, size_t elems) {
    if (elems <= m->op_cap) return L2_OK;
    L2_HIP(hipStreamSynchronize(m->stream));
    dfree(m->op_x);
    dfree(m->op_xg);
    dfree(m->op_y);
    m->op_x = m->op_xg = m->op_y = nullptr;
    m->op_cap = 0;
    L2_TRY(dalloc(&m->op_x, elems));
    L2_TRY(dalloc(&m->op_xg, elems));
    L2_TRY(dalloc(&m->op_y, elems));
    m->op_cap = elems;
    return L2_OK;
}

extern "C" int l2_model_qmatvec(l2_model *m, int layer, int proj, const float *x_host, int B, float *y_host) {
    if (!m || !x_host || !y_host) return l2_fail(L2_ERR_ARG, "null argument");
    if (proj < 0 || proj > 6 || layer < 0 || layer >= m->d.n_layers)
        return l2_fail(L2_ERR_RANGE, "projection %d, layer %d", proj, layer);
    if (B < 1 || B > 4096) return l2_fail(L2_ERR_RANGE, "batch %d (1..4096)", B);
    const DevQLinear &q = m->q[proj][layer];
    L2_TRY(op_scratch(m, (size_t)B * std::max(std::max(q.in, q.out), m->d.vocab_size)));
    if (q.dense) { // Linear::matvec<B> (src/model.rs:22-31)
        hipStream_t st = m->stream;
        L2_HIP(hipMemcpyAsync(m->op_x, x_host, (size_t)B * q.in * 4, hipMemcpyHostToDevice, st));
        DenseArgs a{};
        a.y = m->op_y, a.w = q.dense, a.x = m->op_x, a.in = q.in, a.out = q.out, a.batch = B;
        L2_TRY(dense_launch(a, st));
        L2_HIP(hipMemcpyAsync(y_host, m->op_y, (size_t)B * q.out * 4, hipMemcpyDeviceToHost, st));
        L2_HIP(hipStreamSynchronize(st));
        return L2_OK;
    }
    if (B > 1 && m->prefill_mode == L2_PREFILL_MFMA && q4_gemm_supports(q.in, q.out, q.group_size)) {
        // the prefill form of the same operator: gather, round to fp16, dequant -> MFMA
        hipStream_t st = m->stream;
        L2_TRY(ensure_batch_mfma(m, B));
        L2_HIP(hipMemcpyAsync(m->op_x, x_host, (size_t)B * q.in * 4, hipMemcpyHostToDevice, st));
        L2_TRY(gather_launch(m->op_xg, m->op_x, q.g_index, q.in, B, st));
        L2_TRY(prep_f16_launch(m->h16a, m->op_xg, nullptr, q.in, B, st));
        Q4Launch Q = launch_of(q, B, 0.f);
        Q.m[0] = mat_of(q, nullptr, nullptr, m->op_y);
        XhList X{{m->h16a, nullptr, nullptr}};
        L2_TRY(q4_gemm_launch(Q, X, nullptr, m->gemm_ws, m->gemm_ws_floats, st));
        L2_HIP(hipMemcpyAsync(y_host, m->op_y, (size_t)B * q.out * 4, hipMemcpyDeviceToHost, st));
        L2_HIP(hipStreamSynchronize(st));
        return L2_OK;
    }
    return matvec_host(q, m->op_x, m->op_xg, m->op_y, x_host, B, y_host, m->stream);
}

extern "C" int l2_model_classifier(l2_model *m, const float *x_host, float *y_host) {
    if (!m || !x_host || !y_host) return l2_fail(L2_ERR_ARG, "null argument");
    L2_TRY(op_scratch(m, (size_t)std::max(m->d.dim, m->d.vocab_size)));
    L2_HIP(hipMemcpyAsync(m->op_x, x_host, (size_t)m->d.dim * 4, hipMemcpyHostToDevice, m->stream));
    L2_TRY(dense_matvec_launch(m->op_y, m->wcls, m->op_x, nullptr, 0.f, m->d.dim, m->d.vocab_size, nullptr, m->stream));
    L2_HIP(hipMemcpyAsync(y_host, m->op_y, (size_t)m->d.vocab_size * 4, hipMemcpyDeviceToHost, m->stream));
    L2_HIP(hipStreamSynchronize(m->stream));
    return L2_OK;
}

// ---------------------------------------------------------------------------
// transformer<B>

// How the timesteps of a decode step are cut across blocks: one block per kv head up to 256 timesteps,
// beyond that one block per CU where the context allows it, at least 64 timesteps each.  (Two per CU, the
// earlier rule, left some CUs with two blocks and the launch as long as those: 70B behind 4096 positions
// 18.6 -> 16.5 us per layer, 13B behind 1000 positions 16.7 -> 15.3, 7B unchanged; half a block per CU is
// slower everywhere.)
static void attn_split_policy(int n_t, int n_kv_heads, int *ts_out, int *n_splits_out) {
    if (n_t <= 256) {
        *ts_out = 256;
        *n_splits_out = 1;
        return;
    }
    int want = (cu_count() + n_kv_heads - 1) / n_kv_heads;
    if (want > kMaxSplits) want = kMaxSplits;
    int ts = ((n_t + want - 1) / want + 63) / 64 * 64;
    if (ts < 64) ts = 64;
    *ts_out = ts;
    *n_splits_out = (n_t + ts - 1) / ts;
}

// Enqueue one forward pass for the B tokens / positions already in m->dtok /
// m->dpos.  max_pos is the largest position among them (sizes the attention
// scratch).  With want_logits the classifier and the running argmax follow.
//
// Five launches per layer when B == 1: q|k|v with the attention rmsnorm in
// front; attention with RoPE and the cache write folded in; wo with the
// residual add behind; w1|w3 with the ffn rmsnorm in front and the SiLU gate
// behind; w2 with the residual add behind.  Every producer writes its result
// in the input order (g_index) of whoever reads it next.
static int forward_enqueue_dense(l2_model *m, l2_state *s, int B, int max_pos, bool want_logits);

static int check_position(const l2_model *m, int max_pos) {
    // No kernel clamps a position: the RoPE table and the cache end at max_seq (the reference panics on its
    // fixed [SEQ_LEN] arrays, src/models.rs:29-33).
    if (max_pos < 0 || max_pos >= m->max_seq)
        return l2_fail(L2_ERR_RANGE, "position %d outside 0..%d", max_pos, m->max_seq - 1);
    return L2_OK;
}

static int forward_enqueue(l2_model *m, l2_state *s, int B, int max_pos, bool want_logits) {
    L2_TRY(check_position(m, max_pos));
    if (m->d.group_size == 0) return forward_enqueue_dense(m, s, B, max_pos, want_logits);
    const l2_dims &d = m->d;
    const int dim = d.dim, hid = d.hidden_dim, kvd = m->kv_dim, L = d.n_layers;
    hipStream_t st = m->stream;
    {   // :189-191
        ScatterTargets t{};
        t.n = 3;
        t.inv[0] = m->q[L2_WQ][0].inv_index, t.inv[1] = m->q[L2_WK][0].inv_index, t.inv[2] = m->q[L2_WV][0].inv_index;
        t.out[0] = m->xq, t.out[1] = m->xk, t.out[2] = m->xv;
        LAUNCH(K_EMBED, embed_launch(m->x, m->tok_emb, m->dtok, dim, B, t, m->amax, st));
    }
    for (int l = 0; l < L; l++) {
        const DevQLinear &wq = m->q[L2_WQ][l], &wk = m->q[L2_WK][l], &wv = m->q[L2_WV][l],
                         &wo = m->q[L2_WO][l], &w1 = m->q[L2_W1][l], &w2 = m->q[L2_W2][l],
                         &w3 = m->q[L2_W3][l];
        const float *wn = m->dwn + (size_t)l * 5 * dim;
        {   // attention rmsnorm (:217-219) + q, k, v (:224-226)
            Q4Launch Q = launch_of(wq, B, m->rms_eps);
            Q.m[0] = mat_of(wq, m->xq, wn + 0 * (size_t)dim, m->qv);
            Q.m[1] = mat_of(wk, m->xk, wn + 1 * (size_t)dim, m->kv);
            Q.m[2] = mat_of(wv, m->xv, wn + 2 * (size_t)dim, m->vv);
            Q.n_mats = 3;
            LAUNCH(K_Q4_QKV, q4_matvec_launch(Q, st));
        }
        float *kc = s->kcache + (size_t)l * m->max_seq * kvd;
        float *vc = s->vcache + (size_t)l * m->max_seq * kvd;
        if (B == 1) { // rope (:228-230), cache write (:236-249), attention (:250-256)
            AttnDecode a{};
            a.q = m->qv, a.k_new = m->kv, a.v_new = m->vv;
            a.kcache = kc, a.vcache = vc;
            a.cos_t = m->rope_cos, a.sin_t = m->rope_sin;
            a.pos = max_pos;
            a.dpos = m->capturing ? m->dpos : nullptr; // a captured step serves every position up to max_pos
            a.out = m->attg, a.scatter = wo.inv_index;
            a.part = m->attn_part;
            a.n_heads = d.n_heads, a.n_kv_heads = d.n_kv_heads;
            a.max_splits = kMaxSplits;
            attn_split_policy(max_pos + 1, d.n_kv_heads, &a.ts, &a.n_splits);
            if (a.n_splits > kMaxSplits)
                return l2_fail(L2_ERR_RANGE, "attention: position %d needs %d splits", max_pos, a.n_splits);
            LAUNCH(K_ATTENTION, attention_decode_launch(a, st));
        } else {
            LAUNCH(K_ROPE_KV, rope_kv_launch(m->qv, m->kv, m->vv, m->dpos, m->rope_cos, m->rope_sin, kc, vc, d.n_heads,
                                             d.n_kv_heads, m->head_size, B, st));
            LAUNCH(K_ATTENTION, attention_launch(m->attg, nullptr, m->qv, kc, vc, m->dpos, wo.inv_index, d.n_heads,
                                                 d.n_kv_heads, m->head_size, max_pos, B, st));
        }
        {   // wo (:260) + residual (:263-264); the new x also goes out in w1's and w3's order
            Q4Launch Q = launch_of(wo, B, 0.f);
            Q.m[0] = mat_of(wo, m->attg, nullptr, m->x);
            Q.e.kind = Q4_EPI_RESIDUAL;
            Q.e.res = m->x;
            Q.e.n_scatter = 2;
            Q.e.sc_idx[0] = w1.inv_index, Q.e.sc_out[0] = m->x1;
            Q.e.sc_idx[1] = w3.inv_index, Q.e.sc_out[1] = m->x3;
            LAUNCH(K_Q4_WO, q4_matvec_launch(Q, st));
        }
        {   // ffn rmsnorm (:266) + w1 | w3 (:271-272) + silu gate (:274-276), in w2's order
            Q4Launch Q = launch_of(w1, B, m->rms_eps);
            Q.m[0] = mat_of(w1, m->x1, wn + 3 * (size_t)dim, nullptr);
            Q.m[1] = mat_of(w3, m->x3, wn + 4 * (size_t)dim, nullptr);
            Q.n_mats = 2;
            Q.pair = 1;
            Q.e.kind = Q4_EPI_SCATTER_ONLY;
            Q.e.n_scatter = 1;
            Q.e.sc_idx[0] = w2.inv_index, Q.e.sc_out[0] = m->hg;
            LAUNCH(K_Q4_W13, q4_matvec_launch(Q, st));
        }
        {   // w2 (:279) + residual (:283-285); the new x goes out in the next layer's q, k, v order
            Q4Launch Q = launch_of(w2, B, 0.f);
            Q.m[0] = mat_of(w2, m->hg, nullptr, m->x);
            Q.e.kind = Q4_EPI_RESIDUAL;
            Q.e.res = m->x;
            if (l + 1 < L) {
                Q.e.n_scatter = 3;
                Q.e.sc_idx[0] = m->q[L2_WQ][l + 1].inv_index, Q.e.sc_out[0] = m->xq;
                Q.e.sc_idx[1] = m->q[L2_WK][l + 1].inv_index, Q.e.sc_out[1] = m->xk;
                Q.e.sc_idx[2] = m->q[L2_WV][l + 1].inv_index, Q.e.sc_out[2] = m->xv;
            }
            LAUNCH(K_Q4_W2, q4_matvec_launch(Q, st));
        }
        (void)hid;
    }
    if (want_logits) // final rmsnorm + classifier (:288-297, B == 1 only) + running argmax
        LAUNCH(K_CLASSIFIER, dense_matvec_launch(m->logits, m->wcls, m->x, m->rms_final, m->rms_eps, dim,
                                                 d.vocab_size, m->amax, st));
    return L2_OK;
}

// The same schedule for the model without quantisation (TransformerWeights, src/model.rs:36-67):
// every projection is a dense matvec with its rmsnorm in front (q, k, v, w1, w3), the SiLU gate behind
// (w3) or the residual add behind (wo, w2).  No act-order, so nothing is scattered.
static int forward_enqueue_dense(l2_model *m, l2_state *s, int B, int max_pos, bool want_logits) {
    const l2_dims &d = m->d;
    const int dim = d.dim, hid = d.hidden_dim, kvd = m->kv_dim, L = d.n_layers;
    hipStream_t st = m->stream;
    {
        ScatterTargets t{};
        LAUNCH(K_EMBED, embed_launch(m->x, m->tok_emb, m->dtok, dim, B, t, m->amax, st));
    }
    auto dense = [&](const DevQLinear &w, const float *x, const float *wn, float *y, const float *res,
                     const float *gate) {
        DenseArgs a{};
        a.y = y, a.w = w.dense, a.x = x, a.wn = wn, a.eps = m->rms_eps, a.in = w.in, a.out = w.out, a.batch = B;
        a.res = res, a.gate = gate;
        return dense_launch(a, st);
    };
    for (int l = 0; l < L; l++) {
        const float *att_n = m->rms_att + (size_t)l * dim, *ffn_n = m->rms_ffn + (size_t)l * dim;
        LAUNCH(K_Q4_QKV, dense(m->q[L2_WQ][l], m->x, att_n, m->qv, nullptr, nullptr)); // :217-226
        L2_TRY(dense(m->q[L2_WK][l], m->x, att_n, m->kv, nullptr, nullptr));
        L2_TRY(dense(m->q[L2_WV][l], m->x, att_n, m->vv, nullptr, nullptr));
        float *kc = s->kcache + (size_t)l * m->max_seq * kvd;
        float *vc = s->vcache + (size_t)l * m->max_seq * kvd;
        if (B == 1) {
            AttnDecode a{};
            a.q = m->qv, a.k_new = m->kv, a.v_new = m->vv;
            a.kcache = kc, a.vcache = vc;
            a.cos_t = m->rope_cos, a.sin_t = m->rope_sin;
            a.pos = max_pos;
            a.dpos = m->capturing ? m->dpos : nullptr; // a captured step serves every position up to max_pos
            a.out = m->attg, a.scatter = nullptr;
            a.part = m->attn_part;
            a.n_heads = d.n_heads, a.n_kv_heads = d.n_kv_heads;
            a.max_splits = kMaxSplits;
            attn_split_policy(max_pos + 1, d.n_kv_heads, &a.ts, &a.n_splits);
            if (a.n_splits > kMaxSplits)
                return l2_fail(L2_ERR_RANGE, "attention: position %d needs %d splits", max_pos, a.n_splits);
            LAUNCH(K_ATTENTION, attention_decode_launch(a, st));
        } else {
            LAUNCH(K_ROPE_KV, rope_kv_launch(m->qv, m->kv, m->vv, m->dpos, m->rope_cos, m->rope_sin, kc, vc, d.n_heads,
                                             d.n_kv_heads, m->head_size, B, st));
            LAUNCH(K_ATTENTION, attention_launch(m->attg, nullptr, m->qv, kc, vc, m->dpos, nullptr, d.n_heads,
                                                 d.n_kv_heads, m->head_size, max_pos, B, st));
        }
        LAUNCH(K_Q4_WO, dense(m->q[L2_WO][l], m->attg, nullptr, m->x, m->x, nullptr));       // :260-264
        LAUNCH(K_Q4_W13, dense(m->q[L2_W1][l], m->x, ffn_n, m->hd, nullptr, nullptr));        // :266-271
        L2_TRY(dense(m->q[L2_W3][l], m->x, ffn_n, m->hg, nullptr, m->hd));                    // :272-276
        LAUNCH(K_Q4_W2, dense(m->q[L2_W2][l], m->hg, nullptr, m->x, m->x, nullptr));          // :279-285
        (void)hid;
    }
    if (want_logits)
        LAUNCH(K_CLASSIFIER, dense_matvec_launch(m->logits, m->wcls, m->x, m->rms_final, m->rms_eps, dim,
                                                 d.vocab_size, m->amax, st));
    return L2_OK;
}

static int ensure_batch_mfma(l2_model *m, int B) {
    if (B <= m->cap_B_mfma) return L2_OK;
    L2_TRY(drain_streams(m));
    void **bufs[] = {&m->h16a, &m->h16b, &m->h16c, (void **)&m->hb, (void **)&m->hb2, (void **)&m->ssb,
                     (void **)&m->gemm_ws};
    m->gemm_ws_floats = 0;
    for (void **b : bufs) {
        dfree(*b);
        *b = nullptr;
    }
    m->cap_B_mfma = 0;
    const size_t wide = (size_t)std::max(m->d.dim, m->d.hidden_dim);
    uint16_t *p = nullptr;
    L2_TRY(dalloc(&p, B * wide));
    m->h16a = p;
    L2_TRY(dalloc(&p, B * wide));
    m->h16b = p;
    L2_TRY(dalloc(&p, B * wide));
    m->h16c = p;
    L2_TRY(dalloc(&m->hb, B * (size_t)m->d.hidden_dim));
    L2_TRY(dalloc(&m->hb2, B * (size_t)m->d.hidden_dim));
    L2_TRY(dalloc(&m->ssb, (size_t)B));
    // split-K partial tiles: up to 8 slices of the widest launch (w1|w3 or q|k|v)
    m->gemm_ws_floats = (size_t)8 * B * std::max((size_t)2 * m->d.hidden_dim, (size_t)m->d.dim + 2 * m->kv_dim) / 2;
    L2_TRY(dalloc(&m->gemm_ws, m->gemm_ws_floats));
    m->cap_B_mfma = B;
    return L2_OK;
}

// A prefill chunk through the matrix cores: the same schedule as forward_enqueue,
// with every QLinear as a dequant -> fp16 -> MFMA GEMM over the B tokens and the
// element-wise steps as kernels of their own.  Logits are never produced here
// (src/models.rs:288).
static l2_model::ChunkBufs primary_bufs(const l2_model *m) {
    l2_model::ChunkBufs b;
    b.x = m->x, b.xq = m->xq, b.xk = m->xk, b.xv = m->xv, b.qv = m->qv, b.kv = m->kv, b.vv = m->vv;
    b.h16a = m->h16a, b.h16b = m->h16b, b.h16c = m->h16c;
    b.hb = m->hb, b.hb2 = m->hb2, b.ssb = m->ssb, b.gemm_ws = m->gemm_ws, b.gemm_ws_floats = m->gemm_ws_floats;
    b.dtok = m->dtok, b.dpos = m->dpos;
    return b;
}

// The chunk's buffers and stream are arguments: l2_prefill_chunks runs consecutive chunks on two streams.  What a
// chunk needs from the ones before it is their cache rows of the same layer, so `before_attn[l]` (the event of the
// chunk before) is waited for in front of the attention of layer l, behind the kernel that writes this chunk's own
// rows of layer l, and `after_kv[l]` is recorded right there (either may be null).
static int forward_enqueue_mfma(l2_model *m, l2_state *s, int B, int max_pos, const l2_model::ChunkBufs &b,
                                hipStream_t st, const hipEvent_t *after_kv, const hipEvent_t *before_attn) {
    L2_TRY(check_position(m, max_pos));
    const l2_dims &d = m->d;
    const int dim = d.dim, hid = d.hidden_dim, kvd = m->kv_dim, L = d.n_layers;
    {
        ScatterTargets t{};
        t.n = 3;
        t.inv[0] = m->q[L2_WQ][0].inv_index, t.inv[1] = m->q[L2_WK][0].inv_index, t.inv[2] = m->q[L2_WV][0].inv_index;
        t.out[0] = b.xq, t.out[1] = b.xk, t.out[2] = b.xv;
        L2_TRY(embed_launch(b.x, m->tok_emb, b.dtok, dim, B, t, nullptr, st));
        // the first layer's inputs; every later layer gets them from the kernel that ends the layer before
        L2_TRY(rms_scale_launch(b.ssb, b.x, m->rms_eps, dim, B, st));
        PrepList P{};
        P.n_mats = 3;
        P.out[0] = b.h16a, P.x[0] = b.xq, P.wn[0] = m->dwn + 0 * (size_t)dim;
        P.out[1] = b.h16b, P.x[1] = b.xk, P.wn[1] = m->dwn + 1 * (size_t)dim;
        P.out[2] = b.h16c, P.x[2] = b.xv, P.wn[2] = m->dwn + 2 * (size_t)dim;
        L2_TRY(prep_f16_multi_launch(P, dim, B, st));
    }
    for (int l = 0; l < L; l++) {
        const DevQLinear &wq = m->q[L2_WQ][l], &wk = m->q[L2_WK][l], &wv = m->q[L2_WV][l],
                         &wo = m->q[L2_WO][l], &w1 = m->q[L2_W1][l], &w2 = m->q[L2_W2][l],
                         &w3 = m->q[L2_W3][l];
        RopeKvArgs R{};
        {
            Q4Launch Q = launch_of(wq, B, m->rms_eps);
            Q.m[0] = mat_of(wq, nullptr, nullptr, b.qv);
            Q.m[1] = mat_of(wk, nullptr, nullptr, b.kv);
            Q.m[2] = mat_of(wv, nullptr, nullptr, b.vv);
            Q.n_mats = 3;
            XhList X{{b.h16a, b.h16b, b.h16c}};
            // partial tiles; the kernel that adds them also applies the rms scale, RoPE and the cache write
            L2_TRY(q4_gemm_launch(Q, X, b.ssb, b.gemm_ws, b.gemm_ws_floats, st, &R.KS));
        }
        float *kc = s->kcache + (size_t)l * m->max_seq * kvd;
        float *vc = s->vcache + (size_t)l * m->max_seq * kvd;
        R.ws = b.gemm_ws, R.B = B, R.ss = b.ssb, R.pos = b.dpos, R.cos_t = m->rope_cos, R.sin_t = m->rope_sin;
        R.q = b.qv, R.kcache = kc, R.vcache = vc, R.n_heads = d.n_heads, R.n_kv_heads = d.n_kv_heads;
        L2_TRY(gemm_rope_kv_launch(R, st));
        // Wait first, record second: the event of this chunk then stands for its own rows of layer l AND, through
        // the event it waited for, for those of every chunk before it, so that a chunk two or more lanes behind
        // needs to wait for its direct predecessor only.
        if (before_attn) L2_HIP(hipStreamWaitEvent(st, before_attn[l], 0));
        if (after_kv) L2_HIP(hipEventRecord(after_kv[l], st));
        L2_TRY(attention_launch(nullptr, b.h16a, b.qv, kc, vc, b.dpos, wo.inv_index, d.n_heads, d.n_kv_heads,
                                m->head_size, max_pos, B, st));
        {   // wo: partial tiles, then residual + rms scale + the fp16 inputs of w1 and w3 in one kernel
            Q4Launch Q = launch_of(wo, B, 0.f);
            Q.m[0] = mat_of(wo, nullptr, nullptr, b.x);
            XhList X{{b.h16a, nullptr, nullptr}};
            ResNormPrep R{};
            L2_TRY(q4_gemm_launch(Q, X, nullptr, b.gemm_ws, b.gemm_ws_floats, st, &R.KS));
            R.ws = b.gemm_ws, R.B = B, R.out = dim, R.res = b.x, R.x = b.x, R.ss = b.ssb, R.eps = m->rms_eps;
            R.n = 2, R.wn = m->rms_ffn + (size_t)l * dim;
            R.inv[0] = w1.inv_index, R.out_h[0] = b.h16a;
            R.inv[1] = w3.inv_index, R.out_h[1] = b.h16b;
            L2_TRY(gemm_residual_norm_prep_launch(R, st));
        }
        {
            Q4Launch Q = launch_of(w1, B, m->rms_eps);
            Q.m[0] = mat_of(w1, nullptr, nullptr, b.hb);
            Q.m[1] = mat_of(w3, nullptr, nullptr, b.hb2);
            Q.n_mats = 2;
            XhList X{{b.h16a, b.h16b, nullptr}};
            L2_TRY(q4_gemm_launch(Q, X, b.ssb, b.gemm_ws, b.gemm_ws_floats, st));
        }
        L2_TRY(silu_scatter_launch(nullptr, b.h16a, b.hb, b.hb2, w2.inv_index, hid, B, st));
        {
            Q4Launch Q = launch_of(w2, B, 0.f);
            Q.m[0] = mat_of(w2, nullptr, nullptr, b.x);
            XhList X{{b.h16a, nullptr, nullptr}};
            if (l + 1 < L) { // the same kernel hands the next layer its q, k and v inputs
                ResNormPrep R{};
                L2_TRY(q4_gemm_launch(Q, X, nullptr, b.gemm_ws, b.gemm_ws_floats, st, &R.KS));
                R.ws = b.gemm_ws, R.B = B, R.out = dim, R.res = b.x, R.x = b.x, R.ss = b.ssb, R.eps = m->rms_eps;
                R.n = 3, R.wn = m->rms_att + (size_t)(l + 1) * dim;
                R.inv[0] = m->q[L2_WQ][l + 1].inv_index, R.out_h[0] = b.h16a;
                R.inv[1] = m->q[L2_WK][l + 1].inv_index, R.out_h[1] = b.h16b;
                R.inv[2] = m->q[L2_WV][l + 1].inv_index, R.out_h[2] = b.h16c;
                L2_TRY(gemm_residual_norm_prep_launch(R, st));
            } else {
                Q.e.kind = Q4_EPI_RESIDUAL;
                Q.e.res = b.x;
                L2_TRY(q4_gemm_launch(Q, X, nullptr, b.gemm_ws, b.gemm_ws_floats, st));
            }
        }
    }
    return L2_OK;
}

static int forward_enqueue_mfma(l2_model *m, l2_state *s, int B, int max_pos) {
    L2_TRY(ensure_batch_mfma(m, B));
    return forward_enqueue_mfma(m, s, B, max_pos, primary_bufs(m), m->stream, nullptr, nullptr);
}

static int check_tokens(const l2_model *m, const int32_t *tokens, const int32_t *pos, int B, int *max_pos) {
    int mp = 0;
    for (int b = 0; b < B; b++) {
        if (tokens[b] < 0 || tokens[b] >= m->d.vocab_size)
            return l2_fail(L2_ERR_RANGE, "token id %d outside 0..%d", tokens[b], m->d.vocab_size - 1);
        if (pos[b] < 0 || pos[b] >= m->max_seq)
            return l2_fail(L2_ERR_RANGE, "position %d outside 0..%d", pos[b], m->max_seq - 1);
        mp = std::max(mp, pos[b]);
    }
    *max_pos = mp;
    return L2_OK;
}

extern "C" int l2_forward(l2_model *m, l2_state *s, const int32_t *tokens, const int32_t *pos, int B,
                          float *logits_host) {
    if (!m || !s || !tokens || !pos) return l2_fail(L2_ERR_ARG, "null argument");
    if (s->m != m) return l2_fail(L2_ERR_ARG, "state belongs to another model");
    if (B < 1 || B > 4096) return l2_fail(L2_ERR_RANGE, "batch %d (1..4096)", B);
    int max_pos = 0;
    L2_TRY(check_tokens(m, tokens, pos, B, &max_pos));
    L2_TRY(ensure_batch(m, B));
    L2_HIP(hipMemcpyAsync(m->dtok, tokens, (size_t)B * 4, hipMemcpyHostToDevice, m->stream));
    L2_HIP(hipMemcpyAsync(m->dpos, pos, (size_t)B * 4, hipMemcpyHostToDevice, m->stream));
    if (B > 1 && m->prefill_mode == L2_PREFILL_MFMA)
        L2_TRY(forward_enqueue_mfma(m, s, B, max_pos));
    else
        L2_TRY(forward_enqueue(m, s, B, max_pos, B == 1));
    if (B == 1 && logits_host)
        L2_HIP(hipMemcpyAsync(logits_host, m->logits, (size_t)m->d.vocab_size * 4, hipMemcpyDeviceToHost, m->stream));
    L2_HIP(hipStreamSynchronize(m->stream));
    return L2_OK;
}

// The second set of chunk buffers, the second stream and the per-layer events of l2_prefill_chunks.
static int ensure_prefill_pipeline(l2_model *m, int B, int n) {
    const int lanes = B > 0 ? m->n_lanes : 1;
    for (int i = 0; i + 1 < lanes; i++)
        if (!m->extra_stream[i]) L2_HIP(hipStreamCreate(&m->extra_stream[i])); // default priority, as the model's own
    if (!m->pf_join) L2_HIP(hipEventCreateWithFlags(&m->pf_join, hipEventDisableTiming));
    for (int i = 0; i < lanes; i++)
        while ((int)m->pf_ev[i].size() < m->d.n_layers) {
            hipEvent_t e = nullptr;
            L2_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            m->pf_ev[i].push_back(e);
        }
    if (n > m->cap_pf) {
        L2_TRY(drain_streams(m));
        dfree(m->pf_tok), dfree(m->pf_pos);
        m->pf_tok = m->pf_pos = nullptr, m->cap_pf = 0;
        L2_TRY(dalloc(&m->pf_tok, (size_t)n));
        L2_TRY(dalloc(&m->pf_pos, (size_t)n));
        m->cap_pf = n;
    }
    for (int i = 0; i + 1 < lanes; i++) {
        if (B <= m->cap_B_extra[i]) continue;
        L2_TRY(drain_streams(m));
        l2_model::ChunkBufs &a = m->extra[i];
        void **bufs[] = {(void **)&a.x, (void **)&a.xq, (void **)&a.xk, (void **)&a.xv, (void **)&a.qv, (void **)&a.kv,
                         (void **)&a.vv, &a.h16a, &a.h16b, &a.h16c, (void **)&a.hb, (void **)&a.hb2, (void **)&a.ssb,
                         (void **)&a.gemm_ws};
        for (void **b : bufs) {
            dfree(*b);
            *b = nullptr;
        }
        m->cap_B_extra[i] = 0;
        const size_t dim = m->d.dim, hid = m->d.hidden_dim, kvd = m->kv_dim, wide = std::max(dim, hid);
        L2_TRY(dalloc(&a.x, B * dim));
        L2_TRY(dalloc(&a.xq, B * dim));
        L2_TRY(dalloc(&a.xk, B * dim));
        L2_TRY(dalloc(&a.xv, B * dim));
        L2_TRY(dalloc(&a.qv, B * dim));
        L2_TRY(dalloc(&a.kv, B * kvd));
        L2_TRY(dalloc(&a.vv, B * kvd));
        uint16_t *h = nullptr;
        L2_TRY(dalloc(&h, B * wide));
        a.h16a = h;
        L2_TRY(dalloc(&h, B * wide));
        a.h16b = h;
        L2_TRY(dalloc(&h, B * wide));
        a.h16c = h;
        L2_TRY(dalloc(&a.hb, B * hid));
        L2_TRY(dalloc(&a.hb2, B * hid));
        L2_TRY(dalloc(&a.ssb, (size_t)B));
        a.gemm_ws_floats = (size_t)8 * B * std::max((size_t)2 * hid, dim + 2 * kvd) / 2;
        L2_TRY(dalloc(&a.gemm_ws, a.gemm_ws_floats));
        m->cap_B_extra[i] = B;
    }
    return L2_OK;
}

// prefill<A> (src/inference.rs:16-40) for a whole prompt: tokens[i] at position pos0 + i, in chunks of `chunk`,
// no logits.  With the matrix-core mode consecutive chunks run on n_lanes streams, each with buffers of its own:
// a chunk needs from its predecessor only that chunk's cache rows of the same layer (an event per layer), so
// every chunk follows one layer behind the one before it and its kernels fill the compute units that the
// others' short launches leave idle.  The arithmetic of a chunk is that of l2_forward on the same chunk.
extern "C" int l2_prefill_chunks(l2_model *m, l2_state *s, const int32_t *tokens, int n, int pos0, int chunk) {
    if (!m || !s || !tokens) return l2_fail(L2_ERR_ARG, "null argument");
    if (s->m != m) return l2_fail(L2_ERR_ARG, "state belongs to another model");
    if (n < 1 || chunk < 1 || chunk > 4096) return l2_fail(L2_ERR_RANGE, "%d tokens in chunks of %d (1..4096)", n, chunk);
    if (pos0 < 0 || (long)pos0 + n > m->max_seq)
        return l2_fail(L2_ERR_RANGE, "positions %d..%ld outside 0..%d", pos0, (long)pos0 + n - 1, m->max_seq - 1);
    for (int i = 0; i < n; i++)
        if (tokens[i] < 0 || tokens[i] >= m->d.vocab_size)
            return l2_fail(L2_ERR_RANGE, "token id %d outside 0..%d", tokens[i], m->d.vocab_size - 1);
    const int Bmax = std::min(chunk, n);
    L2_TRY(ensure_batch(m, Bmax));
    const bool mfma = m->prefill_mode == L2_PREFILL_MFMA;
    if (mfma) L2_TRY(ensure_batch_mfma(m, Bmax));
    L2_TRY(ensure_prefill_pipeline(m, mfma ? Bmax : 0, n));
    std::vector<int32_t> pos((size_t)n);
    for (int i = 0; i < n; i++) pos[(size_t)i] = pos0 + i;
    // synchronous copies: the host arrays are the caller's and this function's own
    L2_HIP(hipStreamSynchronize(m->stream));
    L2_HIP(hipMemcpy(m->pf_tok, tokens, (size_t)n * 4, hipMemcpyHostToDevice));
    L2_HIP(hipMemcpy(m->pf_pos, pos.data(), (size_t)n * 4, hipMemcpyHostToDevice));
    // Everything that is enqueued on the two streams; a failure half-way returns through the caller below, which
    // first waits for what earlier chunks already have in flight on either stream.
    const int lanes = mfma ? m->n_lanes : 1;
    // the model's stream waits for everything the other lanes have been given so far
    auto join_lanes = [&]() -> int {
        for (int i = 0; i + 1 < lanes; i++) {
            L2_HIP(hipEventRecord(m->pf_join, m->extra_stream[i]));
            L2_HIP(hipStreamWaitEvent(m->stream, m->pf_join, 0));
        }
        return L2_OK;
    };
    auto enqueue_all = [&]() -> int {
        int c = 0;
        for (int c0 = 0; c0 < n; c0 += chunk, c++) {
            const int B = std::min(chunk, n - c0);
            const int max_pos = pos0 + c0 + B - 1;
            if (mfma && B > 1) {
                const int lane = c % lanes, before = (c + lanes - 1) % lanes;
                l2_model::ChunkBufs b = lane ? m->extra[lane - 1] : primary_bufs(m);
                b.dtok = m->pf_tok + c0, b.dpos = m->pf_pos + c0;
                hipStream_t st = lane ? m->extra_stream[lane - 1] : m->stream;
                L2_TRY(forward_enqueue_mfma(m, s, B, max_pos, b, st, m->pf_ev[lane].data(),
                                            c > 0 ? m->pf_ev[before].data() : nullptr));
            } else {
                // one token left over, or the fp32 mode: the fp32 kernels on the model's stream, behind everything
                if (c > 0 && mfma) L2_TRY(join_lanes());
                L2_HIP(hipMemcpyAsync(m->dtok, m->pf_tok + c0, (size_t)B * 4, hipMemcpyDeviceToDevice, m->stream));
                L2_HIP(hipMemcpyAsync(m->dpos, m->pf_pos + c0, (size_t)B * 4, hipMemcpyDeviceToDevice, m->stream));
                L2_TRY(forward_enqueue(m, s, B, max_pos, false));
            }
        }
        if (mfma) L2_TRY(join_lanes());
        return L2_OK;
    };
    const int rc = enqueue_all();
    if (rc != L2_OK) {
        // kernels of earlier chunks may still be writing cache rows and chunk buffers on both streams: nothing
        // returns to the caller (who may reset the state or free the model next) before they are done.  The
        // error text of the failure that brought us here is kept.
        char keep[sizeof g_err];
        memcpy(keep, g_err, sizeof keep);
        (void)hipStreamSynchronize(m->stream);
        for (hipStream_t es : m->extra_stream)
            if (es) (void)hipStreamSynchronize(es);
        memcpy(g_err, keep, sizeof keep);
        return rc;
    }
    L2_HIP(hipStreamSynchronize(m->stream));
    return L2_OK;
}

static int ensure_loop_buffers(l2_model *m, int n_prompt, int n_out);
static int loop_begin(l2_model *m, int n_prompt, int pos0);
static int loop_step(l2_model *m, l2_state *s, int pos, int n_prompt, int pos0);

extern "C" int l2_decode_greedy(l2_model *m, l2_state *s, int32_t token, int32_t pos, int32_t *next) {
    if (!m || !s || !next) return l2_fail(L2_ERR_ARG, "null argument");
    if (s->m != m) return l2_fail(L2_ERR_ARG, "state belongs to another model");
    int max_pos = 0;
    L2_TRY(check_tokens(m, &token, &pos, 1, &max_pos));
    L2_TRY(ensure_batch(m, 1));
    L2_TRY(ensure_loop_buffers(m, 1, 1));
    L2_TRY(set_i32_launch(m->dtok, token, m->dpos, pos, m->stream));
    L2_TRY(loop_begin(m, 0, pos));
    L2_TRY(loop_step(m, s, pos, 0, pos)); // the argmax stays in m->amax; the hand-over it also does is harmless
    unsigned long long key = 0;
    L2_HIP(hipMemcpyAsync(&key, m->amax, 8, hipMemcpyDeviceToHost, m->stream));
    L2_HIP(hipStreamSynchronize(m->stream));
    *next = (int32_t)(key & 0xFFFFFFFFull);
    return L2_OK;
}

static int ensure_loop_buffers(l2_model *m, int n_prompt, int n_out) {
    if (n_prompt > m->cap_prompt) {
        L2_HIP(hipStreamSynchronize(m->stream));
        m->buf_epoch++;
        dfree(m->dprompt);
        m->dprompt = nullptr;
        m->cap_prompt = 0;
        L2_TRY(dalloc(&m->dprompt, (size_t)n_prompt));
        m->cap_prompt = n_prompt;
    }
    if (n_out > m->cap_out) {
        L2_HIP(hipStreamSynchronize(m->stream));
        m->buf_epoch++;
        dfree(m->dout_ids);
        m->dout_ids = nullptr;
        m->cap_out = 0;
        L2_TRY(dalloc(&m->dout_ids, (size_t)n_out));
        m->cap_out = n_out;
    }
    return L2_OK;
}

// The B=1 loop body with everything on the device: forward from m->dtok at
// m->dpos (== pos, which the host tracks only to size the attention scratch),
// then next = prompt[pos] if still inside the prompt else argmax
// (src/inference.rs:146-162), stored to out_ids[pos - pos0], fed back as the
// token, and the device position advanced.
static int loop_step_eager(l2_model *m, l2_state *s, int pos, int n_prompt, int pos0) {
    L2_TRY(forward_enqueue(m, s, 1, pos, true));
    LAUNCH(K_NEXT_TOKEN, next_token_launch(m->amax, m->dprompt, n_prompt, m->dpos, m->dout_ids, pos0, m->dtok, m->stream));
    return L2_OK;
}

static void step_graph_drop(StepGraph &g) {
    if (g.exec) (void)hipGraphExecDestroy(g.exec);
    if (g.graph) (void)hipGraphDestroy(g.graph);
    g = StepGraph{};
}

// The captured form of the same step for every position below `upper`: the kernels read the position, the
// prompt length and the first position of the loop from device memory (m->dpos, m->dloop), attention is
// cut for `upper` timesteps and blocks beyond the current position leave at once.
static int step_graph_get(l2_model *m, l2_state *s, int upper, hipGraphExec_t *out) {
    StepGraph &g = s->steps[upper];
    if (g.exec && g.epoch == m->buf_epoch) {
        *out = g.exec;
        return L2_OK;
    }
    step_graph_drop(g);
    L2_HIP(hipStreamBeginCapture(m->stream, hipStreamCaptureModeRelaxed));
    m->capturing = true;
    int rc = forward_enqueue(m, s, 1, upper - 1, true);
    if (rc == L2_OK)
        rc = next_token_launch(m->amax, m->dprompt, 0, m->dpos, m->dout_ids, 0, m->dtok, m->stream, m->dloop);
    m->capturing = false;
    hipGraph_t graph = nullptr;
    const hipError_t e = hipStreamEndCapture(m->stream, &graph);
    if (rc != L2_OK) {
        if (graph) (void)hipGraphDestroy(graph);
        return rc;
    }
    if (e != hipSuccess) return l2_fail(L2_ERR_HIP, "hipStreamEndCapture: %s", hipGetErrorString(e));
    g.graph = graph;
    const hipError_t e2 = hipGraphInstantiate(&g.exec, graph, nullptr, nullptr, 0);
    if (e2 != hipSuccess) {
        step_graph_drop(g);
        return l2_fail(L2_ERR_HIP, "hipGraphInstantiate: %s", hipGetErrorString(e2));
    }
    g.epoch = m->buf_epoch;
    *out = g.exec;
    return L2_OK;
}

// Positions are served in buckets [0, 256), [256, 512), [512, 1024), ...: one captured step each.
static int step_bucket(const l2_model *m, int pos) {
    long upper = 256;
    while (upper <= pos) upper *= 2;
    if (upper > m->max_seq) upper = m->max_seq;
    return (int)upper;
}

// One step of a loop whose {n_prompt, pos0} are already in m->dloop (loop_begin).
static int loop_step(l2_model *m, l2_state *s, int pos, int n_prompt, int pos0) {
    if (!m->use_graph || m->prof_on) return loop_step_eager(m, s, pos, n_prompt, pos0);
    hipGraphExec_t exec = nullptr;
    L2_TRY(step_graph_get(m, s, step_bucket(m, pos), &exec));
    L2_HIP(hipGraphLaunch(exec, m->stream));
    return L2_OK;
}

static int loop_begin(l2_model *m, int n_prompt, int pos0) {
    return set_i32_launch(m->dloop, n_prompt, m->dloop + 1, pos0, m->stream);
}

// Position at which prefill<64>, <32>, ... <2> (src/inference.rs:78-127) leave off for a prompt of n_prompt
// tokens: each takes chunks of A positions while pos + A < n_prompt (:24).
int l2_prefill_ladder_end(int n_prompt) {
    int pos = 0;
    for (int A = 64; A >= 2; A /= 2)
        while (pos + A < n_prompt) pos += A;
    return pos;
}

extern "C" int l2_generate_greedy(l2_model *m, l2_state *s, const int32_t *prompt, int n_prompt, int steps,
                                  int use_prefill, int32_t *out_ids, int *n_out, double *ms) {
    if (!m || !s || !out_ids || !n_out || (n_prompt > 0 && !prompt)) return l2_fail(L2_ERR_ARG, "null argument");
    if (s->m != m) return l2_fail(L2_ERR_ARG, "state belongs to another model");
    if (n_prompt < 0 || steps < 0) return l2_fail(L2_ERR_ARG, "negative count");
    if (steps > m->max_seq) return l2_fail(L2_ERR_RANGE, "steps %d exceeds the cache length %d", steps, m->max_seq);
    // The ladder runs whatever `steps` is: a prompt it would carry past the cache is refused before any launch
    // (the reference panics there on its fixed [SEQ_LEN] arrays).
    if (use_prefill && l2_prefill_ladder_end(n_prompt) > m->max_seq)
        return l2_fail(L2_ERR_RANGE, "a prompt of %d tokens prefills %d positions, the cache holds %d", n_prompt,
                       l2_prefill_ladder_end(n_prompt), m->max_seq);
    for (int i = 0; i < n_prompt; i++)
        if (prompt[i] < 0 || prompt[i] >= m->d.vocab_size)
            return l2_fail(L2_ERR_RANGE, "prompt token %d outside 0..%d", prompt[i], m->d.vocab_size - 1);
    L2_TRY(l2_state_reset(s)); // RunState::new per call (:59)
    L2_TRY(ensure_batch(m, use_prefill ? 64 : 1));
    L2_TRY(ensure_loop_buffers(m, std::max(n_prompt, 1), std::max(steps, 1)));
    if (n_prompt > 0)
        L2_HIP(hipMemcpyAsync(m->dprompt, prompt, (size_t)n_prompt * 4, hipMemcpyHostToDevice, m->stream));
    L2_HIP(hipStreamSynchronize(m->stream));
    const auto t0 = std::chrono::steady_clock::now(); // :72
    int pos = 0;
    if (use_prefill) { // :78-127
        static const int ladder[6] = {64, 32, 16, 8, 4, 2};
        std::vector<int32_t> toks(64), poss(64);
        for (int A : ladder) {
            while (pos + A < n_prompt) { // :24
                for (int i = 0; i < A; i++) {
                    toks[i] = pos == 0 ? 1 : prompt[pos - 1]; // START, :29-33
                    poss[i] = pos;
                    pos++;
                }
                L2_HIP(hipMemcpyAsync(m->dtok, toks.data(), (size_t)A * 4, hipMemcpyHostToDevice, m->stream));
                L2_HIP(hipMemcpyAsync(m->dpos, poss.data(), (size_t)A * 4, hipMemcpyHostToDevice, m->stream));
                if (m->prefill_mode == L2_PREFILL_MFMA)
                    L2_TRY(forward_enqueue_mfma(m, s, A, pos - 1));
                else
                    L2_TRY(forward_enqueue(m, s, A, pos - 1, false));
                L2_HIP(hipStreamSynchronize(m->stream)); // toks/poss are reused
            }
        }
    }
    const int32_t first = pos == 0 ? 1 : prompt[pos - 1]; // :128-132
    L2_TRY(set_i32_launch(m->dtok, first, m->dpos, pos, m->stream));
    const int pos0 = pos;
    L2_TRY(loop_begin(m, n_prompt, pos0));
    int n = 0;
    while (pos < steps) { // :141
        L2_TRY(loop_step(m, s, pos, n_prompt, pos0));
        n++;
        pos++;
    }
    L2_HIP(hipStreamSynchronize(m->stream));
    const auto t1 = std::chrono::steady_clock::now(); // :192
    if (n > 0) L2_HIP(hipMemcpy(out_ids, m->dout_ids, (size_t)n * 4, hipMemcpyDeviceToHost));
    *n_out = n;
    if (ms) *ms = std::chrono::duration<double, std::milli>(t1 - t0).count();
    return L2_OK;
}

// ---------------------------------------------------------------------------
// measurement hooks

extern "C" int l2_qlinear_bench(l2_qlinear **qs, int n, int iters, float *ms_total) {
    if (!qs || n < 1 || iters < 1 || !ms_total) return l2_fail(L2_ERR_ARG, "bad argument");
    hipStream_t st = qs[0]->stream;
    for (int i = 0; i < n; i++) {
        if (!qs[i]) return l2_fail(L2_ERR_ARG, "null qlinear %d", i);
        L2_TRY(qlinear_scratch(qs[i], 1));
        L2_TRY(fill_pattern_launch(qs[i]->x, (size_t)qs[i]->q.in, 17 + i, st));
    }
    hipEvent_t e0, e1;
    L2_HIP(hipEventCreate(&e0));
    L2_HIP(hipEventCreate(&e1));
    for (int i = 0; i < n; i++) L2_TRY(q4_one_natural(qs[i]->q, qs[i]->x, qs[i]->xg, qs[i]->y, 1, st)); // warm-up
    L2_HIP(hipStreamSynchronize(st));
    L2_HIP(hipEventRecord(e0, st));
    for (int it = 0; it < iters; it++) { // the whole operator: x in its natural order -> y, the act-order gather included
        l2_qlinear *q = qs[it % n];
        L2_TRY(q4_one_natural(q->q, q->x, q->xg, q->y, 1, st));
    }
    L2_HIP(hipEventRecord(e1, st));
    L2_HIP(hipEventSynchronize(e1));
    L2_HIP(hipEventElapsedTime(ms_total, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return L2_OK;
}

extern "C" int l2_qlinear_bench_dispatch(l2_qlinear **qs, int n, int iters, float *ms_sum) {
    if (!qs || n < 1 || iters < 1 || iters > 65536 || !ms_sum) return l2_fail(L2_ERR_ARG, "bad argument");
    hipStream_t st = qs[0]->stream;
    for (int i = 0; i < n; i++) {
        if (!qs[i]) return l2_fail(L2_ERR_ARG, "null qlinear %d", i);
        L2_TRY(qlinear_scratch(qs[i], 1));
        L2_TRY(fill_pattern_launch(qs[i]->x, (size_t)qs[i]->q.in, 17 + i, st));
    }
    for (int i = 0; i < n; i++) {
        Q4Launch probe = launch_of(qs[i]->q, 1, 0.f);
        probe.m[0] = mat_of(qs[i]->q, qs[i]->x, nullptr, qs[i]->y);
        if (!q4_gathers_in_kernel(probe))
            return l2_fail(L2_ERR_ARG, "dispatch timing covers the one-launch form of the operator only (in=%d)", qs[i]->q.in);
        L2_TRY(q4_one_natural(qs[i]->q, qs[i]->x, qs[i]->xg, qs[i]->y, 1, st)); // warm-up
    }
    L2_HIP(hipStreamSynchronize(st));
    std::vector<hipEvent_t> ev((size_t)iters * 2, nullptr);
    int rc = L2_OK;
    for (auto &e : ev)
        if (rc == L2_OK && hipEventCreate(&e) != hipSuccess) rc = l2_fail(L2_ERR_HIP, "hipEventCreate failed");
    int launched = 0;
    for (int it = 0; it < iters && rc == L2_OK; it++) {
        l2_qlinear *q = qs[it % n];
        g_q4_prof.start = ev[2 * (size_t)it];
        g_q4_prof.stop = ev[2 * (size_t)it + 1];
        g_q4_prof.armed = true;
        rc = q4_one_natural(q->q, q->x, q->xg, q->y, 1, st);
        if (rc == L2_OK && g_q4_prof.armed) rc = l2_fail(L2_ERR_ARG, "this form of the kernel takes no dispatch events");
        g_q4_prof.armed = false;
        if (rc == L2_OK) launched++;
    }
    const hipError_t es = hipStreamSynchronize(st);
    double sum = 0.0;
    for (int it = 0; it < launched && rc == L2_OK && es == hipSuccess; it++) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, ev[2 * (size_t)it], ev[2 * (size_t)it + 1]) != hipSuccess)
            rc = l2_fail(L2_ERR_HIP, "hipEventElapsedTime failed on dispatch %d", it);
        sum += ms;
    }
    for (auto &e : ev)
        if (e) (void)hipEventDestroy(e);
    if (rc != L2_OK) return rc;
    if (es != hipSuccess) return l2_fail(L2_ERR_HIP, "matvec bench: %s", hipGetErrorString(es));
    *ms_sum = (float)sum;
    return L2_OK;
}

extern "C" int l2_qlinear_kernel(l2_qlinear *q, char *out, size_t cap) {
    if (!q || !out || cap < 2) return l2_fail(L2_ERR_ARG, "bad argument");
    out[0] = '\0';
    const float *some = (const float *)q->bufs[2]; // only null / non-null matters for the choice of kernel
    Q4Launch L = launch_of(q->q, 1, 0.f);
    L.m[0] = mat_of(q->q, some, nullptr, nullptr);
    if (q4_gathers_in_kernel(L)) L.m[0].gidx = q->q.inv_index;
    g_q4_name.buf = out;
    g_q4_name.cap = (int)cap;
    g_q4_name.armed = true;
    const int rc = q4_matvec_launch(L, q->stream);
    const bool answered = !g_q4_name.armed;
    g_q4_name.armed = false;
    L2_TRY(rc);
    if (!answered) return l2_fail(L2_ERR_ARG, "the launcher did not name its kernel");
    return L2_OK;
}

extern "C" int l2_decode_bench(l2_model *m, l2_state *s, int32_t token, int32_t pos, int n_tokens,
                               int32_t *out_ids, float *ms_total) {
    if (!m || !s || !ms_total || n_tokens < 1) return l2_fail(L2_ERR_ARG, "bad argument");
    if (s->m != m) return l2_fail(L2_ERR_ARG, "state belongs to another model");
    if (pos < 0 || pos + n_tokens > m->max_seq) return l2_fail(L2_ERR_RANGE, "positions [%d,%d) exceed the cache", pos, pos + n_tokens);
    if (token < 0 || token >= m->d.vocab_size) return l2_fail(L2_ERR_RANGE, "token %d", token);
    L2_TRY(ensure_batch(m, 1));
    L2_TRY(ensure_loop_buffers(m, 1, n_tokens));
    L2_TRY(set_i32_launch(m->dtok, token, m->dpos, pos, m->stream));
    L2_TRY(loop_begin(m, 0, pos));
    if (m->use_graph) { // capture (if need be) outside the timed region
        hipGraphExec_t exec = nullptr;
        for (int b = step_bucket(m, pos);; b = step_bucket(m, b)) {
            L2_TRY(step_graph_get(m, s, b, &exec));
            if (b > pos + n_tokens - 1 || b >= m->max_seq) break;
        }
    }
    hipEvent_t e0, e1;
    L2_HIP(hipEventCreate(&e0));
    L2_HIP(hipEventCreate(&e1));
    L2_HIP(hipStreamSynchronize(m->stream));
    L2_HIP(hipEventRecord(e0, m->stream));
    for (int i = 0; i < n_tokens; i++) L2_TRY(loop_step(m, s, pos + i, 0, pos));
    L2_HIP(hipEventRecord(e1, m->stream));
    L2_HIP(hipEventSynchronize(e1));
    L2_HIP(hipEventElapsedTime(ms_total, e0, e1));
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (out_ids) L2_HIP(hipMemcpy(out_ids, m->dout_ids, (size_t)n_tokens * 4, hipMemcpyDeviceToHost));
    return L2_OK;
}

// Which kernel each q4 launch class of this model's decode step runs: "class=kernel;..." with the kernel's
// name as a profiler prints it (template arguments included).  Nothing is launched.
extern "C" int l2_model_q4_kernels(l2_model *m, char *out, size_t cap) {
    if (!m || !out || cap < 2) return l2_fail(L2_ERR_ARG, "bad argument");
    out[0] = '\0';
    if (m->d.group_size == 0) return L2_OK; // the model without quantisation has no q4 launches
    const int layer = 0;
    const DevQLinear &wq = m->q[L2_WQ][layer], &wk = m->q[L2_WK][layer], &wv = m->q[L2_WV][layer],
                     &wo = m->q[L2_WO][layer], &w1 = m->q[L2_W1][layer], &w2 = m->q[L2_W2][layer],
                     &w3 = m->q[L2_W3][layer];
    const float *some = (const float *)m->dimage; // only null / non-null matters for the choice of kernel
    struct { const char *cls; Q4Launch L; } items[4];
    items[0].cls = "q4_qkv";
    items[0].L = launch_of(wq, 1, m->rms_eps);
    items[0].L.m[0] = mat_of(wq, some, some, nullptr);
    items[0].L.m[1] = mat_of(wk, some, some, nullptr);
    items[0].L.m[2] = mat_of(wv, some, some, nullptr);
    items[0].L.n_mats = 3;
    items[1].cls = "q4_wo";
    items[1].L = launch_of(wo, 1, 0.f);
    items[1].L.m[0] = mat_of(wo, some, nullptr, nullptr);
    items[2].cls = "q4_w13";
    items[2].L = launch_of(w1, 1, m->rms_eps);
    items[2].L.m[0] = mat_of(w1, some, some, nullptr);
    items[2].L.m[1] = mat_of(w3, some, some, nullptr);
    items[2].L.n_mats = 2;
    items[2].L.pair = 1;
    items[3].cls = "q4_w2";
    items[3].L = launch_of(w2, 1, 0.f);
    items[3].L.m[0] = mat_of(w2, some, nullptr, nullptr);
    std::string all;
    for (auto &it : items) {
        char name[160] = "";
        g_q4_name.buf = name;
        g_q4_name.cap = (int)sizeof(name);
        g_q4_name.armed = true;
        const int rc = q4_matvec_launch(it.L, m->stream);
        const bool answered = !g_q4_name.armed;
        g_q4_name.armed = false;
        L2_TRY(rc);
        if (!answered) return l2_fail(L2_ERR_ARG, "the launcher of %s did not name its kernel", it.cls);
        all += std::string(it.cls) + "=" + name + ";";
    }
    if (all.size() + 1 > cap) return l2_fail(L2_ERR_ARG, "buffer of %zu bytes, %zu needed", cap, all.size() + 1);
    memcpy(out, all.c_str(), all.size() + 1);
    return L2_OK;
}

extern "C" int l2_q4_plan(int in, const int32_t *out, int n_mats, int group_size, int pair, int norm, char *kernel,
                          size_t cap, int32_t *geometry) {
    if (!out || !kernel || cap < 2 || !geometry || n_mats < 1 || n_mats > 3) return l2_fail(L2_ERR_ARG, "bad argument");
    if (group_size != 32 && group_size != 64 && group_size != 128) return l2_fail(L2_ERR_ARG, "group size %d", group_size);
    if (in <= 0 || in % 32 || in % group_size) return l2_fail(L2_ERR_ARG, "in=%d", in);
    static const float dummy[4] = {0.f, 0.f, 0.f, 0.f}; // only null / non-null matters: nothing is launched
    Q4Launch L{};
    L.n_mats = n_mats;
    L.in = in;
    L.groups = in / group_size;
    L.group_size = group_size;
    L.batch = 1;
    L.pair = pair ? 1 : 0;
    L.eps = 1e-5f;
    L.e.kind = pair ? Q4_EPI_SCATTER_ONLY : Q4_EPI_STORE;
    for (int i = 0; i < n_mats; i++) {
        if (out[i] <= 0 || out[i] % 8) return l2_fail(L2_ERR_ARG, "out[%d]=%d", i, out[i]);
        L.m[i].x = dummy;
        L.m[i].wn = norm ? dummy : nullptr;
        L.m[i].out = out[i];
    }
    kernel[0] = '\0';
    g_q4_name = Q4NameHook{};
    g_q4_name.buf = kernel;
    g_q4_name.cap = (int)cap;
    g_q4_name.armed = true;
    const int rc = q4_matvec_launch(L, nullptr);
    const bool answered = !g_q4_name.armed;
    g_q4_name.armed = false;
    L2_TRY(rc);
    if (!answered) return l2_fail(L2_ERR_ARG, "the launcher did not name its kernel");
    geometry[0] = g_q4_name.grid, geometry[1] = g_q4_name.block, geometry[2] = g_q4_name.rows_per_block;
    geometry[3] = (int32_t)g_q4_name.lds;
    // every row of every matrix belongs to exactly one block, and the blocks of all matrices fit the grid
    long blocks = 0;
    for (int i = 0; i < (pair ? 1 : n_mats); i++) blocks += (out[i] + geometry[2] - 1) / geometry[2];
    if (blocks != geometry[0]) return l2_fail(L2_ERR_ARG, "plan: %ld row blocks for a grid of %d", blocks, geometry[0]);
    return L2_OK;
}

extern "C" int l2_kernel_class_count(void) { return K_NCLASS; }

extern "C" const char *l2_kernel_class_name(int cls) { return cls >= 0 && cls < K_NCLASS ? kClassNames[cls] : ""; }

extern "C" int l2_decode_profile(l2_model *m, l2_state *s, int32_t token, int32_t pos, int n_tokens,
                                 float *ms_by_class, int32_t *launches_by_class) {
    if (!m || !s || !ms_by_class || !launches_by_class || n_tokens < 1) return l2_fail(L2_ERR_ARG, "bad argument");
    if (s->m != m) return l2_fail(L2_ERR_ARG, "state belongs to another model");
    if (pos < 0 || pos + n_tokens > m->max_seq) return l2_fail(L2_ERR_RANGE, "positions [%d,%d) exceed the cache", pos, pos + n_tokens);
    if (token < 0 || token >= m->d.vocab_size) return l2_fail(L2_ERR_RANGE, "token %d", token);
    L2_TRY(ensure_batch(m, 1));
    L2_TRY(ensure_loop_buffers(m, 1, n_tokens));
    L2_TRY(set_i32_launch(m->dtok, token, m->dpos, pos, m->stream));
    L2_TRY(loop_begin(m, 0, pos));
    L2_HIP(hipStreamSynchronize(m->stream));
    m->prof.clear();
    m->prof_on = true;
    int rc = L2_OK;
    for (int i = 0; i < n_tokens && rc == L2_OK; i++) rc = loop_step(m, s, pos + i, 0, pos);
    m->prof_on = false;
    hipError_t e = hipStreamSynchronize(m->stream);
    for (int c = 0; c < K_NCLASS; c++) {
        ms_by_class[c] = 0.f;
        launches_by_class[c] = 0;
    }
    for (auto &r : m->prof) {
        float ms = 0.f;
        if (rc == L2_OK && e == hipSuccess && r.e0 && r.e1 && hipEventElapsedTime(&ms, r.e0, r.e1) == hipSuccess) {
            ms_by_class[r.cls] += ms;
            launches_by_class[r.cls] += 1;
        }
        if (r.e0) (void)hipEventDestroy(r.e0);
        if (r.e1) (void)hipEventDestroy(r.e1);
    }
    m->prof.clear();
    if (rc != L2_OK) return rc;
    if (e != hipSuccess) return l2_fail(L2_ERR_HIP, "profile run: %s", hipGetErrorString(e));
    return L2_OK;
}

extern "C" int l2_copy_bench(size_t nbytes, int iters, float *ms_total) {
    if (!ms_total || nbytes < 16 || iters < 1) return l2_fail(L2_ERR_ARG, "bad argument");
    L2_TRY(require_device());
    char *a = nullptr, *b = nullptr;
    L2_TRY(dalloc(&a, nbytes));
    if (dalloc(&b, nbytes) != L2_OK) {
        dfree(a);
        return L2_ERR_HIP;
    }
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    (void)hipMemcpyAsync(b, a, nbytes, hipMemcpyDeviceToDevice, nullptr);
    (void)hipDeviceSynchronize();
    (void)hipEventRecord(e0, nullptr);
    for (int i = 0; i < iters; i++) (void)hipMemcpyAsync(b, a, nbytes, hipMemcpyDeviceToDevice, nullptr);
    (void)hipEventRecord(e1, nullptr);
    hipError_t e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipEventElapsedTime(ms_total, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    dfree(a);
    dfree(b);
    if (e != hipSuccess) return l2_fail(L2_ERR_HIP, "copy bench: %s", hipGetErrorString(e));
    return L2_OK;
}
