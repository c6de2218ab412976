/*
 * CPU restatement of the llama2.rs token loop.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the parity checker for the HIP path and the reported CPU
 * baseline.  Nothing on the product path may link, load or call it; only the
 * tests, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Every function restates one reference function operation for operation
 * (same association order, rounded multiply then rounded add, no fused
 * multiply-add: build with -ffp-contract=off) and cites it.  OpenMP over
 * output rows / heads stands where the reference uses rayon; an 8-lane GCC
 * vector stands where it uses core::simd::f32x8.
 *
 * What pins each function (see tests/test_oracle_*.py):
 *   or_qmatvec     closed-form constant cases held by src/gptq_test.rs:40-62 and
 *                  src/kernel.py:100-103; fp64 brute force of the AutoGPTQ-form
 *                  sum on the untransformed tensors; linearity, unit-vector
 *                  read-back, batch-column independence.
 *   or_dense_matvec  numpy dot (textbook).
 *   or_rmsnorm, or_silu_gate, or_softmax, or_attention  fp64 numpy closed forms,
 *                  softmax invariants, GQA head mapping by constant kv heads.
 *   or_rope        pos=0 identity, first half == textbook rotate-half, second
 *                  half == q[i]c + q'[i-h]s.  No fixture exists in the
 *                  reference and its Rust cannot be built here: parity with
 *                  the reference's in-place update order is by reading only.
 *   or_argmax      duplicates resolve to the last index.
 *   or_str_lookup, or_bpe_encode  the reference's test (tests/test_tokenizer.py:8-23)
 *                  asserts equality with the SentencePiece BPE encoding of the same
 *                  vocabulary; tests/test_oracle_tokenizer.py builds that SentencePiece
 *                  model from tokenizer.bin (pieces and scores as they stand) and compares
 *                  ids on the reference's two prompts and on seeded ordinary text; a toy
 *                  vocabulary checks the merge order by hand and the ids-from-260-first rule.
 *   or_transformer, or_generate_greedy  parity unpinned by any reference
 *                  fixture (the reference holds no checkpoint and no expected
 *                  tokens); pinned structurally: batched prefill == token by
 *                  token, output length == steps - start position.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

typedef float v8f __attribute__((vector_size(32)));
typedef int32_t v8i __attribute__((vector_size(32)));

/* Dimensions the reference fixes at compile time (src/constants.rs:7-74),
 * carried at run time here. */
typedef struct {
    int32_t dim;
    int32_t hidden_dim;
    int32_t n_layers;
    int32_t n_heads;
    int32_t n_kv_heads; /* N_HEADS / ATTN_GROUPS */
    int32_t vocab_size;
    int32_t seq_len;    /* rows of the deprecated freq tables in the file (2048) */
    int32_t group_size;
    int32_t max_seq;    /* KV cache length (reference: SEQ_LEN) */
} or_dims;

/* One QLinear viewed in place (src/gptq.rs:68-84). */
typedef struct {
    const int32_t *qweight; /* [OUT][IN/8] */
    const int32_t *qzeros;  /* [OUT/8][GROUPS] */
    const float *scales;    /* [OUT][GROUPS] */
    const int32_t *g_index; /* [IN] */
    int32_t in, out, groups;
    const float *dense;     /* quant = "no": Linear<IN,OUT>.w [OUT][IN] (src/model.rs:11-15), the others null */
} or_qlinear;

typedef struct {
    or_dims d;
    float rms_eps;
    const float *tok_emb;
    const float *rms_att;
    or_qlinear *wq, *wk, *wv, *wo;
    const float *rms_ffn;
    or_qlinear *w1, *w2, *w3;
    const float *rms_final;
    const float *wcls;
} or_model;

typedef struct {
    float *key_cache;   /* [L][max_seq][KVH][HS] */
    float *value_cache;
} or_state;

int or_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

void or_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}

static int64_t div_up(int64_t x, int64_t y) { return x / y + (x % y == 0 ? 0 : 1); }

/* src/gptq.rs:94-176.  x[B][IN], xout[B][OUT]. */
void or_qmatvec(const int32_t *qweight, const int32_t *qzeros, const float *scales,
                const int32_t *g_index, int in, int out, int group_size, int B,
                const float *x, float *xout) {
    const int ing = in / 8;
    const int groups = (int)div_up(in, group_size);
    const int ipg = group_size / 8; /* packed words per group, :127 */
    /* :110-122  act-order gather, then 8-wide transposed input */
    v8f *x_temp = (v8f *)aligned_alloc(32, (size_t)ing * B * sizeof(v8f));
    for (int b = 0; b < B; b++)
        for (int i = 0; i < ing; i++) {
            v8f t;
            for (int k = 0; k < 8; k++) t[k] = x[(size_t)b * in + g_index[i * 8 + k]];
            x_temp[(size_t)i * B + b] = t;
        }
    const v8i shift_right = {0, 4, 8, 12, 16, 20, 24, 28}; /* :129 */
    const v8i mask_4bits = {15, 15, 15, 15, 15, 15, 15, 15};

#pragma omp parallel for schedule(static)
    for (int oi = 0; oi < out; oi++) { /* :132 */
        const int32_t *qz_row = qzeros + (size_t)(oi / 8) * groups;
        const int out_elem = oi % 8;
        const int32_t *qw_row = qweight + (size_t)oi * ing;
        const float *sc_row = scales + (size_t)oi * groups;
        v8f sum[B > 0 ? B : 1];
        for (int b = 0; b < B; b++) sum[b] = (v8f){0, 0, 0, 0, 0, 0, 0, 0};
        /* zip of scales, qweight.chunks_exact(ipg), x_temp.chunks_exact(G/8), qzeros: :142-147 */
        const int ngroups_full = ing / ipg;
        const int ng = ngroups_full < groups ? ngroups_full : groups;
        for (int g = 0; g < ng; g++) {
            const int32_t qz = ((qz_row[g] >> (4 * out_elem)) & 15) + 1; /* :148 */
            const float scale = sc_row[g];
            const v8f scale_simd = {scale, scale, scale, scale, scale, scale, scale, scale};
            const v8i zero_simd = {qz, qz, qz, qz, qz, qz, qz, qz};
            for (int w = 0; w < ipg; w++) { /* :152 */
                const int32_t v = qw_row[g * ipg + w];
                const v8i num_simd = {v, v, v, v, v, v, v, v};
                const v8i qw = (num_simd >> shift_right) & mask_4bits; /* :155 */
                const v8f combine = __builtin_convertvector(qw - zero_simd, v8f);
                const v8f weight = scale_simd * combine; /* :157 */
                const v8f *xs = x_temp + (size_t)(g * ipg + w) * B;
                for (int b = 0; b < B; b++) sum[b] = sum[b] + weight * xs[b]; /* :161 */
            }
        }
        for (int b = 0; b < B; b++) { /* :166-168, ordered reduce_sum from 0 */
            float r = 0.0f;
            for (int k = 0; k < 8; k++) r = r + sum[b][k];
            xout[(size_t)b * out + oi] = 0.0f + r;
        }
    }
    free(x_temp);
}

/* src/model.rs:22-31.  w[OUT][IN]; strictly sequential fold from 0. */
void or_dense_matvec(const float *w, int in, int out, int B, const float *x, float *xout) {
    for (int b = 0; b < B; b++) {
        const float *xb = x + (size_t)b * in;
        float *ob = xout + (size_t)b * out;
#pragma omp parallel for schedule(static)
        for (int i = 0; i < out; i++) {
            const float *row = w + (size_t)i * in;
            float acc = 0.0f;
            for (int j = 0; j < in; j++) acc = acc + row[j] * xb[j];
            ob[i] = acc;
        }
    }
}

/* src/models.rs:47-51 */
void or_accum(float *a, const float *b, int n) {
    for (int i = 0; i < n; i++) a[i] += b[i];
}

/* src/models.rs:53-66 */
void or_rmsnorm(float *o, const float *xo, const float *weight, float epsilon, int dim) {
    float ss = 0.0f;
    for (int j = 0; j < dim; j++) ss = ss + xo[j] * xo[j];
    ss /= (float)dim;
    ss += epsilon;
    ss = 1.0f / sqrtf(ss);
    for (int j = 0; j < dim; j++) o[j] = weight[j] * ss * xo[j];
}

/* src/models.rs:68-81 */
void or_softmax(float *x, int n) {
    float max_val = x[0];
    for (int i = 0; i < n; i++) max_val = fmaxf(max_val, x[i]);
    float sum = 0.0f;
    for (int i = 0; i < n; i++) {
        x[i] = expf(x[i] - max_val);
        sum += x[i];
    }
    for (int i = 0; i < n; i++) x[i] /= sum;
}

/* src/models.rs:83-89 */
static float or_dot(const float *q, const float *k, int n) {
    float s = 0.0f;
    for (int i = 0; i < n; i++) s = s + q[i] * k[i];
    return s;
}

/* src/models.rs:92-98 */
void or_silu_gate(float *s, const float *s2, int n) {
    for (int i = 0; i < n; i++) {
        s[i] = s[i] * (1.0f / (1.0f + expf(-s[i])));
        s[i] = s[i] * s2[i];
    }
}

/* src/models.rs:100-129.  The update is in place: the second half of each head
 * reads first-half entries that this same call has already rotated. */
void or_rope(float *queries, float *keys, int pos, int n_heads, int n_kv_heads, int head_size) {
    const int half = head_size / 2;
    for (int h = 0; h < n_heads; h++) {
        float *q = queries + (size_t)h * head_size;
        for (int i = 0; i < head_size; i++) {
            const float freq =
                1.0f / powf(10000.0f, ((float)((2 * i) % head_size)) / (float)head_size);
            const float val = (float)pos * freq;
            const float fcr = cosf(val);
            const float fci = sinf(val);
            if (i < half)
                q[i] = q[i] * fcr - q[half + i] * fci;
            else
                q[i] = q[i] * fcr + q[i - half] * fci;
            if (h < n_kv_heads) {
                float *k = keys + (size_t)h * head_size;
                if (i < half)
                    k[i] = k[i] * fcr - k[half + i] * fci;
                else
                    k[i] = k[i] * fcr + k[i - half] * fci;
            }
        }
    }
}

/* cos/sin of the angle the reference recomputes per element (models.rs:107-110),
 * exposed so that a table-driven implementation can be checked against the very
 * same libm calls.  cos_out/sin_out: [head_size/2]. */
void or_rope_table_row(int pos, int head_size, float *cos_out, float *sin_out) {
    for (int i = 0; i < head_size / 2; i++) {
        const float freq =
            1.0f / powf(10000.0f, ((float)((2 * i) % head_size)) / (float)head_size);
        const float val = (float)pos * freq;
        cos_out[i] = cosf(val);
        sin_out[i] = sinf(val);
    }
}

/* src/models.rs:131-176.  One layer's caches: [max_seq][KVH][HS].
 * out/queries: [B][DIM]. */
void or_attention(float *out, const float *queries, const float *value_cache,
                  const float *key_cache, const int *pos, int B, int n_heads, int n_kv_heads,
                  int head_size) {
    const int dim = n_heads * head_size;
    const int attn_groups = n_heads / n_kv_heads;
    const size_t row = (size_t)n_kv_heads * head_size;
    for (int b = 0; b < B; b++) {
        const int p = pos[b];
#pragma omp parallel for schedule(dynamic, 1)
        for (int h = 0; h < n_heads; h++) {
            const float *q = queries + (size_t)b * dim + (size_t)h * head_size;
            float *xb = out + (size_t)b * dim + (size_t)h * head_size;
            float *att = (float *)malloc(sizeof(float) * (size_t)(p + 1));
            const size_t hoff = (size_t)(h / attn_groups) * head_size;
            for (int t = 0; t <= p; t++) {
                const float *k = key_cache + (size_t)t * row + hoff;
                att[t] = or_dot(q, k, head_size) / sqrtf((float)head_size);
            }
            or_softmax(att, p + 1);
            for (int i = 0; i < head_size; i++) xb[i] = 0.0f;
            for (int t = 0; t <= p; t++) {
                const float *v = value_cache + (size_t)t * row + hoff;
                for (int i = 0; i < head_size; i++) xb[i] += att[t] * v[i];
            }
            free(att);
        }
    }
}

/* src/util.rs:39-46.  reduce(|a,b| if a.1 > b.1 {a} else {b}): ties (and any
 * comparison that is false) keep the later element. */
int or_argmax(const float *v, int n) {
    int bi = 0;
    float bv = v[0];
    for (int i = 1; i < n; i++) {
        if (bv > v[i]) {
        } else {
            bi = i;
            bv = v[i];
        }
    }
    return bi;
}

/* ------------------------------------------------------------------------- */
/* Checkpoint image: src/gptq.rs:34-84 field order, src/lib.rs:88-104 sizing. */

static size_t qlinear_bytes(int in, int out, int g) {
    const size_t groups = (size_t)div_up(in, g);
    return (size_t)out * (in / 8) * 4 + (size_t)(out / 8) * groups * 4 +
           (size_t)out * groups * 4 + (size_t)in * 4;
}

/* size_of::<TransformerWeights>() (src/model.rs:36-67): the build without quantisation,
 * GROUPSIZE = 0 (src/constants.rs:58-61); every projection a dense Linear. */
static size_t dense_weights_bytes(const or_dims *d) {
    const int hs = d->dim / d->n_heads;
    const size_t kv_dim = (size_t)d->n_kv_heads * hs, dim = (size_t)d->dim, hid = (size_t)d->hidden_dim;
    const size_t L = (size_t)d->n_layers;
    size_t n = 4 + (size_t)d->vocab_size * dim * 4 + L * dim * 4;
    n += L * (dim * dim + 2 * kv_dim * dim + dim * dim) * 4; /* wq wk wv wo */
    n += L * dim * 4;
    n += L * 3 * hid * dim * 4;                              /* w1 w2 w3 */
    n += dim * 4 + (size_t)d->seq_len * (hs / 2) * 4 * 2 + (size_t)d->vocab_size * dim * 4;
    return n;
}

/* size_of::<QTransformerWeights>() for these dims (the part after the 28-byte header). */
size_t or_weights_bytes(const or_dims *d) {
    if (d->group_size == 0) return dense_weights_bytes(d);
    const int hs = d->dim / d->n_heads;
    const int kv_dim = d->n_kv_heads * hs;
    const size_t L = (size_t)d->n_layers;
    size_t n = 4;                                   /* rms_eps */
    n += (size_t)d->vocab_size * d->dim * 4;        /* token_embedding_table */
    n += L * d->dim * 4;                            /* rms_att_weight */
    n += L * qlinear_bytes(d->dim, d->dim, d->group_size);     /* wq */
    n += L * qlinear_bytes(d->dim, kv_dim, d->group_size) * 2; /* wk wv */
    n += L * qlinear_bytes(d->dim, d->dim, d->group_size);     /* wo */
    n += L * d->dim * 4;                            /* rms_ffn_weight */
    n += L * qlinear_bytes(d->dim, d->hidden_dim, d->group_size) * 2; /* w1 w3 */
    n += L * qlinear_bytes(d->hidden_dim, d->dim, d->group_size);     /* w2 */
    n += (size_t)d->dim * 4;                        /* rms_final_weight */
    n += (size_t)d->seq_len * (hs / 2) * 4 * 2;     /* deprecated freq tables */
    n += (size_t)d->vocab_size * d->dim * 4;        /* wcls */
    return n;
}

static const char *take_qlinears(const char *p, or_qlinear *ql, int L, int in, int out, int g) {
    if (g == 0) { /* dense Linear<IN,OUT> */
        for (int l = 0; l < L; l++) {
            ql[l].in = in;
            ql[l].out = out;
            ql[l].dense = (const float *)p;
            p += (size_t)out * in * 4;
        }
        return p;
    }
    const int groups = (int)div_up(in, g);
    for (int l = 0; l < L; l++) {
        ql[l].in = in;
        ql[l].out = out;
        ql[l].groups = groups;
        ql[l].qweight = (const int32_t *)p;
        p += (size_t)out * (in / 8) * 4;
        ql[l].qzeros = (const int32_t *)p;
        p += (size_t)(out / 8) * groups * 4;
        ql[l].scales = (const float *)p;
        p += (size_t)out * groups * 4;
        ql[l].g_index = (const int32_t *)p;
        p += (size_t)in * 4;
    }
    return p;
}

/* View a weights image (bytes after the header) as a model.  Returns NULL if
 * nbytes differs from the struct size (src/lib.rs:97). */
or_model *or_model_view(const void *weights, size_t nbytes, const or_dims *d) {
    if (nbytes != or_weights_bytes(d)) return NULL;
    or_model *m = (or_model *)calloc(1, sizeof(or_model));
    m->d = *d;
    const int L = d->n_layers;
    const int hs = d->dim / d->n_heads;
    const int kv_dim = d->n_kv_heads * hs;
    or_qlinear *all = (or_qlinear *)calloc((size_t)7 * L, sizeof(or_qlinear));
    m->wq = all;
    m->wk = all + L;
    m->wv = all + 2 * L;
    m->wo = all + 3 * L;
    m->w1 = all + 4 * L;
    m->w2 = all + 5 * L;
    m->w3 = all + 6 * L;
    const char *p = (const char *)weights;
    memcpy(&m->rms_eps, p, 4);
    p += 4;
    m->tok_emb = (const float *)p;
    p += (size_t)d->vocab_size * d->dim * 4;
    m->rms_att = (const float *)p;
    p += (size_t)L * d->dim * 4;
    p = take_qlinears(p, m->wq, L, d->dim, d->dim, d->group_size);
    p = take_qlinears(p, m->wk, L, d->dim, kv_dim, d->group_size);
    p = take_qlinears(p, m->wv, L, d->dim, kv_dim, d->group_size);
    p = take_qlinears(p, m->wo, L, d->dim, d->dim, d->group_size);
    m->rms_ffn = (const float *)p;
    p += (size_t)L * d->dim * 4;
    p = take_qlinears(p, m->w1, L, d->dim, d->hidden_dim, d->group_size);
    p = take_qlinears(p, m->w2, L, d->hidden_dim, d->dim, d->group_size);
    p = take_qlinears(p, m->w3, L, d->dim, d->hidden_dim, d->group_size);
    m->rms_final = (const float *)p;
    p += (size_t)d->dim * 4;
    p += (size_t)d->seq_len * (hs / 2) * 4 * 2;
    m->wcls = (const float *)p;
    return m;
}

void or_model_free(or_model *m) {
    if (!m) return;
    free(m->wq);
    free(m);
}

/* src/models.rs:36-41 */
or_state *or_state_new(const or_model *m) {
    const or_dims *d = &m->d;
    const int hs = d->dim / d->n_heads;
    const size_t n = (size_t)d->n_layers * d->max_seq * d->n_kv_heads * hs;
    or_state *s = (or_state *)calloc(1, sizeof(or_state));
    s->key_cache = (float *)calloc(n, sizeof(float));
    s->value_cache = (float *)calloc(n, sizeof(float));
    if (!s->key_cache || !s->value_cache) {
        free(s->key_cache);
        free(s->value_cache);
        free(s);
        return NULL;
    }
    return s;
}

void or_state_free(or_state *s) {
    if (!s) return;
    free(s->key_cache);
    free(s->value_cache);
    free(s);
}

float *or_state_key_cache(or_state *s) { return s->key_cache; }
float *or_state_value_cache(or_state *s) { return s->value_cache; }

static void qmv(const or_qlinear *q, int g, int B, const float *x, float *y) {
    if (q->dense) {
        or_dense_matvec(q->dense, q->in, q->out, B, x, y);
        return;
    }
    or_qmatvec(q->qweight, q->qzeros, q->scales, q->g_index, q->in, q->out, g, B, x, y);
}

/* src/models.rs:178-298.  logits[vocab] is written only when B == 1. */
void or_transformer(const or_model *m, or_state *s, const int *tokens, const int *pos, int B,
                    float *logits) {
    const or_dims *d = &m->d;
    const int dim = d->dim, hid = d->hidden_dim, L = d->n_layers;
    const int hs = dim / d->n_heads;
    const int kv_dim = d->n_kv_heads * hs;
    const int G = d->group_size;
    const size_t layer_stride = (size_t)d->max_seq * kv_dim;
    float *x = (float *)malloc(sizeof(float) * (size_t)B * dim);
    float *xb = (float *)malloc(sizeof(float) * (size_t)B * dim);
    float *xb2 = (float *)malloc(sizeof(float) * (size_t)B * dim);
    float *hb = (float *)malloc(sizeof(float) * (size_t)B * hid);
    float *hb2 = (float *)malloc(sizeof(float) * (size_t)B * hid);
    float *q = (float *)malloc(sizeof(float) * (size_t)B * dim);
    float *k = (float *)malloc(sizeof(float) * (size_t)B * kv_dim);
    float *v = (float *)malloc(sizeof(float) * (size_t)B * kv_dim);

    for (int b = 0; b < B; b++) /* :189-191 */
        memcpy(x + (size_t)b * dim, m->tok_emb + (size_t)tokens[b] * dim, sizeof(float) * dim);

    for (int l = 0; l < L; l++) {
        for (int b = 0; b < B; b++) /* :217-219 */
            or_rmsnorm(xb + (size_t)b * dim, x + (size_t)b * dim, m->rms_att + (size_t)l * dim,
                       m->rms_eps, dim);
        qmv(&m->wq[l], G, B, xb, q); /* :224-226 */
        qmv(&m->wk[l], G, B, xb, k);
        qmv(&m->wv[l], G, B, xb, v);
        for (int b = 0; b < B; b++) /* :228-230 */
            or_rope(q + (size_t)b * dim, k + (size_t)b * kv_dim, pos[b], d->n_heads,
                    d->n_kv_heads, hs);
        float *kc = s->key_cache + (size_t)l * layer_stride;
        float *vc = s->value_cache + (size_t)l * layer_stride;
        for (int b = 0; b < B; b++) { /* :236-249 */
            memcpy(kc + (size_t)pos[b] * kv_dim, k + (size_t)b * kv_dim, sizeof(float) * kv_dim);
            memcpy(vc + (size_t)pos[b] * kv_dim, v + (size_t)b * kv_dim, sizeof(float) * kv_dim);
        }
        or_attention(xb, q, vc, kc, pos, B, d->n_heads, d->n_kv_heads, hs); /* :250-256 */
        qmv(&m->wo[l], G, B, xb, xb2); /* :260 */
        for (int b = 0; b < B; b++) { /* :263-267 */
            or_accum(x + (size_t)b * dim, xb2 + (size_t)b * dim, dim);
            or_rmsnorm(xb + (size_t)b * dim, x + (size_t)b * dim, m->rms_ffn + (size_t)l * dim,
                       m->rms_eps, dim);
        }
        qmv(&m->w1[l], G, B, xb, hb); /* :271-272 */
        qmv(&m->w3[l], G, B, xb, hb2);
        for (int b = 0; b < B; b++) /* :274-276 */
            or_silu_gate(hb + (size_t)b * hid, hb2 + (size_t)b * hid, hid);
        qmv(&m->w2[l], G, B, hb, xb); /* :279 */
        for (int b = 0; b < B; b++) /* :283-285 */
            or_accum(x + (size_t)b * dim, xb + (size_t)b * dim, dim);
    }
    if (B == 1) { /* :288-297 */
        or_rmsnorm(xb, x, m->rms_final, m->rms_eps, dim);
        or_dense_matvec(m->wcls, dim, d->vocab_size, 1, xb, logits);
    }
    free(x);
    free(xb);
    free(xb2);
    free(hb);
    free(hb2);
    free(q);
    free(k);
    free(v);
}

/* src/inference.rs:16-44 */
static void or_prefill(int A, int *pos, or_state *s, const int *prompt, int n_prompt,
                       const or_model *m) {
    int *tokens = (int *)malloc(sizeof(int) * A);
    int *positions = (int *)malloc(sizeof(int) * A);
    while (*pos + A < n_prompt) {
        for (int i = 0; i < A; i++) {
            const int next = (*pos == 0) ? 1 /* START */ : prompt[*pos - 1];
            positions[i] = *pos;
            tokens[i] = next;
            *pos += 1;
        }
        or_transformer(m, s, tokens, positions, A, NULL);
    }
    free(tokens);
    free(positions);
}

/* src/inference.rs:49-193 at temperature 0, on token ids.  `steps` counts
 * prompt positions too (:141).  out_ids receives `next` of every loop
 * iteration (:178-186); returns how many were written (steps - start pos).
 * use_prefill mirrors model.prefill() (:78).  A fresh RunState is made per
 * call (:59) unless state is given. */
int or_generate_greedy(const or_model *m, or_state *state, const int *prompt, int n_prompt,
                       int steps, int use_prefill, int *out_ids, float *last_logits) {
    or_state *own = NULL;
    if (!state) {
        own = or_state_new(m);
        state = own;
    }
    int pos = 0;
    if (use_prefill) {
        static const int ladder[6] = {64, 32, 16, 8, 4, 2}; /* :79-126 */
        for (int i = 0; i < 6; i++) or_prefill(ladder[i], &pos, state, prompt, n_prompt, m);
    }
    int token = (pos == 0) ? 1 : prompt[pos - 1]; /* :128-132 */
    float *logits = (float *)malloc(sizeof(float) * (size_t)m->d.vocab_size);
    int n = 0;
    while (pos < steps) { /* :141 */
        or_transformer(m, state, &token, &pos, 1, logits);
        int next;
        if (pos < n_prompt)
            next = prompt[pos]; /* :154-156 */
        else
            next = or_argmax(logits, m->d.vocab_size); /* :160-162 */
        out_ids[n++] = next;
        token = next;
        pos += 1;
    }
    if (last_logits && n > 0) memcpy(last_logits, logits, sizeof(float) * (size_t)m->d.vocab_size);
    free(logits);
    or_state_free(own);
    return n;
}

/* ---- tokenizer --------------------------------------------------------------
 * The vocabulary as Tokenizer::load leaves it (src/tokenizer.rs:22-37): n strings,
 * string i = bytes[off[i] .. off[i+1]), and their scores. */

/* util::str_lookup (src/util.rs:29-37): the first perfect match among ids 260.., and only if there is none
 * the first match from the start.  A linear scan, as in the reference.  -1 = None. */
int or_str_lookup(const char *str, int len, const char *bytes, const int32_t *off, int n) {
    for (int i = 260; i < n; i++)
        if (off[i + 1] - off[i] == len && memcmp(bytes + off[i], str, (size_t)len) == 0) return i;
    for (int i = 0; i < n; i++)
        if (off[i + 1] - off[i] == len && memcmp(bytes + off[i], str, (size_t)len) == 0) return i;
    return -1;
}

static int utf8_len(unsigned char c) { return c < 0x80 ? 1 : (c >> 5) == 6 ? 2 : (c >> 4) == 14 ? 3 : 4; }

/* Tokenizer::bpe_encode (src/tokenizer.rs:46-108).  text: UTF-8, text_len bytes.  Returns the number of
 * tokens written to `tokens` (capacity cap >= number of characters), -1 if a character is not in the
 * vocabulary (the reference's expect("not good")), -2 if cap is too small or the text is empty (the
 * reference's `0..(tokens.len() - 1)` underflows on an empty vector). */
int or_bpe_encode(const char *text, int text_len, const char *bytes, const int32_t *off, const float *scores,
                  int n, int32_t *tokens, int cap) {
    int nt = 0;
    /* :52-61 every character (Unicode scalar value) on its own */
    for (int i = 0; i < text_len;) {
        int l = utf8_len((unsigned char)text[i]);
        if (i + l > text_len) l = text_len - i;
        const int id = or_str_lookup(text + i, l, bytes, off, n);
        if (id < 0) return -1;
        if (nt >= cap) return -2;
        tokens[nt++] = id;
        i += l;
    }
    if (nt == 0) return -2;
    char *buf = (char *)malloc(1 << 16);
    if (!buf) return -2;
    for (;;) { /* :64-107 merge the best consecutive pair until none is in the vocabulary */
        float best_score = -1e10f;
        int best_id = 0, best_idx = -1;
        for (int i = 0; i < nt - 1; i++) {
            const int a = tokens[i], b = tokens[i + 1];
            const int la = off[a + 1] - off[a], lb = off[b + 1] - off[b];
            if (la + lb > (1 << 16)) continue;
            memcpy(buf, bytes + off[a], (size_t)la);
            memcpy(buf + la, bytes + off[b], (size_t)lb);
            const int id = or_str_lookup(buf, la + lb, bytes, off, n);
            if (id >= 0 && scores[id] > best_score) { /* strict: the leftmost of equal scores stays */
                best_score = scores[id];
                best_id = id;
                best_idx = i;
            }
        }
        if (best_idx < 0) break;
        tokens[best_idx] = best_id;
        for (int i = best_idx + 1; i < nt - 1; i++) tokens[i] = tokens[i + 1];
        nt--;
    }
    free(buf);
    return nt;
}
