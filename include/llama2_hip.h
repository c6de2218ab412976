/*
 * llama2_hip.h — C ABI of the MI355X (gfx950) token loop for llama2.rs.
 *
 * One shared library, libllama2_hip.so, stands where the reference's CUDA
 * path (src/gptq_cuda.rs + src/gptq.ptx) and its per-token CPU math stand.
 * Every entry point takes plain pointers and sizes; none takes or returns a
 * torch or HIP type.  Citations are file:line in the reference tree.
 *
 * Conventions
 *   - Every function that can fail returns an int: 0 on success, a negative
 *     L2_ERR_* otherwise, and never throws or aborts across the boundary.
 *     l2_last_error() returns the text of the calling thread's last failure.
 *     (The reference panics instead — src/lib.rs:89,96, src/gptq_cuda.rs:166;
 *     a Rust or Python wrapper turns a non-zero code into that panic or an
 *     exception.)
 *   - Handles are single-threaded, like the reference's single driver thread:
 *     one HIP stream per model, calls on one handle serialised by the caller.
 *   - "host" pointers are ordinary process memory; the library copies.
 *   - There is no CPU fallback: without a usable gfx950 device every compute
 *     entry point fails with L2_ERR_HIP.
 */
#ifndef LLAMA2_HIP_H
#define LLAMA2_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define L2_OK 0
#define L2_ERR_ARG (-1)    /* null pointer, bad size, unsupported shape          */
#define L2_ERR_IO (-2)     /* open/stat/mmap failed                               */
#define L2_ERR_FORMAT (-3) /* header != expected dims, or file size != struct size */
#define L2_ERR_HIP (-4)    /* no device, allocation or launch failure             */
#define L2_ERR_RANGE (-5)  /* token id, position, layer or batch out of range     */

/* Projection selector for l2_model_qmatvec: the QLinear fields of
 * QTransformerWeights in declaration order (src/gptq.rs:45-55). */
enum { L2_WQ = 0, L2_WK = 1, L2_WV = 2, L2_WO = 3, L2_W1 = 4, L2_W2 = 5, L2_W3 = 6 };

/* How l2_forward treats B > 1 (a prefill chunk). */
enum {
    L2_PREFILL_FP32 = 0, /* same fp32 kernels as decode, one pass per column: identical to B=1 */
    L2_PREFILL_MFMA = 1  /* dequant -> fp16 tiles -> MFMA, fp32 accumulate (tolerance 2e-3)    */
};

/* Run-time form of the reference's compile-time constants
 * (src/constants.rs:7-74: DIM, HIDDEN_DIM, N_LAYERS, N_HEADS, N_KV_HEADS =
 * N_HEADS / ATTN_GROUPS, VOCAB_SIZE, SEQ_LEN, GROUPSIZE). */
typedef struct l2_dims {
    int32_t dim;
    int32_t hidden_dim;
    int32_t n_layers;
    int32_t n_heads;
    int32_t n_kv_heads;
    int32_t vocab_size;
    int32_t seq_len;    /* rows of the deprecated freq tables stored in the file (2048) */
    int32_t group_size; /* 32, 64 or 128; 0 = the model without quantisation (GROUPSIZE 0, src/constants.rs:58-61):
                         * TransformerWeights, every projection a dense [OUT][IN] fp32 matrix (src/model.rs:36-67) */
} l2_dims;

/* Config as read from the 28-byte header (src/constants.rs:80-89, 102-119). */
typedef struct l2_config {
    int32_t dim;
    int32_t hidden_dim;
    int32_t n_layers;
    int32_t n_heads;
    int32_t n_kv_heads;
    int32_t vocab_size;
    int32_t seq_len;
    int32_t shared_weight;
} l2_config;

typedef struct l2_model l2_model;     /* LlamaModel + uploaded TWeights */
typedef struct l2_state l2_state;     /* RunState: the device KV cache  */
typedef struct l2_qlinear l2_qlinear; /* one uploaded QLinear           */

const char *l2_last_error(void);

/* Number of usable gfx950 devices (0 if none).  Never fails. */
int l2_device_count(void);

/* Cargo features "7B" | "13B" | "70B" with group_32 | group_64 | group_128
 * (Cargo.toml:28-42, build.rs:5-36, src/constants.rs:7-61). */
int l2_preset(const char *model_size, int group_size, l2_dims *out);

/* size_of::<QTransformerWeights>() for these dims: the byte count that
 * src/lib.rs:97 asserts the mapped file (after its 28-byte header) to have. */
size_t l2_weights_bytes(const l2_dims *dims);

/* LlamaModel::from_file (src/lib.rs:88-104, gpu variant :45-63): open, read
 * the header, check it against `expect` as Config::check_static does
 * (src/constants.rs:94-100: dim, hidden_dim, n_layers, n_heads, vocab_size),
 * map the file, check its size, upload once.  max_seq is the KV-cache length
 * (the reference's SEQ_LEN); 0 means expect->seq_len. */
int l2_model_open(const char *path, const l2_dims *expect, int max_seq, l2_model **out);

/* convert(&QTransformerWeights) (src/gptq_cuda.rs:50-90): upload a weights
 * image that the caller already holds in memory (e.g. its own mmap at byte 28
 * of the file).  The image is not referenced after the call returns. */
int l2_model_from_image(const void *weights, size_t nbytes, const l2_dims *dims, int max_seq,
                        l2_model **out);

void l2_model_close(l2_model *m);

/* LlamaModel.config (src/lib.rs:32,75). */
int l2_model_config(const l2_model *m, l2_config *out);
int l2_model_dims(const l2_model *m, l2_dims *out);
int l2_model_max_seq(const l2_model *m);

/* LlamaModel::prefill() (src/lib.rs:41-43 returns false for the CUDA build,
 * :84-86 true for the CPU build): 1 here, batched forward is supported. */
int l2_prefill_supported(const l2_model *m);

/* Choose how B > 1 is computed (L2_PREFILL_*).  Default L2_PREFILL_FP32. */
int l2_model_set_prefill_mode(l2_model *m, int mode);

/* Decode steps (B = 1 inside l2_generate_greedy, l2_decode_greedy, l2_decode_bench) as captured HIP graphs,
 * one per bucket of positions [0,256), [256,512), [512,1024), ..., replayed with one host call per token.
 * No counterpart in the reference.  Off by default (the step is bound by its kernels, not by their
 * launches); on, the results are the same tokens.  Environment: L2_STEP_GRAPH=1 turns it on at load. */
int l2_model_set_step_graph(l2_model *m, int on);

/* RunState::new (src/models.rs:36-41): zero-filled fp32 KV cache
 * [n_layers][max_seq][n_kv_heads][head_size] x2 in device memory. */
int l2_state_new(l2_model *m, l2_state **out);
void l2_state_free(l2_state *s);
int l2_state_reset(l2_state *s);
/* Copy cache rows [pos0, pos0+npos) of one layer to host: k,v are
 * [npos][n_kv_heads][head_size].  For tests (the reference's fields are
 * private, src/models.rs:29-33). */
int l2_state_read_kv(l2_state *s, int layer, int pos0, int npos, float *k_host, float *v_host);
/* The inverse: overwrite cache rows [pos0, pos0+npos) of one layer from host
 * arrays of the same shape.  With l2_state_read_kv this snapshots and restores
 * a RunState (the reference clones the boxed struct, src/models.rs:29-42), so
 * that a shared prompt prefix is computed once. */
int l2_state_write_kv(l2_state *s, int layer, int pos0, int npos, const float *k_host, const float *v_host);
/* QLinear::convert + QLinearCuda (src/gptq_cuda.rs:70-110): upload the four
 * arrays of one QLinear in `.bin` layout (src/gptq.rs:68-84):
 *   qweight i32[out][in/8], qzeros i32[out/8][groups], scales f32[out][groups],
 *   g_index i32[in].   Requires in % 32 == 0, out % 8 == 0, in % group_size == 0. */
int l2_qlinear_create(const int32_t *qweight, const int32_t *qzeros, const float *scales,
                      const int32_t *g_index, int in, int out, int group_size, l2_qlinear **ql);
void l2_qlinear_free(l2_qlinear *q);

/* QLinear::matvec<B> / QLinearCuda::matvec<1> (src/gptq.rs:94-176,
 * src/gptq_cuda.rs:120-179): x_host f32[B][in] -> y_host f32[B][out], fully
 * overwritten, synchronous.  fp32 throughout (the CUDA path's fp16 rounding of
 * x and y is not reproduced; the CPU path is the parity target). */
int l2_qlinear_matvec(l2_qlinear *q, const float *x_host, int B, float *y_host);

/* The same operator for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  x_dev f32[B][in] and
 * y_dev f32[B][out] are DEVICE pointers; the gather and the matvec are enqueued on hip_stream (a
 * hipStream_t; NULL is the default stream) and the call returns without waiting.  It calls no hipMalloc,
 * hipFree or other allocating routine: the one intermediate (x in the layer's act-order) lives in a fixed
 * device array of L2_MATVEC_DEVICE_MAX_ELEMS floats (4 MiB) that each GPU holds until the process
 * ends, so B * in must not exceed that count (L2_ERR_RANGE otherwise).  All calls on one GPU share the array:
 * calls that overlap in time on one GPU (two streams, two threads) race; serialise them.  y equals
 * l2_qlinear_matvec's bit for bit.  What a first launch does besides enqueueing (loading the code object on the
 * device, raising the kernel's LDS limit, resolving the array's address) l2_qlinear_create has already done, with
 * the device that is current at that time: a handle is used on the device it was created on, and every call
 * here, the first included, may be made while hip_stream is being captured into a graph.  Nothing it enqueues
 * is a memset node. */
#define L2_MATVEC_DEVICE_MAX_ELEMS (1u << 20)
int l2_qlinear_matvec_device(l2_qlinear *q, const float *x_dev, int B, float *y_dev, void *hip_stream);

/* The same operator on a projection of a loaded model: w.wq[layer].matvec(..). */
int l2_model_qmatvec(l2_model *m, int layer, int proj, const float *x_host, int B, float *y_host);

/* Linear::matvec<1> for wcls (src/model.rs:22-31, called at src/models.rs:295):
 * x_host f32[dim] -> y_host f32[vocab_size]. */
int l2_model_classifier(l2_model *m, const float *x_host, float *y_host);

/* transformer::<B> (src/models.rs:178-298): tokens/pos are host i32[B].
 * logits_host f32[vocab_size] is written only when B == 1 (:288) and may be
 * NULL to skip the copy.  All B cache rows are written before attention (:236-256). */
int l2_forward(l2_model *m, l2_state *s, const int32_t *tokens, const int32_t *pos, int B,
               float *logits_host);

/* prefill::<A> over a whole prompt (src/inference.rs:16-40, the calls at :78-127 with one A): tokens[i], host
 * i32[n], goes to position pos0 + i; the prompt is cut into chunks of `chunk` tokens (the last one may be
 * shorter) and every chunk is what l2_forward computes for it, cache rows included; no logits.  In the
 * matrix-core mode consecutive chunks run on two HIP streams of the model, one layer apart (a chunk needs from
 * the one before it only that chunk's cache rows of the same layer); the call returns when all are done. */
int l2_prefill_chunks(l2_model *m, l2_state *s, const int32_t *tokens, int n, int pos0, int chunk);

/* One iteration of the B=1 loop at temperature 0 (src/inference.rs:141-162):
 * forward, then util::argmax (src/util.rs:39-46, ties -> last index) on the
 * device.  Only the token id crosses the boundary. */
int l2_decode_greedy(l2_model *m, l2_state *s, int32_t token, int32_t pos, int32_t *next);

/* generate() at temperature 0 on token ids (src/inference.rs:49-193): resets
 * the state (:59), runs the prefill ladder 64/32/16/8/4/2 if use_prefill
 * (:78-127), then the B=1 loop with prompt forcing (:141-190).  `steps` counts
 * prompt positions too.  out_ids receives `next` of every loop iteration
 * (capacity >= steps); *n_out how many; *ms wall-clock milliseconds of the
 * same region the reference times (:72,192), prefill included. */
int l2_generate_greedy(l2_model *m, l2_state *s, const int32_t *prompt, int n_prompt, int steps,
                       int use_prefill, int32_t *out_ids, int *n_out, double *ms);

/* ---- text surface: tokenizer, Random, generate on strings ----------------- */

typedef struct l2_tokenizer l2_tokenizer; /* Tokenizer (src/tokenizer.rs:13-19) */
typedef struct l2_random l2_random;       /* Random    (src/util.rs:55-58)      */

/* Tokenizer::new (src/tokenizer.rs:41-44, load :22-37): the llama2.c format,
 * i32 max_token_length then vocab_size x {f32 score, i32 len, bytes}.  The
 * reference reads VOCAB_SIZE entries; pass that count. */
int l2_tokenizer_open(const char *path, int vocab_size, l2_tokenizer **out);
void l2_tokenizer_free(l2_tokenizer *t);
int l2_tokenizer_vocab_size(const l2_tokenizer *t);
/* vocab[id] (not NUL-terminated: use *len) and vocab_scores[id]. */
int l2_tokenizer_token(const l2_tokenizer *t, int id, const char **str, int *len, float *score);
/* Tokenizer::bpe_encode (src/tokenizer.rs:46-108) with util::str_lookup's
 * ids-from-260-first rule (src/util.rs:29-37).  text is UTF-8; *n receives the
 * count; ids may be NULL to ask for it.  A character missing from the
 * vocabulary is an error (the reference's expect("not good")). */
int l2_tokenizer_encode(const l2_tokenizer *t, const char *text, int32_t *ids, int cap, int *n);

/* Random::new (src/util.rs:61-69) seeds from the wall clock in seconds
 * (from_clock != 0); a fixed seed is offered for tests. */
int l2_random_new(uint64_t seed, int from_clock, l2_random **out);
void l2_random_free(l2_random *r);
float l2_random_f32(l2_random *r);                                   /* Random::random, :79-82  */
int l2_random_sample(l2_random *r, const float *probabilities, int n); /* Random::sample, :102-113 */

/* generate() (src/inference.rs:49-193): " " + prompt.trim() is encoded, the
 * prefill ladder and the B=1 loop run as in l2_generate_greedy; at temperature
 * != 0 the logits come back to the host each step and are scaled, soft-maxed
 * and sampled there as the reference does (:165-172).  `out` receives the token
 * strings of get_token (src/util.rs:116-123) one after the other, each followed
 * by a NUL; *n_tokens how many; *ms the elapsed wall-clock milliseconds.  With
 * print_tokens the strings are also written to stdout. */
int l2_generate(l2_model *m, l2_state *s, const l2_tokenizer *t, const char *prompt, int steps,
                l2_random *rng, float temperature, int print_tokens, char *out, size_t out_cap,
                int *n_tokens, int64_t *ms);

#ifdef __cplusplus
}
#endif
#endif /* LLAMA2_HIP_H */
