/*
 * llama2_hip_bench.h -- measurement and synthetic-data hooks of libllama2_hip.so.
 *
 * Not part of the drop-in surface (that is llama2_hip.h): nothing here stands
 * where a function of the reference stands.  The reference has no benchmark
 * harness beyond the tok/s line of src/main.rs:62-65 and loads only exported
 * checkpoints (export.py:25-122); these entry points exist so that a benchmark
 * can time the kernels with inputs resident in device memory and can build a
 * random-init model where no checkpoint can be fetched.  Same conventions as
 * llama2_hip.h (int status, l2_last_error()).
 */
#ifndef LLAMA2_HIP_BENCH_H
#define LLAMA2_HIP_BENCH_H

#include "llama2_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- synthetic data ------------------------------------------------------- */

/* Fill `buf` (l2_weights_bytes(dims) bytes of host memory) with a random-init
 * weights image in the `.bin` layout: uniform nibbles, scales U[0.002,0.02],
 * act-order g_index (stable argsort of a shuffled i/group_size), norm weights,
 * embedding and classifier N(0, 0.02), rms_eps 1e-5.  Deterministic in `seed`.
 * No counterpart in the reference (it only loads exported checkpoints,
 * export.py:25-122); stands in for one where no checkpoint can be fetched. */
int l2_synth_image(const l2_dims *dims, uint64_t seed, void *buf, size_t nbytes);

/* Overwrite cache rows [pos0, pos0+npos) of every layer with a deterministic
 * pattern in (-1, 1) derived from seed: stands in for a long prompt when a
 * benchmark needs a deep cache without paying for its prefill. */
int l2_state_fill_synthetic(l2_state *s, int pos0, int npos, uint64_t seed);

/* ---- timing ---------------------------------------------------------------- */

/* Launch the B=1 matvec of qs[0..n) round-robin `iters` times on device-resident
 * random x in its natural order (no host copies inside the timed region): the
 * whole operator, QLinear::matvec<1> with its act-order permutation of x
 * (src/gptq.rs:99-122), one launch per matvec where the kernel applies the
 * permutation itself (rows of up to 8192 inputs), else a gather and the matvec.
 * Timed with HIP events on the launch stream: *ms_total is the elapsed time of
 * all iters matvecs. */
int l2_qlinear_bench(l2_qlinear **qs, int n, int iters, float *ms_total);

/* The same launches, each carrying its own start/stop events (hipExtLaunchKernel): *ms_sum is the sum of the
 * iters dispatch durations, without the gaps between dispatches. */
int l2_qlinear_bench_dispatch(l2_qlinear **qs, int n, int iters, float *ms_sum);

/* The kernel a B=1 matvec of q runs, named as a profiler prints it.  Launches nothing. */
int l2_qlinear_kernel(l2_qlinear *q, char *out, size_t cap);

/* Decode `n_tokens` greedy steps from (token,pos), the argmax fed back on the
 * device, with HIP events around the whole run on the launch stream; out_ids
 * may be NULL. */
int l2_decode_bench(l2_model *m, l2_state *s, int32_t token, int32_t pos, int n_tokens,
                    int32_t *out_ids, float *ms_total);

/* The same loop with a pair of HIP events around every kernel launch (so it
 * runs slower than l2_decode_bench): per kernel class, the summed event time
 * in ms and the number of launches.  Arrays hold l2_kernel_class_count()
 * entries, named by l2_kernel_class_name(). */
int l2_kernel_class_count(void);
const char *l2_kernel_class_name(int cls);
int l2_decode_profile(l2_model *m, l2_state *s, int32_t token, int32_t pos, int n_tokens,
                      float *ms_by_class, int32_t *launches_by_class);

/* Which kernel each q4 launch class of the decode step runs for this model, as
 * "q4_qkv=<kernel>;q4_wo=<kernel>;q4_w13=<kernel>;q4_w2=<kernel>;" with the names a profiler prints
 * (template arguments included), so that counter readings taken per kernel name can be matched to the
 * launches of a run.  Launches nothing. */
int l2_model_q4_kernels(l2_model *m, char *out, size_t cap);

/* What the B=1 q4 launcher would do for a shape, without a device and without launching: n_mats (1..3) matrices
 * of `in` inputs and out[i] outputs in one launch (pair != 0: a w1|w3 pair with the SiLU gate behind), with
 * (norm != 0) or without an rmsnorm in front.  kernel receives the kernel's name as a profiler prints it;
 * geometry[4] receives {blocks, threads per block, rows per block, dynamic LDS bytes}. */
int l2_q4_plan(int in, const int32_t *out, int n_mats, int group_size, int pair, int norm, char *kernel, size_t cap,
               int32_t *geometry);

/* Plain device-to-device copy of nbytes, iters times: the box's achievable
 * copy bandwidth (bytes moved = 2*nbytes per iteration). */
int l2_copy_bench(size_t nbytes, int iters, float *ms_total);

#ifdef __cplusplus
}
#endif
#endif /* LLAMA2_HIP_BENCH_H */
