#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode tok/s of a random-init Llama-2-7B
(GPTQ 4-bit, group 128, act-order) on one MI355X, with the q4 matvec's HBM
roofline fraction and the CPU restatement of the reference timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the token loop's hot path: one transformer<1> forward
plus the greedy argmax, i.e. one decoded token.  The W warm-up steps are the
prompt positions (forced tokens through the same B=1 loop); the K timed steps
are greedy decode steps with the argmax fed back on the device.  Weights and
KV cache are resident in HBM before the timed region starts.

Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "llama2.rs_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak

# HBM bytes per layer moved by the four q4 launches, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# (each scaled by the reading of the plain copy kernel of known size in the same run):
# the summaries are profiles/q4_matvec_<model>_decode_hbm_counters.txt.
MEASURED_Q4_TRAFFIC_PER_LAYER = {
    "7B": 49226169 + 2 * 18683076 + 24774068 + 234963 + 2 * 125403 + 265887,
}


def q4_bytes(n_in: int, n_out: int, G: int) -> int:
    """Algorithmic bytes of one B=1 QLinear::matvec in the reference's format:
    qweight + qzeros + scales(fp32) + g_index + x + y."""
    groups = -(-n_in // G)
    return n_out * (n_in // 8) * 4 + (n_out // 8) * groups * 4 + n_out * groups * 4 + n_in * 4 + n_in * 4 + n_out * 4


def class_bytes(d) -> dict:
    """Algorithmic bytes per launch of each q4 launch class of the decode step."""
    G = d.group_size
    return {
        "q4_qkv": q4_bytes(d.dim, d.dim, G) + 2 * q4_bytes(d.dim, d.kv_dim, G),
        "q4_wo": q4_bytes(d.dim, d.dim, G),
        "q4_w13": 2 * q4_bytes(d.dim, d.hidden_dim, G),
        "q4_w2": q4_bytes(d.hidden_dim, d.dim, G),
        "classifier": d.vocab_size * d.dim * 4 + d.dim * 4 + d.vocab_size * 4,
    }


def token_bytes(d, pos: int) -> int:
    """Bytes the forward pass must read per decoded token: all weights once,
    norms, one embedding row, the classifier, plus the KV cache up to pos."""
    cb = class_bytes(d)
    per_layer = cb["q4_qkv"] + cb["q4_wo"] + cb["q4_w13"] + cb["q4_w2"] + 2 * d.dim * 4
    kv = 2 * d.n_layers * d.kv_dim * 4 * (pos + 1)
    return d.n_layers * per_layer + cb["classifier"] + d.dim * 4 + d.dim * 4 + kv


MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 matrix peak


def prefill_workload(a, d, m, img, np) -> int:
    """BASELINE config 2: a prompt of --prompt-len random ids prefilled in chunks of --chunk tokens
    through the dequant->fp16 MFMA GEMM path, followed by --steps greedy decode steps."""
    from llama2_rs import _lib
    n, chunk, K = a.prompt_len, a.chunk, a.steps
    rng = np.random.default_rng(a.seed)
    prompt = rng.integers(0, d.vocab_size, size=n).astype(np.int32)
    flops_per_token = 2 * d.n_layers * (2 * d.dim * d.dim + 2 * d.dim * d.kv_dim + 3 * d.dim * d.hidden_dim)

    def run(mode):
        m.set_prefill_mode(mode)
        m.reset()
        m.forward(prompt[:min(chunk, n)], np.arange(min(chunk, n), dtype=np.int32))  # warm-up chunk
        m.reset()
        t0 = time.perf_counter()
        for c0 in range(0, n, chunk):
            c1 = min(c0 + chunk, n)
            toks = np.concatenate([[1], prompt[:c1 - 1]])[c0:c1].astype(np.int32)  # START-shifted, as prefill<A> does
            m.forward(toks, np.arange(c0, c1, dtype=np.int32))
        return time.perf_counter() - t0

    t_mfma = run(_lib.PREFILL_MFMA)
    ids, ms_dec = m.decode_bench(int(prompt[-1]), n, K)
    t_fp32 = run(_lib.PREFILL_FP32) if a.cpu_tokens >= 0 else None
    ids32, _ = m.decode_bench(int(prompt[-1]), n, K)
    same = int(np.sum(np.cumprod(ids == ids32)))
    tok_s = n / t_mfma
    tflops = flops_per_token * tok_s / 1e12
    result = {
        "metric": f"{a.model} q4 prefill tok/s on 1 MI355X", "value": round(tok_s, 1), "unit": "tok/s", "n_gpus": 1,
        "steps": n // chunk, "warmup": 1, "ms_per_step": round(t_mfma * 1e3 / max(1, (n + chunk - 1) // chunk), 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 x f16 -> f32 (MFMA)",
        "data": "synthetic",
        "config": {"workload": f"Llama-2-{a.model} GPTQ 4-bit group {d.group_size} act-order, random-init; {n}-token random "
                               f"prompt prefilled in chunks of {chunk} through the dequant->fp16 MFMA GEMM, then {K} greedy steps",
                   "seed": a.seed},
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None,
                     "flops_per_token": flops_per_token},
        "fp32_path_tok_s": round(n / t_fp32, 1) if t_fp32 else None,
        "decode_after_prefill_tok_s": round(K / (ms_dec * 1e-3), 1),
        "greedy_tokens_same_as_after_fp32_prefill": f"{same}/{K}",
    }
    m.close()
    print(json.dumps(result))
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps = the prompt, forced through the loop (default 16; 32 for 13B, as its config asks)")
    ap.add_argument("--model", default="7B", choices=["7B", "13B", "70B"])
    ap.add_argument("--group", type=int, default=0, help="group size (default: 128, 64 for 70B)")
    ap.add_argument("--kv-prefill", type=int, default=0,
                    help="fill this many cache positions synthetically before the prompt (70B long-context case)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=0, help="decoded tokens of the CPU sample (0 = sized to ~20 s)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--workload", default="decode", choices=["decode", "prefill"],
                    help="prefill: BASELINE config 2 (prompt in chunks through the dequant->fp16 MFMA GEMM, then decode)")
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--chunk", type=int, default=128)
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no sharding, no collectives); "
              f"--gpus {a.gpus} is not supported", file=sys.stderr)
        return 2
    if a.warmup is None:
        a.warmup = 32 if a.model == "13B" else 16
    K, W = a.steps, a.warmup
    if K < 1 or W < 0:
        print("bench.py: --steps must be >= 1 and --warmup >= 0", file=sys.stderr)
        return 2

    import numpy as np
    from llama2_rs import ops

    G = a.group or (64 if a.model == "70B" else 128)
    d = ops.preset(a.model, G)
    max_seq = max(d.seq_len, a.kv_prefill + W + K + 8)
    t0 = time.time()
    img = ops.synth_image(d, a.seed)
    t_synth = time.time() - t0
    t0 = time.time()
    m = ops.Model(img, d, max_seq=max_seq)
    t_upload = time.time() - t0

    if a.workload == "prefill":
        return prefill_workload(a, d, m, img, np)

    rng = np.random.default_rng(a.seed)
    prompt = rng.integers(0, d.vocab_size, size=W).astype(np.int32)
    pos0 = a.kv_prefill
    if pos0:
        m.fill_kv_synthetic(0, pos0, seed=a.seed)

    # plain device copy of known size: the box's copy bandwidth, and the known-size
    # kernel that counter readings are scaled by
    copy_bytes = 1 << 28
    copy_ms = ops.copy_bench(copy_bytes, 8)
    copy_gbs = 2 * copy_bytes * 8 / (copy_ms * 1e-3) / 1e9

    # warm-up: the prompt positions, forced through the B=1 loop
    tok = 1
    for i in range(W):
        m.decode_greedy(tok, pos0 + i)
        tok = int(prompt[i])
    # timed: K greedy steps, argmax fed back on the device
    t0 = time.perf_counter()
    ids, ms_events = m.decode_bench(tok, pos0 + W, K)
    wall_ms = (time.perf_counter() - t0) * 1e3
    tok_s = K / (wall_ms * 1e-3)

    # per-launch event timing of the same loop, for the roofline of the dominant kernel
    n_prof = min(8, K)
    prof = m.decode_profile(int(ids[-1]), pos0 + W + K, n_prof) if pos0 + W + K + n_prof <= max_seq else {}
    cb = class_bytes(d)
    q4_classes = ["q4_qkv", "q4_wo", "q4_w13", "q4_w2"]
    kern = {}
    for c in q4_classes + ["classifier"]:
        if c in prof and prof[c][1] > 0:
            us = prof[c][0] / prof[c][1] * 1e3
            kern[c] = {"us": round(us, 2), "bytes": cb[c], "GBs": round(cb[c] / us / 1e3, 1)}
    roofline = None
    if all(c in kern for c in q4_classes):
        tot_b = sum(cb[c] * prof[c][1] for c in q4_classes)
        tot_ms = sum(prof[c][0] for c in q4_classes)
        achieved = tot_b / (tot_ms * 1e-3) / 1e9
        traffic = MEASURED_Q4_TRAFFIC_PER_LAYER.get(a.model)
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4),
                    # mean HBM bytes per q4 launch (a layer has four), beside the algorithmic mean
                    "traffic": round(traffic / 4) if traffic else None,
                    "algorithmic_bytes_per_launch": round(sum(cb[c] for c in q4_classes) / 4),
                    "kernel": "q4 matvec: the four q4 launches of a layer (q|k|v, wo, w1|w3, w2), durations from "
                              "the dispatches' own start/stop events",
                    "per_launch": kern}

    result = {
        "metric": f"{a.model} q4 decode tok/s on 1 MI355X",
        "value": round(tok_s, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": round(wall_ms / K, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": (f"Llama-2-{a.model} GPTQ 4-bit group {G} act-order, random-init; batch-1 greedy decode of "
                         f"{K} tokens after a {W}-token random prompt"
                         + (f", KV cache pre-filled to {pos0} positions" if pos0 else "")),
            "seed": a.seed, "max_seq": max_seq,
        },
        "event_ms_per_step": round(ms_events / K, 4),
        "bytes_per_token": token_bytes(d, pos0 + W + K // 2),
        "decode_GBs": round(token_bytes(d, pos0 + W + K // 2) * tok_s / 1e9, 1),
        "decode_frac_of_hbm_peak": round(token_bytes(d, pos0 + W + K // 2) * tok_s / 1e9 / HBM_PEAK_GBS, 4),
        "roofline": roofline,
        "copy_GBs": round(copy_gbs, 1),
        "setup_s": {"synth": round(t_synth, 1), "upload": round(t_upload, 1)},
    }

    if not a.no_cpu_baseline:
        from oracle import oracle_lib
        o = oracle_lib.Model(img, d, max_seq=max_seq)
        cores = oracle_lib.num_threads()
        # bounded sample of the same workload: the same prompt, then n_cpu greedy tokens
        n_cpu = a.cpu_tokens
        o.new_state()
        if pos0:
            kc, vc = o.kv_cache()
            for l in range(d.n_layers):
                k, v = m.read_kv(l, 0, pos0)
                kc[l, :pos0] = k
                vc[l, :pos0] = v
        tokc = 1
        t0 = time.perf_counter()
        for i in range(W):
            o.transformer([tokc], [pos0 + i])
            tokc = int(prompt[i])
        t_prompt = time.perf_counter() - t0
        if n_cpu <= 0:
            per_tok = max(t_prompt / max(W, 1), 1e-3) if W else 1.0
            n_cpu = int(max(4, min(K, 20.0 / per_tok - W)))
        cpu_ids = []
        t0 = time.perf_counter()
        for i in range(n_cpu):
            logits = o.transformer([tokc], [pos0 + W + i])
            tokc = oracle_lib.argmax(logits)
            cpu_ids.append(tokc)
        t_dec = time.perf_counter() - t0
        same = int(np.sum(np.cumprod(np.asarray(cpu_ids) == ids[:n_cpu])))
        result["cpu_baseline"] = {
            "value": round(n_cpu / t_dec, 3), "unit": "tok/s", "cores": cores, "kind": "port",
            "sample": (f"C restatement of the reference CPU path (OpenMP over rows/heads, 8-lane AVX2), same weights and "
                       f"prompt: {W} prompt positions then {n_cpu} greedy tokens of the {K}; decode-only timing"),
        }
        result["greedy_tokens_identical_to_cpu"] = f"{same}/{n_cpu}"
        o.close()

    m.close()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
