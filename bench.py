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

The top level of the JSON line is that run (K and W as given).  Beside it, in
the same process and the same line, "configs" carries the stated workloads at
their stated lengths: the standalone 4096x4096 group-128 matvec over 64 weight
instances, the 7B decode of 256 tokens after a 16-token prompt, the
7B prefill of a 512-token prompt in chunks of 128 through the MFMA path, the
13B decode (32 + 256), and the 70B group-64 decode of 128 tokens behind 4096
cached positions, each with its own roofline object (--configs none skips
them, --configs 1,4 selects).

Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "llama2.rs_amd"))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E peak
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 matrix peak
Q4_CLASSES = ["q4_qkv", "q4_wo", "q4_w13", "q4_w2"]


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


def measured_traffic(model: str, kernels: dict):
    """Mean HBM bytes per q4 launch of a layer from the committed rocprofv3 counter summary
    profiles/q4_matvec_<model>_decode_hbm_counters.txt (FETCH_SIZE + WRITE_SIZE per dispatch, already scaled
    to bytes there), matched by kernel name against the kernels this build launches.  Returns
    (bytes or None, note): None with the reason when the summary is missing or names another build's kernels."""
    path = os.path.join(ROOT, "profiles", f"q4_matvec_{model}_decode_hbm_counters.txt")
    if not os.path.exists(path):
        return None, f"no counter summary profiles/{os.path.basename(path)}"
    table = counter_table(path)
    total = 0
    for cls in Q4_CLASSES:
        name = kernels.get(cls, "?") + "(Q4Launch)"
        for section in ("FETCH_SIZE", "WRITE_SIZE"):
            if name not in table[section]:
                return None, (f"profiles/{os.path.basename(path)} holds no {section} reading for {name} ({cls}): "
                              "it was taken with other kernels, take it again")
            total += table[section][name]
    return round(total / len(Q4_CLASSES)), f"profiles/{os.path.basename(path)}"


def counter_table(path: str) -> dict:
    """{"FETCH_SIZE": {kernel: bytes}, "WRITE_SIZE": {...}} of a committed counter summary."""
    table = {"FETCH_SIZE": {}, "WRITE_SIZE": {}}
    section = None
    for line in open(path):
        m = re.match(r"^(FETCH_SIZE|WRITE_SIZE):", line)
        if m:
            section = m.group(1)
            continue
        m = re.match(r"^\s+(\d+)\s+([\d.]+)\s+(\d+)\s+(\S.*)$", line)
        if m and section:
            table[section][m.group(4).strip()] = int(m.group(3))
    return table


def matvec_run(np, ops, n_inst: int, iters: int, reps: int, cpu: bool) -> dict:
    """BASELINE config 0: the standalone GPTQ 4-bit matvec at the 7B q_proj shape (in = out = 4096, group 128,
    act-order, batch 1), launched back to back over n_inst distinct weight instances (more bytes than the 256 MB
    memory-side cache holds, so every launch streams its weights from HBM).  What is timed is the whole operator on
    device-resident x in its natural order, the act-order permutation of x included (one launch: the kernel applies it
    while it stages x).  Instance 0 is config 0 itself (numpy
    default_rng(0): AutoGPTQ-layout tensors through the exporter's transform, x ~ N(0,1)) and is checked against
    the CPU restatement; the others draw the same distributions in the `.bin` layout directly."""
    from llama2_rs import checkpoint as ck
    n_in = n_out = 4096
    G = 128
    groups = n_in // G
    rng0 = np.random.default_rng(0)
    qw0, qz0, sc0, gi0 = ck.synth_qlinear(rng0, n_in, n_out, G, act_order=True)
    x0 = rng0.standard_normal(n_in).astype(np.float32)
    qs = [ops.QLinear(qw0, qz0, sc0, gi0, G)]
    host = [(qw0, qz0, sc0, gi0)]
    for i in range(1, n_inst):
        rng = np.random.default_rng(i)
        qw = rng.integers(0, 1 << 32, size=(n_out, n_in // 8), dtype=np.uint64).astype(np.uint32).view(np.int32)
        qz = rng.integers(0, 1 << 32, size=(n_out // 8, groups), dtype=np.uint64).astype(np.uint32).view(np.int32)
        sc = rng.uniform(0.002, 0.02, size=(n_out, groups)).astype(np.float32)
        gi = np.argsort(rng.permutation(np.arange(n_in) // G), kind="stable").astype(np.int32)
        qs.append(ops.QLinear(qw, qz, sc, gi, G))
        if i < 8:
            host.append((qw, qz, sc, gi))
    nbytes = q4_bytes(n_in, n_out, G)
    y_gpu = qs[0].matvec(x0)
    cadence = sorted(ops.qlinear_bench(qs, iters) / iters * 1e3 for _ in range(reps))  # us per launch, events around the loop
    us_cad = cadence[len(cadence) // 2]
    n_disp = min(iters, 1024)
    us_disp = ops.qlinear_bench_dispatch(qs, n_disp) / n_disp * 1e3               # us per dispatch, its own events
    kernel = ops.qlinear_kernel(qs[0])
    traffic, note = None, "no counter summary profiles/q4_matvec_cfg0_hbm_counters.txt"
    path = os.path.join(ROOT, "profiles", "q4_matvec_cfg0_hbm_counters.txt")
    if os.path.exists(path):
        t = counter_table(path)
        name = kernel + "(Q4Launch)"
        if name in t["FETCH_SIZE"] and name in t["WRITE_SIZE"]:
            traffic, note = t["FETCH_SIZE"][name] + t["WRITE_SIZE"][name], "profiles/q4_matvec_cfg0_hbm_counters.txt"
        else:
            note = f"profiles/q4_matvec_cfg0_hbm_counters.txt holds no reading for {name}: take it again"
    gbs = nbytes / us_cad / 1e3   # HIP events around the timed region on the launch stream, divided by its launches
    out = {
        "workload": (f"standalone GPTQ 4-bit act-order matvec (x in natural order -> y), in {n_in}, out {n_out}, group {G}, batch 1; {n_inst} distinct "
                     f"weight instances ({n_inst * nbytes / 1e6:.0f} MB) launched round-robin, {iters} launches x {reps} runs"),
        "value": round(gbs, 1), "unit": "GB/s", "steps": iters, "warmup": n_inst,
        "ms_per_step": round(us_cad * 1e-3, 6),
        "us_per_dispatch_own_events": round(us_disp, 3),
        "GBs_by_dispatch_events": round(nbytes / us_disp / 1e3, 1),
        "dtype": "f32",
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": note,
                     "algorithmic_bytes_per_launch": nbytes, "kernel": kernel,
                     "duration": "HIP events around the timed launches on their stream, divided by the launches (median of the runs); "
                                 "the mean of the dispatches' own start/stop events beside it"},
    }
    if cpu:
        from oracle import oracle_lib
        cores = oracle_lib.num_threads()
        y_cpu = oracle_lib.qmatvec(qw0, qz0, sc0, gi0, G, x0)
        scale = np.maximum(np.abs(y_cpu), np.sqrt(np.mean(y_cpu.astype(np.float64) ** 2)))
        out["max_rel_err_vs_cpu"] = float(np.max(np.abs(y_gpu - y_cpu) / scale))
        xs = np.random.default_rng(99).standard_normal(n_in).astype(np.float32)
        n_cpu, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < 5.0:
            for h in host:
                oracle_lib.qmatvec(*h, G, xs)
            n_cpu += len(host)
        t_cpu = (time.perf_counter() - t0) / n_cpu
        out["cpu_baseline"] = {"value": round(nbytes / t_cpu / 1e9, 2), "unit": "GB/s", "cores": cores, "kind": "port",
                               "us_per_matvec": round(t_cpu * 1e6, 1),
                               "sample": f"C restatement of QLinear::matvec<1> (OpenMP over rows, 8-lane AVX2) on {len(host)} of "
                                         f"the instances round-robin, {n_cpu} matvecs in about 5 s"}
    for q in qs:
        q.close()
    return out


class Loaded:
    """A random-init model of one preset resident on the GPU, with its host image (the CPU baseline reads it)."""

    def __init__(self, ops, name: str, group: int, layers: int, max_seq: int, seed: int):
        from llama2_rs import checkpoint as ck
        self.ops, self.name, self.seed = ops, name, seed
        d = ops.preset(name, group or (64 if name == "70B" else 128))
        if layers:
            d = ck.Dims(d.dim, d.hidden_dim, layers, d.n_heads, d.n_kv_heads, d.vocab_size, d.seq_len, d.group_size)
        self.d = d
        self.max_seq = max(d.seq_len, max_seq)
        t0 = time.time()
        self.img = ops.synth_image(d, seed)
        self.t_synth = time.time() - t0
        t0 = time.time()
        self.m = ops.Model(self.img, d, max_seq=self.max_seq)
        self.t_upload = time.time() - t0
        self.label = f"Llama-2-{name} GPTQ 4-bit group {d.group_size} act-order, random-init" + \
                     (f", {layers} of its layers" if layers else "")

    def close(self):
        self.m.close()
        self.img = None


def decode_run(np, M: Loaded, W: int, K: int, pos0: int, cpu: bool, cpu_tokens: int) -> dict:
    """W prompt positions forced through the B=1 loop (untimed), then K greedy steps timed; the q4 roofline from
    per-dispatch events of further steps; optionally the CPU restatement on a bounded sample of the same run."""
    m, d = M.m, M.d
    rng = np.random.default_rng(M.seed)
    prompt = rng.integers(0, d.vocab_size, size=W).astype(np.int32)
    m.reset()
    if pos0:
        m.fill_kv_synthetic(0, pos0, seed=M.seed)
    tok = 1
    for i in range(W):
        m.decode_greedy(tok, pos0 + i)
        tok = int(prompt[i])
    t0 = time.perf_counter()
    ids, ms_events = m.decode_bench(tok, pos0 + W, K)
    wall_ms = (time.perf_counter() - t0) * 1e3
    tok_s = K / (wall_ms * 1e-3)

    n_prof = min(8, K)
    prof = m.decode_profile(int(ids[-1]), pos0 + W + K, n_prof) if pos0 + W + K + n_prof <= M.max_seq else {}
    cb = class_bytes(d)
    kern = {}
    for c in Q4_CLASSES + ["classifier", "attention"]:
        if c in prof and prof[c][1] > 0:
            us = prof[c][0] / prof[c][1] * 1e3
            kern[c] = {"us": round(us, 2)}
            if c in cb:
                kern[c].update({"bytes": cb[c], "GBs": round(cb[c] / us / 1e3, 1)})
    roofline = None
    if all(c in kern for c in Q4_CLASSES):
        tot_b = sum(cb[c] * prof[c][1] for c in Q4_CLASSES)
        tot_ms = sum(prof[c][0] for c in Q4_CLASSES)
        achieved = tot_b / (tot_ms * 1e-3) / 1e9
        traffic, note = measured_traffic(M.name, m.q4_kernels())
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBS, 4),
                    # mean HBM bytes per q4 launch (a layer has four), beside the algorithmic mean
                    "traffic": traffic, "traffic_source": note,
                    "algorithmic_bytes_per_launch": round(sum(cb[c] for c in Q4_CLASSES) / 4),
                    "kernel": "q4 matvec: the four q4 launches of a layer (q|k|v, wo, w1|w3, w2), durations from "
                              "the dispatches' own start/stop events",
                    "per_launch": kern}
    mid = pos0 + W + K // 2
    out = {
        "workload": (f"{M.label}; batch-1 greedy decode of {K} tokens after a {W}-token random prompt"
                     + (f", KV cache pre-filled to {pos0} positions" if pos0 else "")),
        "value": round(tok_s, 2), "unit": "tok/s", "steps": K, "warmup": W,
        "ms_per_step": round(wall_ms / K, 4), "event_ms_per_step": round(ms_events / K, 4),
        "bytes_per_token": token_bytes(d, mid),
        "decode_GBs": round(token_bytes(d, mid) * tok_s / 1e9, 1),
        "decode_frac_of_hbm_peak": round(token_bytes(d, mid) * tok_s / 1e9 / HBM_PEAK_GBS, 4),
        "roofline": roofline,
    }
    if cpu:
        from oracle import oracle_lib
        o = oracle_lib.Model(M.img, d, max_seq=M.max_seq)
        cores = oracle_lib.num_threads()
        o.new_state()
        if pos0:
            kc, vc = o.kv_cache()
            for l in range(d.n_layers):
                k, v = m.read_kv(l, 0, pos0)
                kc[l, :pos0] = k
                vc[l, :pos0] = v
        # bounded sample of the same workload: the prompt (at most 4 positions of it timed here, the rest
        # taken from the GPU's cache, which the parity tests hold equal), then n_cpu greedy tokens
        w_cpu = min(W, 4)
        if W > w_cpu:
            kc, vc = o.kv_cache()
            for l in range(d.n_layers):
                k, v = m.read_kv(l, pos0, W - w_cpu)
                kc[l, pos0:pos0 + W - w_cpu] = k
                vc[l, pos0:pos0 + W - w_cpu] = v
        tokc = 1 if W == w_cpu else int(prompt[W - w_cpu - 1])
        t0 = time.perf_counter()
        for i in range(W - w_cpu, W):
            o.transformer([tokc], [pos0 + i])
            tokc = int(prompt[i])
        t_prompt = time.perf_counter() - t0
        n_cpu = cpu_tokens
        if n_cpu <= 0:
            per_tok = max(t_prompt / w_cpu, 1e-3) if w_cpu else 1.0
            n_cpu = int(max(4, min(K, 15.0 / per_tok)))
        cpu_ids = []
        t0 = time.perf_counter()
        for i in range(n_cpu):
            logits = o.transformer([tokc], [pos0 + W + i])
            tokc = oracle_lib.argmax(logits)
            cpu_ids.append(tokc)
        t_dec = time.perf_counter() - t0
        same = int(np.sum(np.cumprod(np.asarray(cpu_ids) == ids[:n_cpu])))
        out["cpu_baseline"] = {
            "value": round(n_cpu / t_dec, 3), "unit": "tok/s", "cores": cores, "kind": "port",
            "sample": (f"C restatement of the reference CPU path (OpenMP over rows/heads, 8-lane AVX2), same weights, "
                       f"prompt and cache: {n_cpu} greedy tokens of the {K}; decode-only timing"),
        }
        out["greedy_tokens_identical_to_cpu"] = f"{same}/{n_cpu}"
        o.close()
    return out


def prefill_run(np, M: Loaded, n: int, chunk: int, K: int, compare_fp32: bool, cpu_tokens: int = 0) -> dict:
    """BASELINE config 2: a prompt of n random ids prefilled in chunks through the dequant->fp16 MFMA GEMM path,
    followed by K greedy decode steps."""
    from llama2_rs import _lib
    m, d = M.m, M.d
    rng = np.random.default_rng(M.seed)
    prompt = rng.integers(0, d.vocab_size, size=n).astype(np.int32)
    flops_per_token = 2 * d.n_layers * (2 * d.dim * d.dim + 2 * d.dim * d.kv_dim + 3 * d.dim * d.hidden_dim)

    reps, spread = 5, []

    def run(mode, chunk=chunk):
        m.set_prefill_mode(mode)
        m.reset()
        m.prefill_chunks(np.concatenate([[1], prompt[:n - 1]]).astype(np.int32), 0, chunk)   # untimed: the whole prompt once
        toks = np.concatenate([[1], prompt[:n - 1]]).astype(np.int32)  # START-shifted, as prefill<A> does
        times = []
        for _ in range(reps):   # the whole prompt each time, from an empty cache; the median is reported
            m.reset()
            t0 = time.perf_counter()
            if os.environ.get("L2_BENCH_PREFILL") == "serial":   # chunk by chunk through transformer<B>
                for c0 in range(0, n, chunk):
                    c1 = min(c0 + chunk, n)
                    m.forward(toks[c0:c1], np.arange(c0, c1, dtype=np.int32))
            else:
                m.prefill_chunks(toks, 0, chunk)
            times.append(time.perf_counter() - t0)
        times.sort()
        spread.append((times[0], times[-1]))
        return times[len(times) // 2]

    out = {}
    if chunk < n:
        # The same prompt as ONE pass of n tokens (the reference takes the longest prefill it was compiled with,
        # src/inference.rs:77-125): reported beside the stated chunking, never instead of it.
        t_one = run(_lib.PREFILL_MFMA, n)
        ids_one, _ = m.decode_bench(int(prompt[-1]), n, K)
        spread_one = spread.pop()
    t_mfma = run(_lib.PREFILL_MFMA)
    ids, ms_dec = m.decode_bench(int(prompt[-1]), n, K)
    if chunk < n:
        tf_one = flops_per_token * (n / t_one) / 1e12
        out["one_pass_of_the_prompt"] = {
            "workload": f"the same {n}-token prompt as a single chunk of {n}", "value": round(n / t_one, 1), "unit": "tok/s",
            "timing": f"median of {reps} (fastest {n / spread_one[0]:.0f}, slowest {n / spread_one[1]:.0f} tok/s)",
            "roofline": {"bound": "mfma", "achieved": round(tf_one, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(tf_one / MFMA_F16_PEAK_TFLOPS, 4)},
            "greedy_tokens_same_as_after_the_chunked_prefill": f"{int(np.sum(np.cumprod(ids == ids_one)))}/{K}"}
    if compare_fp32:
        t_fp32 = run(_lib.PREFILL_FP32)
        ids32, _ = m.decode_bench(int(prompt[-1]), n, K)
        out["fp32_path_tok_s"] = round(n / t_fp32, 1)
        out["greedy_tokens_same_as_after_fp32_prefill"] = f"{int(np.sum(np.cumprod(ids == ids32)))}/{K}"
    if cpu_tokens > 0:
        # the CPU restatement's fp32 prefill of the same prompt (chunks of 64, as the reference's ladder starts) and
        # its B=1 loop: the first cpu_tokens greedy tokens against the GPU's after the MFMA prefill
        from oracle import oracle_lib
        o = oracle_lib.Model(M.img, d, max_seq=M.max_seq)
        o.new_state()
        toks = np.concatenate([[1], prompt[:n - 1]]).astype(np.int32)
        t0 = time.perf_counter()
        for c0 in range(0, n, 64):
            c1 = min(c0 + 64, n)
            o.transformer(toks[c0:c1], np.arange(c0, c1, dtype=np.int32))
        t_cpu_prefill = time.perf_counter() - t0
        tokc, cpu_ids = int(prompt[-1]), []
        for i in range(min(cpu_tokens, K)):
            tokc = oracle_lib.argmax(o.transformer([tokc], [n + i]))
            cpu_ids.append(tokc)
        same = int(np.sum(np.cumprod(np.asarray(cpu_ids) == ids[:len(cpu_ids)])))
        out["greedy_tokens_identical_to_cpu"] = f"{same}/{len(cpu_ids)}"
        out["cpu_baseline"] = {"value": round(n / t_cpu_prefill, 1), "unit": "tok/s", "cores": oracle_lib.num_threads(), "kind": "port",
                               "sample": f"C restatement of the reference CPU path: fp32 prefill of the same {n}-token prompt in "
                                         f"chunks of 64 (prefill<64>), then {len(cpu_ids)} greedy tokens for the comparison"}
        o.close()
    m.set_prefill_mode(_lib.PREFILL_FP32)
    tok_s = n / t_mfma
    tflops = flops_per_token * tok_s / 1e12
    n_chunks = (n + chunk - 1) // chunk
    out.update({
        "workload": f"{M.label}; {n}-token random prompt prefilled in chunks of {chunk} through the dequant->fp16 "
                    f"MFMA GEMM, then {K} greedy steps",
        "value": round(tok_s, 1), "unit": "tok/s", "steps": n_chunks, "warmup": 1,
        "ms_per_step": round(t_mfma * 1e3 / n_chunks, 3), "dtype": "f16 x f16 -> f32 (MFMA)",
        "timing": f"one untimed prefill of the whole prompt, then the median of {reps} (fastest {n / spread[0][0]:.0f}, slowest {n / spread[0][1]:.0f} tok/s)",
        "roofline": {"bound": "mfma", "achieved": round(tflops, 1), "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / MFMA_F16_PEAK_TFLOPS, 4), "traffic": None,
                     "flops_per_token": flops_per_token},
        "decode_after_prefill_tok_s": round(K / (ms_dec * 1e-3), 1),
    })
    return out


def vendor_gemm_run() -> dict:
    """Context for the prefill figures, not a product path: what the vendor library's own fp16 GEMM (hipBLASLt
    behind torch.matmul) reaches on the Llama-2-7B projection shapes with fp16 weights already in HBM, so without
    any dequantisation, at the token counts the prefill uses."""
    import torch
    shapes = {"wq|wk|wv": (12288, 4096), "wo": (4096, 4096), "w1|w3": (22016, 4096), "w2": (4096, 11008)}
    out = {"metric": "vendor fp16 GEMM on the 7B projection shapes (context)", "unit": "us per launch", "rows": {}}
    for tokens in (128, 512):
        total = 0.0
        for name, (n_out, n_in) in shapes.items():
            x = torch.randn(tokens, n_in, device="cuda", dtype=torch.float16)
            ws = [torch.randn(n_out, n_in, device="cuda", dtype=torch.float16) for _ in range(6)]   # 6 copies: not L2-resident
            for w in ws:
                x @ w.t()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                for w in ws:
                    x @ w.t()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / 60
            total += us
            tf = 2.0 * tokens * n_in * n_out / us / 1e6
            out["rows"][f"{name} x {tokens} tokens"] = {"us": round(us, 1), "TFLOP/s": round(tf, 1),
                                                         "frac_of_fp16_peak": round(tf / MFMA_F16_PEAK_TFLOPS, 3)}
        out["rows"][f"one layer x {tokens} tokens"] = {"us": round(total, 1)}
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps = the prompt, forced through the loop (default 16; 32 for 13B, as its config asks)")
    ap.add_argument("--model", default="7B", choices=["7B", "13B", "70B"])
    ap.add_argument("--group", type=int, default=0, help="group size (default: 128, 64 for 70B)")
    ap.add_argument("--layers", type=int, default=0,
                    help="keep only this many layers of the architecture (same kernels and shapes per launch; for "
                         "counter runs and quick checks, never a headline)")
    ap.add_argument("--kv-prefill", type=int, default=0,
                    help="fill this many cache positions synthetically before the prompt (70B long-context case)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-tokens", type=int, default=0, help="decoded tokens of the CPU sample (0 = sized to ~15 s)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--workload", default="decode", choices=["decode", "prefill", "matvec", "vendor-gemm"],
                    help="prefill: BASELINE config 2 alone (prompt in chunks through the dequant->fp16 MFMA GEMM, then decode); "
                         "matvec: BASELINE config 0 alone (the standalone 4096x4096 group-128 matvec); "
                         "vendor-gemm: context only, the vendor library's plain fp16 GEMM (torch.matmul on fp16 weights, no "
                         "dequantisation) on the 7B projection shapes at 128 and 512 tokens")
    ap.add_argument("--instances", type=int, default=64, help="matvec: distinct weight instances cycled through")
    ap.add_argument("--iters", type=int, default=2048, help="matvec: launches per timed run")
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--chunk", type=int, default=128)
    ap.add_argument("--configs", default=None,
                    help="which of the stated workloads to run beside the headline: comma list of 0,1,2,3,4, or none "
                         "(default: all for the plain 7B run, none otherwise)")
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
    plain = a.model == "7B" and not a.layers and not a.group and not a.kv_prefill and a.workload == "decode"
    if a.configs is None:
        a.configs = "0,1,2,3,4" if plain else "none"
    want = set() if a.configs == "none" else {int(c) for c in a.configs.split(",") if c}

    import numpy as np
    from llama2_rs import ops

    if a.workload == "matvec":
        ops.copy_bench(1 << 28, 8)   # the plain copy of known size that counter readings of this run are scaled by
        r = matvec_run(np, ops, a.instances, a.iters, 5, not a.no_cpu_baseline)
        result = {"metric": "GPTQ matvec HBM GB/s (% of peak) on 1 MI355X", "value": r["value"], "unit": "GB/s", "n_gpus": 1,
                  "steps": r["steps"], "warmup": r["warmup"], "ms_per_step": r["ms_per_step"], "higher_is_better": True,
                  "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                  "config": {"workload": r["workload"], "seed": 0}}
        result.update({k: v for k, v in r.items() if k not in result and k != "workload"})
        print(json.dumps(result))
        return 0

    if a.workload == "vendor-gemm":
        print(json.dumps(vendor_gemm_run()))
        return 0

    M = Loaded(ops, a.model, a.group, a.layers, a.kv_prefill + max(W + K, 16 + 256) + 16, a.seed)

    if a.workload == "prefill":
        r = prefill_run(np, M, a.prompt_len, a.chunk, K, not a.no_cpu_baseline)
        result = {"metric": f"{a.model} q4 prefill tok/s on 1 MI355X", "value": r["value"], "unit": "tok/s", "n_gpus": 1,
                  "steps": r["steps"], "warmup": 1, "ms_per_step": r["ms_per_step"], "higher_is_better": True,
                  "scaling": "weak", "vs_baseline": None, "dtype": r["dtype"], "data": "synthetic",
                  "config": {"workload": r["workload"], "seed": a.seed}}
        result.update({k: v for k, v in r.items() if k not in result and k != "workload"})
        M.close()
        print(json.dumps(result))
        return 0

    # plain device copy of known size: the box's copy bandwidth, and the known-size
    # kernel that counter readings are scaled by
    copy_bytes = 1 << 28
    copy_ms = ops.copy_bench(copy_bytes, 8)
    copy_gbs = 2 * copy_bytes * 8 / (copy_ms * 1e-3) / 1e9

    r = decode_run(np, M, W, K, a.kv_prefill, not a.no_cpu_baseline, a.cpu_tokens)
    result = {
        "metric": f"{a.model} q4 decode tok/s on 1 MI355X",
        "value": r["value"], "unit": "tok/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": r["workload"], "seed": a.seed, "max_seq": M.max_seq},
    }
    result.update({k: v for k, v in r.items() if k not in result and k != "workload"})
    result["copy_GBs"] = round(copy_gbs, 1)
    result["setup_s"] = {"synth": round(M.t_synth, 1), "upload": round(M.t_upload, 1)}

    configs = {}
    if want:
        t_all = time.time()
        if 0 in want:   # config 0: the standalone matvec the GB/s half of the metric is quoted on
            configs["cfg0_q4_matvec_4096x4096_g128"] = matvec_run(np, ops, 64, 2048, 5, not a.no_cpu_baseline)
        if 1 in want:   # config 1 at its stated length
            configs["cfg1_7B_decode_16+256"] = decode_run(np, M, 16, 256, 0, False, 0)
        if 2 in want:   # config 2: 512-token prompt in chunks of 128 through the MFMA path, then 64 greedy steps
            configs["cfg2_7B_prefill_512_by_128"] = prefill_run(np, M, 512, 128, 64, False,
                                                                 0 if a.no_cpu_baseline else 16)
        M.close()
        if 3 in want:
            M3 = Loaded(ops, "13B", 0, 0, 32 + 256 + 16, a.seed)
            configs["cfg3_13B_decode_32+256"] = decode_run(np, M3, 32, 256, 0, False, 0)
            M3.close()
        if 4 in want:   # the configuration the 60 % target is stated on
            M4 = Loaded(ops, "70B", 0, 0, 4096 + 4 + 128 + 16, a.seed)
            configs["cfg4_70B_g64_decode_128_behind_4096"] = decode_run(np, M4, 4, 128, 4096, not a.no_cpu_baseline, 8)
            M4.close()
        result["configs"] = configs
        result["configs_wall_s"] = round(time.time() - t_all, 1)
    else:
        M.close()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
