"""GPU parity at the presets' own dimensions (src/constants.rs:7-41): the token loop of
src/inference.rs:141-190 on random-init checkpoints of the 7B and 13B architectures in full, and of the
70B architecture (64 query / 8 kv heads, group 64) with fewer layers behind 4096 cached positions, against
the CPU oracle: the first 64 greedy tokens identical, logits within 1e-4 (fp32 path).  The 7B-wide prefill
of 512 prompt tokens in chunks of 128 goes through the dequant -> fp16 MFMA GEMM path at 2e-3."""
import numpy as np
import pytest

from llama2_rs import checkpoint as ck

pytestmark = pytest.mark.gpu

REL_FP32 = 1e-4
REL_MFMA = 2e-3   # fp16 tiles into MFMA, fp32 accumulate


def nrel(got, want):
    want = np.asarray(want, np.float64)
    scale = np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)) + 1e-30)
    return float(np.max(np.abs(np.asarray(got, np.float64) - want) / scale))


@pytest.fixture(scope="module")
def ops():
    from llama2_rs import ops as o, _lib
    assert _lib.lib().l2_device_count() >= 1, "no HIP device: the GPU tests cannot run"
    return o


def _loop_vs_oracle(ops, oracle, dims, n_prompt, n_greedy):
    """generate() at temperature 0 with the prefill ladder: every token of the loop equals the oracle's,
    and the logits of the three positions that follow agree."""
    img = ops.synth_image(dims, 0)
    rng = np.random.default_rng(0)
    prompt = rng.integers(0, dims.vocab_size, size=n_prompt).astype(np.int32)
    steps = n_prompt + n_greedy
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    got, _ = m.generate_greedy(prompt, steps, use_prefill=True)
    want = o.generate_greedy(prompt, steps, use_prefill=True)
    assert len(want) >= n_greedy
    np.testing.assert_array_equal(got, want)
    tok = int(want[-1])
    for pos in range(steps, steps + 3):
        ref = o.transformer([tok], [pos])
        out = m.forward([tok], [pos])
        assert nrel(out, ref) < REL_FP32, pos
        tok = oracle.argmax(ref)
        assert int(np.argmax(out)) == tok
    k, v = m.read_kv(dims.n_layers - 1, 0, steps + 3)
    ko, vo = o.kv_cache()
    assert nrel(k, ko[-1, :steps + 3]) < REL_FP32
    assert nrel(v, vo[-1, :steps + 3]) < REL_FP32
    m.close()
    o.close()


def test_7b_preset_greedy_64_tokens(ops, oracle):
    """Llama-2-7B architecture in full, group 128, act-order: 16 random prompt ids, then 64 greedy tokens."""
    _loop_vs_oracle(ops, oracle, ops.preset("7B", 128), 16, 64)


def test_13b_preset_greedy_64_tokens(ops, oracle):
    """Llama-2-13B architecture in full, group 128, act-order: 32 random prompt ids, then 64 greedy tokens."""
    _loop_vs_oracle(ops, oracle, ops.preset("13B", 128), 32, 64)


def _reduced(ops, size, group, n_layers, seq_len=None):
    d = ops.preset(size, group)
    return ck.Dims(d.dim, d.hidden_dim, n_layers, d.n_heads, d.n_kv_heads, d.vocab_size, seq_len or d.seq_len,
                   d.group_size)


_W70 = {}   # fp64 dequantised projections of the reduced 70B model's second layer, made once


@pytest.fixture(scope="module")
def reduced_70b(ops, oracle):
    """The 70B architecture (dim 8192, hidden 28672, 64 query / 8 kv heads, group 64) with 2 layers."""
    dims = _reduced(ops, "70B", 64, 2)
    img = ops.synth_image(dims, 0)
    m = ops.Model(img, dims, max_seq=4096 + 64 + 8)
    o = oracle.Model(img, dims, max_seq=4096 + 64 + 8)
    yield dims, img, m, o
    _W70.clear()
    m.close()
    o.close()


def test_70b_reduced_greedy_behind_4096_positions(ops, oracle, reduced_70b):
    """64 greedy tokens behind a cache pre-filled to 4096 positions (synthetic rows, written on the device
    and copied into the oracle's cache): split-KV attention at 8 query heads per kv head, the 8192- and
    28672-wide group-64 launches, the classifier."""
    dims, img, m, o = reduced_70b
    ctx, n = 4096, 64
    m.reset()
    o.new_state()
    m.fill_kv_synthetic(0, ctx, seed=1)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, ctx)
        ko[l, :ctx] = k
        vo[l, :ctx] = v
    # logits at the first three positions through transformer<1>
    tok = 17
    for pos in range(ctx, ctx + 3):
        ref = o.transformer([tok], [pos])
        out = m.forward([tok], [pos])
        assert nrel(out, ref) < REL_FP32, pos
        tok = oracle.argmax(ref)
        assert int(np.argmax(out)) == tok
    # then the loop with the argmax fed back on the device, against the oracle's loop
    ids, _ = m.decode_bench(tok, ctx + 3, n - 3)
    want = []
    for pos in range(ctx + 3, ctx + n):
        tok = oracle.argmax(o.transformer([tok], [pos]))
        want.append(tok)
    np.testing.assert_array_equal(ids, want)
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, ctx, n)
        assert nrel(k, ko[l, ctx:ctx + n]) < REL_FP32
        assert nrel(v, vo[l, ctx:ctx + n]) < REL_FP32


@pytest.mark.parametrize("B", [5, 64, 128, 130, 256, 300])
def test_70b_shapes_mfma_operator_group_64(ops, oracle, reduced_70b, B):
    """The dequant -> fp16 -> MFMA form of QLinear::matvec<B> at group 64 (K steps of 64, one group per
    step) on the 70B projections: rows of 8192 and of 28672 inputs, 8192, 1024 and 28672 outputs."""
    from llama2_rs import _lib
    import tests.test_oracle_loop as tol
    dims, img, m, o = reduced_70b
    m.set_prefill_mode(_lib.PREFILL_MFMA)
    try:
        rng = np.random.default_rng(B)
        x = rng.standard_normal((B, dims.dim)).astype(np.float32)
        hx = rng.standard_normal((B, dims.hidden_dim)).astype(np.float32)
        if not _W70:
            # exact fp64 weights of the first and last 512 output rows of each projection
            _W70.update(tol._split_image(img, dims, layers=[1], names=["wq", "wk", "w1", "w2"], max_rows=512))
        W = _W70
        for proj, name, xin in ((_lib.WQ, "wq", x), (_lib.WK, "wk", x), (_lib.W1, "w1", x), (_lib.W2, "w2", hx)):
            got = m.qmatvec(1, proj, xin)
            rows = W["rows"][name]
            want = (W[name][1] @ xin.astype(np.float64).T).T
            assert nrel(got[:, rows], want) < REL_MFMA, name
            # every output against the fp32 kernels, themselves within 1e-4 of the exact rows
            m.set_prefill_mode(_lib.PREFILL_FP32)
            fp32 = m.qmatvec(1, proj, xin)
            m.set_prefill_mode(_lib.PREFILL_MFMA)
            assert nrel(fp32[:, rows], want) < REL_FP32, name
            assert nrel(got, fp32) < REL_MFMA, name
    finally:
        m.set_prefill_mode(_lib.PREFILL_FP32)


def test_7b_wide_prefill_512_in_chunks_of_128_mfma(ops, oracle):
    """A 7B-wide model (dim 4096, hidden 11008, 32 heads, group 128) with 2 layers: a 512-token prompt prefilled
    in four chunks of 128 through the MFMA path; every cache row and the logits that follow, against the
    oracle's fp32 prefill of the same chunks."""
    from llama2_rs import _lib
    dims = _reduced(ops, "7B", 128, 2)
    img = ops.synth_image(dims, 3)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    m.set_prefill_mode(_lib.PREFILL_MFMA)
    o.new_state()
    rng = np.random.default_rng(2)
    prompt = rng.integers(0, dims.vocab_size, size=512).astype(np.int32)
    toks = np.concatenate([[1], prompt[:-1]]).astype(np.int32)   # START-shifted, as prefill<A> feeds them
    for c0 in range(0, 512, 128):
        poss = np.arange(c0, c0 + 128, dtype=np.int32)
        assert m.forward(toks[c0:c0 + 128], poss) is None
        o.transformer(toks[c0:c0 + 128], poss)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, 512)
        # observed 1-2e-3 on second-layer rows: the fp16 rounding of the projections in front of them
        assert nrel(k, ko[l, :512]) < 2.5 * REL_MFMA, l
        assert nrel(v, vo[l, :512]) < 2.5 * REL_MFMA, l
    got = m.forward([int(prompt[-1])], [512])
    want = o.transformer([int(prompt[-1])], [512])
    assert nrel(got, want) < REL_MFMA
    # and the greedy tokens that follow equal those after the fp32 prefill of the same prompt
    ids_mfma, _ = m.decode_bench(int(np.argmax(got)), 513, 32)
    m.set_prefill_mode(_lib.PREFILL_FP32)
    m.reset()
    for c0 in range(0, 512, 128):
        m.forward(toks[c0:c0 + 128], np.arange(c0, c0 + 128, dtype=np.int32))
    got32 = m.forward([int(prompt[-1])], [512])
    assert nrel(got32, want) < REL_FP32
    ids_fp32, _ = m.decode_bench(int(np.argmax(got32)), 513, 32)
    np.testing.assert_array_equal(ids_mfma, ids_fp32)
    m.close()
    o.close()


def test_7b_full_depth_prefill_512_mfma_then_64_greedy(ops, oracle):
    """BASELINE config 2 at full depth: the Llama-2-7B architecture in full (32 layers), a 512-token random prompt
    through l2_prefill_chunks (dequant -> fp16 -> MFMA; in chunks of 128 on two streams, and again as one pass of
    512 tokens, which takes the 128-token wave tiles of the GEMM), then 64 greedy tokens, against the oracle's fp32
    prefill of the same prompt and its B=1 loop.  The fp16 rounding of every projection input compounds over 32
    layers: the last layer's cache rows are held to 2.5x the operator's 2e-3 (the bound of the shallow whole-stack
    tests), the logits that follow the prompt to 2e-3, and the greedy tokens are compared one by one; the first
    index at which they part, if any, is printed (fp16 rounding may flip a near-tie; a flip within the first 8
    tokens fails the test)."""
    from llama2_rs import _lib
    dims = ops.preset("7B", 128)
    img = ops.synth_image(dims, 0)
    n, n_greedy = 512, 64
    m = ops.Model(img, dims, max_seq=n + n_greedy + 8)
    o = oracle.Model(img, dims, max_seq=n + n_greedy + 8)
    rng = np.random.default_rng(0)
    prompt = rng.integers(0, dims.vocab_size, size=n).astype(np.int32)
    toks = np.concatenate([[1], prompt[:-1]]).astype(np.int32)   # START-shifted, as prefill<A> feeds them
    o.new_state()
    for c0 in range(0, n, 64):   # the reference's ladder starts with chunks of 64 (src/inference.rs:78-85)
        o.transformer(toks[c0:c0 + 64], np.arange(c0, c0 + 64, dtype=np.int32))
    ko, vo = o.kv_cache()
    want = o.transformer([int(prompt[-1])], [n])
    tok = oracle.argmax(want)
    ref = [tok]
    for pos in range(n + 1, n + n_greedy):
        tok = oracle.argmax(o.transformer([tok], [pos]))
        ref.append(tok)
    ref = np.asarray(ref)
    m.set_prefill_mode(_lib.PREFILL_MFMA)
    for chunk in (128, 512):
        m.reset()
        m.prefill_chunks(toks, 0, chunk)
        errs = []
        for l in (0, dims.n_layers // 2, dims.n_layers - 1):
            k, v = m.read_kv(l, 0, n)
            errs.append((l, nrel(k, ko[l, :n]), nrel(v, vo[l, :n])))
        got = m.forward([int(prompt[-1])], [n])
        e_logits = nrel(got, want)
        print(f"\ncfg2 full depth, chunks of {chunk}: cache rows (layer, k, v) "
              f"{[(l, f'{a:.2e}', f'{b:.2e}') for l, a, b in errs]}, logits after the prompt {e_logits:.2e}")
        ids, _ = m.decode_bench(int(np.argmax(got)), n + 1, n_greedy - 1)
        ids = np.concatenate([[int(np.argmax(got))], ids])
        same = int(np.sum(np.cumprod(ids == ref)))
        print(f"cfg2 full depth, chunks of {chunk}: {same}/{n_greedy} greedy tokens identical to the CPU path"
              + ("" if same == n_greedy else f"; they part at index {same}: GPU {ids[same]} CPU {ref[same]}"))
        assert errs[-1][1] < 2.5 * REL_MFMA and errs[-1][2] < 2.5 * REL_MFMA, (chunk, errs)
        assert e_logits < REL_MFMA, (chunk, e_logits)
        assert same >= 8, (chunk, same, ids[:same + 1], ref[:same + 1])
    m.close()
    o.close()


def test_70b_full_depth_greedy_behind_4096_positions(ops, oracle):
    """BASELINE config 4 at full depth: the Llama-2-70B architecture in full (80 layers, 64 query / 8 kv heads,
    group 64, 41 GB of weights), the cache pre-filled to 4096 positions (synthetic rows written on the device and
    copied into the oracle's cache), then greedy tokens through the B=1 loop with the argmax fed back on the device,
    against the oracle's loop: logits of the first position within 1e-4, 16 tokens identical (the CPU path takes
    more than a second per token at this size), the last layer's new cache rows within 1e-4."""
    dims = ops.preset("70B", 64)
    ctx, n = 4096, 16
    img = ops.synth_image(dims, 0)
    m = ops.Model(img, dims, max_seq=ctx + n + 8)
    o = oracle.Model(img, dims, max_seq=ctx + n + 8)
    m.reset()
    o.new_state()
    m.fill_kv_synthetic(0, ctx, seed=1)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, ctx)
        ko[l, :ctx] = k
        vo[l, :ctx] = v
    tok = 17
    ref = o.transformer([tok], [ctx])
    out = m.forward([tok], [ctx])
    assert nrel(out, ref) < REL_FP32
    tok = oracle.argmax(ref)
    assert int(np.argmax(out)) == tok
    ids, _ = m.decode_bench(tok, ctx + 1, n - 1)
    want = []
    for pos in range(ctx + 1, ctx + n):
        tok = oracle.argmax(o.transformer([tok], [pos]))
        want.append(tok)
    np.testing.assert_array_equal(ids, want)
    k, v = m.read_kv(dims.n_layers - 1, ctx, n)
    assert nrel(k, ko[-1, ctx:ctx + n]) < REL_FP32
    assert nrel(v, vo[-1, ctx:ctx + n]) < REL_FP32
    m.close()
    o.close()
