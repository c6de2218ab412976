"""GPU parity: every C-ABI compute entry point against the CPU oracle on the same
seeded inputs.  fp32 decode path tolerance: norm-relative 1e-4 on matvec
outputs (max|d| / max(|y_ref|, rms(y_ref))); greedy tokens must be identical."""
import numpy as np
import pytest

from llama2_rs import checkpoint as ck

pytestmark = pytest.mark.gpu

REL_FP32 = 1e-4


def nrel(got, want):
    want = np.asarray(want, np.float64)
    scale = np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)) + 1e-30)
    return float(np.max(np.abs(np.asarray(got, np.float64) - want) / scale))


@pytest.fixture(scope="module")
def ops():
    from llama2_rs import ops as o, _lib
    assert _lib.lib().l2_device_count() >= 1, "no HIP device: the GPU tests cannot run"
    return o


def test_kat_constant_cases(ops):
    # src/gptq_test.rs:40-53 and src/kernel.py:100-103, closed forms
    IN, OUT, G = 4096, 2048, 128
    gi = np.arange(IN, dtype=np.int32)
    q = ops.QLinear(np.full((OUT, IN // 8), 1985229328, np.int32), np.zeros((OUT // 8, IN // G), np.int32),
                    np.full((OUT, IN // G), 10.0, np.float32), gi, G)
    assert np.all(q.matvec(np.full(IN, 10.0, np.float32)) == 1024000.0)
    q.close()
    OUT = 4096
    q = ops.QLinear(np.zeros((OUT, IN // 8), np.int32), np.full((OUT // 8, IN // G), 1985229328, np.int32),
                    np.full((OUT, IN // G), -1.0, np.float32), gi, G)
    y = q.matvec(np.ones(IN, np.float32))
    assert np.array_equal(y, (IN * ((np.arange(OUT) % 8) + 1)).astype(np.float32))
    q.close()


@pytest.mark.parametrize("n_in,n_out,G,B", [
    (4096, 4096, 128, 1),      # BASELINE config 0: Llama-2-7B q_proj, seed 0
    (4096, 11008, 128, 1), (11008, 4096, 128, 1),
    (5120, 5120, 128, 1), (13824, 5120, 128, 2),
    (8192, 1024, 64, 1), (8192, 8192, 64, 1), (28672, 8192, 64, 1),
    (256, 64, 32, 3), (512, 40, 64, 1), (1024, 264, 128, 5),
    (4160, 72, 32, 2), (12320, 40, 32, 1),   # rows of 3 and 7 waves with a ragged last wave
])
def test_qmatvec_vs_oracle(ops, oracle, n_in, n_out, G, B):
    rng = np.random.default_rng(0)
    qw, qz, sc, gi = ck.synth_qlinear(rng, n_in, n_out, G, act_order=True)
    x = rng.standard_normal((B, n_in)).astype(np.float32)
    want = oracle.qmatvec(qw, qz, sc, gi, G, x)
    q = ops.QLinear(qw, qz, sc, gi, G)
    got = q.matvec(x)
    assert got.shape == want.shape
    assert nrel(got, want) < REL_FP32
    # batch columns are the B=1 result, bit for bit, and reruns are bit-stable
    np.testing.assert_array_equal(q.matvec(x[0]), got[0])
    np.testing.assert_array_equal(q.matvec(x), got)
    q.close()


_ALT_FORM_SNIPPET = r"""
import sys, numpy as np
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[2])
from llama2_rs import ops, checkpoint as ck
from oracle import oracle_lib as o
worst = 0.0
for n_in, n_out, G, B in ((4096, 512, 128, 1), (1024, 264, 64, 3), (11008, 256, 128, 1), (512, 40, 32, 2)):
    rng = np.random.default_rng(n_in + n_out)
    qw, qz, sc, gi = ck.synth_qlinear(rng, n_in, n_out, G)
    x = rng.standard_normal((B, n_in)).astype(np.float32)
    want = np.asarray(o.qmatvec(qw, qz, sc, gi, G, x), np.float64)
    q = ops.QLinear(qw, qz, sc, gi, G)
    got = np.asarray(q.matvec(x), np.float64)
    scale = np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)) + 1e-30)
    worst = max(worst, float(np.max(np.abs(got - want) / scale)))
    q.close()
print("WORST", worst)
"""


@pytest.mark.parametrize("form", ["tile", "idot"])
def test_selectable_kernel_forms(form):
    """L2_Q4_IMPL=tile|idot select other forms of the q4 kernel when the library is loaded; each runs
    the same parity check in a process of its own."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, L2_Q4_IMPL=form)
    r = subprocess.run([sys.executable, "-c", _ALT_FORM_SNIPPET, os.path.join(root, "llama2.rs_amd"), root],
                       capture_output=True, text=True, env=env, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    worst = float(r.stdout.strip().split("WORST")[-1])
    assert worst < REL_FP32, (form, worst)


def test_qmatvec_unit_vectors_and_linearity(ops):
    rng = np.random.default_rng(5)
    n_in, n_out, G = 512, 96, 64
    qw, qz, sc, gi = ck.synth_qlinear(rng, n_in, n_out, G)
    W = ck.dequant_bin(qw, qz, sc, gi, G)
    q = ops.QLinear(qw, qz, sc, gi, G)
    E = np.zeros((6, n_in), np.float32)
    cols = [0, 7, 8, 63, 64, 511]
    for r, j in enumerate(cols):
        E[r, j] = 1.0
    Y = q.matvec(E)
    for r, j in enumerate(cols):
        np.testing.assert_allclose(Y[r], W[:, j], rtol=1e-6, atol=1e-7)
    assert not ops.QLinear(qw, qz, np.zeros_like(sc), gi, G).matvec(E[0] + 3).any()
    q.close()


def test_bad_arguments_fail_cleanly(ops):
    from llama2_rs._lib import L2Error
    rng = np.random.default_rng(1)
    qw, qz, sc, gi = ck.synth_qlinear(rng, 256, 64, 32)
    bad = gi.copy()
    bad[3] = bad[4]
    with pytest.raises(L2Error):
        ops.QLinear(qw, qz, sc, bad, 32)          # g_index not a permutation
    with pytest.raises((L2Error, ValueError)):
        ops.QLinear(qw, qz, sc, gi, 48)           # group size
    q = ops.QLinear(qw, qz, sc, gi, 32)
    with pytest.raises(ValueError):
        q.matvec(np.zeros(255, np.float32))
    q.close()


TINY = ck.Dims(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=300,
               seq_len=96, group_size=64)
TINY_GQA = ck.Dims(dim=512, hidden_dim=768, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=260,
                   seq_len=80, group_size=128)
MID = ck.Dims(dim=1024, hidden_dim=2816, n_layers=3, n_heads=8, n_kv_heads=2, vocab_size=2000,
              seq_len=256, group_size=32)
# rows of 3 waves (144 chunks, the last wave ragged) behind an rmsnorm, as q|k|v and w1|w3 of the 13B preset
WIDE = ck.Dims(dim=4608, hidden_dim=1536, n_layers=2, n_heads=36, n_kv_heads=9, vocab_size=300,
               seq_len=64, group_size=128)


@pytest.mark.parametrize("dims", [TINY, TINY_GQA, MID, WIDE], ids=["mha_g64", "gqa_g128", "gqa_g32", "wide_g128"])
def test_forward_logits_and_cache_vs_oracle(ops, oracle, dims, tmp_path):
    img = ck.synth_weights_image(dims, seed=11)
    path = str(tmp_path / "m.bin")
    ck.write_checkpoint(path, dims, img)
    m = ops.Model(path, dims)                      # through the mmap loader
    cfg = m.config
    assert (cfg.dim, cfg.n_layers, cfg.vocab_size, cfg.shared_weight) == (dims.dim, dims.n_layers, dims.vocab_size, 0)
    o = oracle.Model(img, dims)
    o.new_state()
    toks = [1, 5, 250, 17, 3, 99, 42]
    for pos, t in enumerate(toks):
        want = o.transformer([t], [pos])
        got = m.forward([t], [pos])
        assert nrel(got, want) < REL_FP32, pos
        assert int(np.argmax(got)) == oracle.argmax(want)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, len(toks))
        assert nrel(k, ko[l, :len(toks)]) < REL_FP32
        assert nrel(v, vo[l, :len(toks)]) < REL_FP32
    # a batched call (B=4) continues the same sequence: cache rows equal the oracle's
    nxt = [7, 8, 9, 10]
    poss = list(range(len(toks), len(toks) + 4))
    assert m.forward(nxt, poss) is None
    o.transformer(nxt, poss)
    k, v = m.read_kv(dims.n_layers - 1, len(toks), 4)
    assert nrel(k, ko[-1, len(toks):len(toks) + 4]) < REL_FP32
    m.close()
    o.close()


@pytest.mark.parametrize("n_heads,n_kv,ctx", [(2, 2, 300), (8, 2, 257), (8, 1, 1000), (4, 2, 4300)],
                         ids=["mha_5splits", "gqa4_first_split", "gqa8_16splits", "gqa2_deep"])
def test_decode_attention_long_context(ops, oracle, n_heads, n_kv, ctx):
    """Decode steps behind a long cache: the timesteps are cut across blocks and merged.  The cache rows
    are synthetic (written on the device, copied into the oracle's cache), so no long prompt is needed."""
    dims = ck.Dims(dim=128 * n_heads, hidden_dim=512, n_layers=2, n_heads=n_heads, n_kv_heads=n_kv,
                   vocab_size=300, seq_len=ctx + 8, group_size=128)
    img = ck.synth_weights_image(dims, seed=7)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    o.new_state()
    m.fill_kv_synthetic(0, ctx, seed=3)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, ctx)
        ko[l, :ctx] = k
        vo[l, :ctx] = v
    tok = 11
    for pos in range(ctx, ctx + 3):
        want = o.transformer([tok], [pos])
        got = m.forward([tok], [pos])
        assert nrel(got, want) < REL_FP32, pos
        tok = oracle.argmax(want)
        assert int(np.argmax(got)) == tok
    # the rows written behind the synthetic ones
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, ctx, 3)
        assert nrel(k, ko[l, ctx:ctx + 3]) < REL_FP32
        assert nrel(v, vo[l, ctx:ctx + 3]) < REL_FP32
    m.close()
    o.close()


_VALU_ATTN_SNIPPET = r"""
import sys, numpy as np
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[2])
from llama2_rs import ops, checkpoint as ck
from oracle import oracle_lib as oracle
worst = 0.0
for n_heads, n_kv, ctx in ((8, 2, 257), (8, 1, 1000), (8, 1, 70)):
    dims = ck.Dims(dim=128 * n_heads, hidden_dim=512, n_layers=2, n_heads=n_heads, n_kv_heads=n_kv,
                   vocab_size=300, seq_len=ctx + 8, group_size=128)
    img = ck.synth_weights_image(dims, seed=7)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    o.new_state()
    m.fill_kv_synthetic(0, ctx, seed=3)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, ctx)
        ko[l, :ctx] = k
        vo[l, :ctx] = v
    tok = 11
    for pos in range(ctx, ctx + 3):
        want = np.asarray(o.transformer([tok], [pos]), np.float64)
        got = np.asarray(m.forward([tok], [pos]), np.float64)
        scale = np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)) + 1e-30)
        worst = max(worst, float(np.max(np.abs(got - want) / scale)))
        tok = oracle.argmax(want)
        assert int(np.argmax(got)) == tok
    m.close()
    o.close()
print("WORST", worst)
"""


def test_valu_decode_attention_for_grouped_queries():
    """L2_ATTN_IMPL=valu keeps the vector-ALU decode attention for 4 and 8 query heads per kv head (the matrix-core
    kernel is the default there): the long-context cases again, in a process of its own."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, L2_ATTN_IMPL="valu")
    r = subprocess.run([sys.executable, "-c", _VALU_ATTN_SNIPPET, os.path.join(root, "llama2.rs_amd"), root],
                       capture_output=True, text=True, env=env, timeout=110)
    assert r.returncode == 0, r.stderr[-2000:]
    worst = float(r.stdout.strip().split("WORST")[-1])
    assert worst < REL_FP32, worst


DENSE = ck.Dims(dim=512, hidden_dim=640, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=260,
                seq_len=80, group_size=0)
DENSE_WIDE = ck.Dims(dim=256, hidden_dim=9216, n_layers=1, n_heads=2, n_kv_heads=2, vocab_size=64,
                     seq_len=32, group_size=0)   # w2 takes two passes over a row (in > 8192)


@pytest.mark.parametrize("dims", [DENSE, DENSE_WIDE], ids=["gqa", "long_rows"])
def test_model_without_quantisation(ops, oracle, dims, tmp_path):
    """group_size 0 = the reference's build without the `quantized` feature: TransformerWeights
    (src/model.rs:36-67), every projection a dense Linear; same loop, same oracle."""
    img = ck.synth_weights_image(dims, seed=5)
    path = str(tmp_path / "dense.bin")
    ck.write_checkpoint(path, dims, img)
    m = ops.Model(path, dims)
    o = oracle.Model(img, dims)
    o.new_state()
    toks = [1, 5, 60, 17, 3]
    for pos, t in enumerate(toks):
        want = o.transformer([t], [pos])
        got = m.forward([t], [pos])
        assert nrel(got, want) < REL_FP32, pos
        assert int(np.argmax(got)) == oracle.argmax(want)
    # a chunk of 4 continues the sequence; then the greedy loop with the prefill ladder
    nxt, poss = [7, 8, 9, 10], list(range(len(toks), len(toks) + 4))
    assert m.forward(nxt, poss) is None
    o.transformer(nxt, poss)
    ko, vo = o.kv_cache()
    k, v = m.read_kv(dims.n_layers - 1, 0, len(toks) + 4)
    assert nrel(k, ko[-1, :len(toks) + 4]) < REL_FP32
    assert nrel(v, vo[-1, :len(toks) + 4]) < REL_FP32
    prompt = np.array([3, 9, 33, 12, 50, 7, 21], np.int32)
    got, _ = m.generate_greedy(prompt, 20, use_prefill=True)
    want = o.generate_greedy(prompt, 20, use_prefill=True)
    np.testing.assert_array_equal(got, want)
    # the operator entry point is Linear::matvec<B>
    from llama2_rs import _lib
    import tests.test_oracle_loop as tol
    W = tol._split_image(img, dims)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, dims.hidden_dim)).astype(np.float32)
    assert nrel(m.qmatvec(0, _lib.W2, x), (W["w2"][0] @ x.astype(np.float64).T).T) < REL_FP32
    from llama2_rs._lib import L2Error
    with pytest.raises(L2Error):
        m.set_prefill_mode(1)   # the MFMA prefill path is the quantised model's
    m.close()
    o.close()


@pytest.mark.parametrize("dims", [TINY_GQA, DENSE], ids=["q4_gqa", "dense"])
def test_decode_steps_as_graphs(ops, oracle, dims):
    """Captured decode steps give the tokens of the launched ones: replays are interleaved with eager
    forward passes, host synchronisation, a reset and a second loop with another prompt length."""
    img = ck.synth_weights_image(dims, seed=4)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    m.set_step_graph(True)
    for n_prompt, steps in ((6, 30), (0, 12), (17, 40)):
        prompt = np.random.default_rng(n_prompt).integers(0, dims.vocab_size, size=n_prompt).astype(np.int32)
        got, _ = m.generate_greedy(prompt, steps, use_prefill=False)
        want = o.generate_greedy(prompt, steps, use_prefill=False)
        np.testing.assert_array_equal(got, want)
        # eager work between loops: a forward pass with logits, then single replayed steps
        m.reset()
        o.new_state()
        logits = m.forward([1], [0])
        assert nrel(logits, o.transformer([1], [0])) < REL_FP32
        tok = 1
        for pos in range(5):
            nxt = m.decode_greedy(tok, pos)
            ref = oracle.argmax(o.transformer([tok], [pos]))
            assert nxt == ref, pos
            tok = nxt
    m.set_step_graph(False)
    got2, _ = m.generate_greedy(prompt, steps, use_prefill=True)
    np.testing.assert_array_equal(got2, o.generate_greedy(prompt, steps, use_prefill=True))
    m.close()
    o.close()


def test_kv_snapshot_restore(ops):
    """read_kv / write_kv: a cache restored into a fresh state continues with the same tokens."""
    dims = TINY_GQA
    img = ck.synth_weights_image(dims, seed=9)
    m = ops.Model(img, dims)
    prompt = np.array([4, 9, 200, 31, 7, 7, 100], np.int32)
    full, _ = m.generate_greedy(prompt, 24, use_prefill=False)
    # replay the first 12 positions, snapshot, restore into another model's state, continue from there
    m.reset()
    tok = 1
    for pos in range(12):
        nxt = m.decode_greedy(tok, pos)
        tok = int(prompt[pos]) if pos < len(prompt) else nxt
    snap = [m.read_kv(l, 0, 12) for l in range(dims.n_layers)]
    m2 = ops.Model(img, dims)
    for l, (k, v) in enumerate(snap):
        m2.write_kv(l, 0, k, v)
    out = []
    for pos in range(12, 24):
        tok = m2.decode_greedy(tok, pos)
        out.append(tok)
    np.testing.assert_array_equal(out, full[12:24])
    from llama2_rs._lib import L2Error
    with pytest.raises(L2Error):
        m2.write_kv(0, dims.seq_len - 1, snap[0][0][:2], snap[0][1][:2])
    m.close()
    m2.close()


def test_model_operator_entry_points(ops, oracle):
    dims = TINY_GQA
    img = ck.synth_weights_image(dims, seed=3)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    rng = np.random.default_rng(2)
    from llama2_rs import _lib
    x = rng.standard_normal((2, dims.dim)).astype(np.float32)
    h = rng.standard_normal(dims.hidden_dim).astype(np.float32)
    # the oracle's view of the same projections, through the struct walk of its own loader
    import tests.test_oracle_loop as tol
    W = tol._split_image(img, dims)
    for proj, name, xin in ((_lib.WQ, "wq", x), (_lib.WK, "wk", x), (_lib.WO, "wo", x), (_lib.W1, "w1", x),
                            (_lib.W2, "w2", h), (_lib.W3, "w3", x)):
        got = m.qmatvec(1, proj, xin)
        want = (W[name][1] @ np.asarray(xin, np.float64).T).T
        assert nrel(got, want) < REL_FP32, name
    fin = rng.standard_normal(dims.dim).astype(np.float32)
    assert nrel(m.classifier(fin), W["wcls"] @ fin.astype(np.float64)) < REL_FP32
    m.close()
    o.close()


@pytest.mark.parametrize("dims,n_prompt,prefill", [(TINY, 0, True), (TINY, 5, False), (TINY, 23, True),
                                                    (TINY_GQA, 70, True), (MID, 9, True)])
def test_generate_greedy_tokens_identical(ops, oracle, dims, n_prompt, prefill):
    img = ck.synth_weights_image(dims, seed=2)
    rng = np.random.default_rng(n_prompt)
    prompt = rng.integers(0, dims.vocab_size, size=n_prompt).astype(np.int32)
    steps = min(n_prompt + 8, dims.seq_len)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    got, ms = m.generate_greedy(prompt, steps, use_prefill=prefill)
    want = o.generate_greedy(prompt, steps, use_prefill=prefill)
    np.testing.assert_array_equal(got, want)
    assert ms >= 0
    # one-step entry point agrees with the loop
    m.reset()
    tok, outs = 1, []
    for pos in range(min(4, steps)):
        nxt = m.decode_greedy(tok, pos)
        tok = int(prompt[pos]) if pos < n_prompt else nxt
        outs.append(tok)
    np.testing.assert_array_equal(outs, o.generate_greedy(prompt, min(4, steps), use_prefill=False))
    m.close()
    o.close()


def test_argmax_last_index_on_ties(ops):
    # a classifier with duplicated rows produces exact ties; the last index must win
    dims = TINY
    img = ck.synth_weights_image(dims, seed=4).copy()
    wcls = img[-dims.vocab_size * dims.dim * 4:].view(np.float32).reshape(dims.vocab_size, dims.dim)
    wcls[:] = 0
    wcls[7] = 1.0
    wcls[123] = 1.0
    wcls[250] = 1.0
    m = ops.Model(img, dims)
    logits = m.forward([1], [0])
    assert logits[7] == logits[123] == logits[250]
    m.reset()
    nxt = m.decode_greedy(1, 0)
    assert nxt == (250 if logits[250] > 0 else dims.vocab_size - 1)
    m.close()


def test_range_errors(ops):
    from llama2_rs._lib import L2Error
    m = ops.Model(ck.synth_weights_image(TINY, seed=4), TINY)
    with pytest.raises(L2Error):
        m.forward([TINY.vocab_size], [0])
    with pytest.raises(L2Error):
        m.forward([1], [TINY.seq_len])
    with pytest.raises(L2Error):
        ops.Model(ck.synth_weights_image(TINY, seed=4)[:-4], TINY)
    # A prompt whose prefill ladder would run past the cache is refused before anything is launched (the
    # reference panics on its [SEQ_LEN] arrays), whatever `steps` says; the model is usable afterwards.
    long_prompt = np.arange(2 * TINY.seq_len + 40, dtype=np.int32) % TINY.vocab_size
    with pytest.raises(L2Error):
        m.generate_greedy(long_prompt, 10, use_prefill=True)
    with pytest.raises(L2Error):
        m.generate_greedy(long_prompt[:TINY.seq_len + 3], TINY.seq_len, use_prefill=True)
    ok, _ = m.generate_greedy(long_prompt[:TINY.seq_len], TINY.seq_len, use_prefill=True)
    assert len(ok) == TINY.seq_len - 94 and np.array_equal(ok, long_prompt[94:TINY.seq_len])
    m.close()


def test_text_generate_api(ops, oracle, tmp_path):
    """The pyO3-shaped surface: LlamaModel / Tokenizer / Random / generate
    (python/llama2_rs/llama2_rs_pylib.pyi, tests/test_model_can_run.py of the reference)."""
    import os
    import llama2_rs
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    dims = ck.Dims(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=32000,
                   seq_len=128, group_size=64)
    img = ck.synth_weights_image(dims, seed=21)
    path = str(tmp_path / "tiny32k.bin")
    ck.write_checkpoint(path, dims, img)
    model = llama2_rs.LlamaModel(path, False, dims=dims)
    tokenizer = llama2_rs.Tokenizer(os.path.join(gold, "tokenizer.bin"))
    random = llama2_rs.Random()
    prompt = "Tell me zero-cost abstractions in Rust "
    ms, toks = llama2_rs.generate(model, tokenizer, prompt, 30, random, 0.0)
    assert isinstance(ms, int) and isinstance(toks, list)
    # the same ids as the oracle's loop on the encoded prompt, rendered by get_token
    ids = tokenizer.bpe_encode(" " + prompt.strip())
    o = oracle.Model(img, dims)
    want = o.generate_greedy(ids, 30, use_prefill=True)
    assert len(toks) == len(want)
    first = 30 - len(want)
    prev = 1 if first == 0 else ids[first - 1]
    for got, nxt in zip(toks, want):
        piece = tokenizer.token(int(nxt))[0]
        if prev == 1 and piece.startswith(" "):
            piece = piece[1:]
        assert got == piece
        prev = int(nxt)
    # temperature sampling (src/inference.rs:165-172, src/util.rs:71-113) restated on the ORACLE's logits:
    # divide by the temperature, or_softmax, xorshift* and the CDF walk in Python integers / float32
    def sampled(seed, temperature, steps):
        state = [seed]

        def rnd():
            x = state[0]
            x ^= x >> 12
            x ^= (x << 25) & 0xFFFFFFFFFFFFFFFF
            x ^= x >> 27
            state[0] = x
            return np.float32(((x * 0x2545F4914F6CDD1D & 0xFFFFFFFFFFFFFFFF) >> 32 >> 8)) / np.float32(16777216.0)
        o.new_state()
        pos = 0
        for A in (64, 32, 16, 8, 4, 2):
            while pos + A < len(ids):
                o.transformer([1 if p == 0 else ids[p - 1] for p in range(pos, pos + A)], list(range(pos, pos + A)))
                pos += A
        token = 1 if pos == 0 else ids[pos - 1]
        first, out = token, []
        while pos < steps:
            logits = o.transformer([token], [pos])
            if pos < len(ids):
                nxt = ids[pos]
            else:
                p = oracle.softmax(logits / np.float32(temperature))
                cdf = np.cumsum(p, dtype=np.float32)      # a running float32 sum, as the loop of :106-111
                hit = np.nonzero(rnd() < cdf)[0]
                nxt = int(hit[0]) if hit.size else len(p) - 1
            out.append(nxt)
            token = nxt
            pos += 1
        return first, out

    def strings(first, nxts):
        prev, res = first, []
        for nxt in nxts:
            piece = tokenizer.token(int(nxt))[0]
            res.append(piece[1:] if prev == 1 and piece.startswith(" ") else piece)
            prev = int(nxt)
        return res
    for seed, temp in ((7, 0.8), (8, 0.8), (123456789, 1.5)):
        got = llama2_rs.generate(model, tokenizer, prompt, 24, llama2_rs.Random(seed), temp)[1]
        assert got == strings(*sampled(seed, temp, 24)), (seed, temp)
    model.close()
    o.close()


def test_generate_prints_tokens_as_the_reference_does(ops, oracle, tmp_path, capfd):
    """print_tokens: the prompt tokens of the prefill ladder (src/inference.rs:36-40), the first token
    (:134-137) and every token of the loop (:180-182) go to stdout, whether greedy or sampled; a prompt
    wrapped in Unicode white space is trimmed as str::trim does (:63)."""
    import os
    import llama2_rs
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    dims = ck.Dims(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=32000,
                   seq_len=128, group_size=64)
    img = ck.synth_weights_image(dims, seed=21)
    path = str(tmp_path / "tiny32k.bin")
    ck.write_checkpoint(path, dims, img)
    model = llama2_rs.LlamaModel(path, False, dims=dims)
    tokenizer = llama2_rs.Tokenizer(os.path.join(gold, "tokenizer.bin"))
    prompt = "Tell me zero-cost abstractions in Rust, and why they matter for a tokenizer that is written in it"
    ids = tokenizer.bpe_encode(" " + prompt)
    assert len(ids) > 18          # the ladder takes chunks of 16 and 2 or so

    def text(tok, nxt):
        piece = tokenizer.token(int(nxt))[0]
        return piece[1:] if tok == 1 and piece.startswith(" ") else piece
    for steps in (40, 6):         # 6: the ladder alone runs past `steps`, the loop returns nothing
        capfd.readouterr()
        quiet = llama2_rs.generate(model, tokenizer, prompt, steps, llama2_rs.Random(1), 0.0)[1]
        assert capfd.readouterr().out == ""
        loud = llama2_rs.generate(model, tokenizer, "\u00a0\u2003 " + prompt + "\u3000\n", steps, llama2_rs.Random(1), 0.0, True)[1]
        printed = capfd.readouterr().out
        assert loud == quiet
        pos, want = 0, ""
        for A in (64, 32, 16, 8, 4, 2):
            while pos + A < len(ids):
                for p in range(pos, pos + A):
                    t = 1 if p == 0 else ids[p - 1]
                    want += text(t, t)
                pos += A
        first = 1 if pos == 0 else ids[pos - 1]
        want += text(first, first) + "".join(quiet)
        assert printed == want
        assert len(quiet) == max(0, steps - pos)
    model.close()


REL_MFMA = 2e-3   # fp16 tiles into MFMA, fp32 accumulate


@pytest.mark.parametrize("n_heads,n_kv,ctx,B,G", [(2, 2, 300, 37, 128), (8, 2, 700, 64, 128), (8, 1, 95, 13, 128),
                                                   (4, 4, 1029, 130, 128), (8, 1, 600, 70, 64), (16, 2, 300, 128, 64)],
                         ids=["mha", "gqa4_two_tiles_per_wave", "gqa8_short", "mha_deep_ragged", "gqa8_g64",
                              "gqa8_g64_full_chunk"])
def test_mfma_prefill_chunk_behind_long_cache(ops, oracle, n_heads, n_kv, ctx, B, G):
    """A prefill chunk in the matrix-core mode behind a long synthetic cache: its attention runs over
    many key tiles per wave, chunk sizes and positions that are not multiples of a tile, 1-8 query heads per
    kv head.  Checked through what depends on it: the cache rows of the second layer and the next logits."""
    from llama2_rs import _lib
    dims = ck.Dims(dim=128 * n_heads, hidden_dim=512, n_layers=2, n_heads=n_heads, n_kv_heads=n_kv,
                   vocab_size=300, seq_len=ctx + B + 8, group_size=G)
    img = ck.synth_weights_image(dims, seed=9)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    m.set_prefill_mode(_lib.PREFILL_MFMA)
    o.new_state()
    m.fill_kv_synthetic(0, ctx, seed=4)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, ctx)
        ko[l, :ctx] = k
        vo[l, :ctx] = v
    rng = np.random.default_rng(B)
    toks = rng.integers(0, dims.vocab_size, size=B).astype(np.int32)
    poss = np.arange(ctx, ctx + B, dtype=np.int32)
    m.forward(toks, poss)
    o.transformer(toks, poss)
    k, v = m.read_kv(1, ctx, B)
    # observed: 1-2e-3 on the rows (the fp16 rounding of the projections), 1-3e-5 on the logits
    assert nrel(k, ko[1, ctx:ctx + B]) < 2.5 * REL_MFMA
    assert nrel(v, vo[1, ctx:ctx + B]) < 2.5 * REL_MFMA
    got = m.forward([7], [ctx + B])
    want = o.transformer([7], [ctx + B])
    assert nrel(got, want) < 2e-4      # three times the largest observed (1.4e-5 .. 6.1e-5)
    m.close()
    o.close()


GQA8_G64 = ck.Dims(dim=1024, hidden_dim=1408, n_layers=2, n_heads=8, n_kv_heads=1, vocab_size=500,
                   seq_len=160, group_size=64)   # the 70B head geometry and group size, small


def _with_seq(d, seq_len):
    return ck.Dims(d.dim, d.hidden_dim, d.n_layers, d.n_heads, d.n_kv_heads, d.vocab_size, seq_len, d.group_size)


_SMALL_QG2 = ck.Dims(dim=512, hidden_dim=768, n_layers=3, n_heads=4, n_kv_heads=2, vocab_size=400, seq_len=0,
                     group_size=128)
_WIDE_7B = ck.Dims(dim=4096, hidden_dim=11008, n_layers=2, n_heads=32, n_kv_heads=32, vocab_size=320, seq_len=0,
                   group_size=128)   # the 7B widths (BASELINE config 2 runs through this path), two layers


@pytest.mark.parametrize("mode", ["mfma", "fp32"])
@pytest.mark.parametrize("geom,n,chunk", [
    (_SMALL_QG2, 512, 128), (_SMALL_QG2, 300, 128), (_SMALL_QG2, 257, 64), (_SMALL_QG2, 40, 64), (_SMALL_QG2, 9, 2),
    (GQA8_G64, 300, 128), (MID, 300, 128), (_WIDE_7B, 300, 128),
    (_SMALL_QG2, 700, 256), (GQA8_G64, 600, 256), (_WIDE_7B, 600, 256)],
    ids=["four_chunks", "short_last_chunk", "one_token_left", "one_short_chunk", "chunks_of_2",
         "gqa8_g64_300_by_128", "qg4_g32_300_by_128", "7b_wide_300_by_128",
         "three_chunks_of_256", "gqa8_g64_600_by_256", "7b_wide_600_by_256"])
def test_prefill_chunks_equals_chunk_by_chunk(ops, geom, n, chunk, mode):
    """prefill<A> over a whole prompt (src/inference.rs:16-40) through l2_prefill_chunks, whose chunks overlap on
    two streams in the matrix-core mode, against the same chunks given to transformer<B> one by one: every cache
    row of every layer and the logits that follow, bit for bit (the kernels and their operands are the same).
    Geometries: 2, 4 and 8 query heads per kv head, groups of 32, 64 and 128, and the 7B widths; chunks of 256
    take the GEMM's 128-token wave tiles."""
    from llama2_rs import _lib
    from llama2_rs._lib import L2Error
    if geom is _WIDE_7B and mode == "fp32":
        pytest.skip("the fp32 mode runs on one stream: covered by the small geometries")
    dims = _with_seq(geom, n + 8)
    img = ops.synth_image(dims, 11) if geom is _WIDE_7B else ck.synth_weights_image(dims, seed=11)
    m = ops.Model(img, dims)
    m.set_prefill_mode(_lib.PREFILL_MFMA if mode == "mfma" else _lib.PREFILL_FP32)
    rng = np.random.default_rng(n)
    toks = rng.integers(0, dims.vocab_size, size=n).astype(np.int32)

    def rows_and_logits():
        rows = [m.read_kv(l, 0, n) for l in range(dims.n_layers)]
        return rows, m.forward([5], [n])

    for rep in range(2):    # the second pass reuses both sets of buffers and the events
        m.reset()
        for c0 in range(0, n, chunk):
            c1 = min(c0 + chunk, n)
            m.forward(toks[c0:c1], np.arange(c0, c1, dtype=np.int32))
        want_rows, want_logits = rows_and_logits()
        m.reset()
        m.prefill_chunks(toks, 0, chunk)
        got_rows, got_logits = rows_and_logits()
        for l in range(dims.n_layers):
            np.testing.assert_array_equal(got_rows[l][0], want_rows[l][0])
            np.testing.assert_array_equal(got_rows[l][1], want_rows[l][1])
        np.testing.assert_array_equal(got_logits, want_logits)
    # arguments: a prompt that does not fit the cache, an id outside the vocabulary
    with pytest.raises(L2Error):
        m.prefill_chunks(toks, 9, chunk)
    bad = toks.copy()
    bad[-1] = dims.vocab_size
    with pytest.raises(L2Error):
        m.prefill_chunks(bad, 0, chunk)
    m.close()


_LANES_SNIPPET = r"""
import sys, numpy as np
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, sys.argv[2])
from llama2_rs import ops, _lib, checkpoint as ck
n, chunk = 700, 128    # six chunks, the last one short: lanes are reused and their events recorded again
dims = ck.Dims(dim=512, hidden_dim=768, n_layers=3, n_heads=4, n_kv_heads=2, vocab_size=400, seq_len=n + 8, group_size=128)
m = ops.Model(ck.synth_weights_image(dims, seed=11), dims)
m.set_prefill_mode(_lib.PREFILL_MFMA)
toks = np.random.default_rng(n).integers(0, dims.vocab_size, size=n).astype(np.int32)
bad = 0
for rep in range(2):
    m.reset()
    for c0 in range(0, n, chunk):
        c1 = min(c0 + chunk, n)
        m.forward(toks[c0:c1], np.arange(c0, c1, dtype=np.int32))
    want = [m.read_kv(l, 0, n) for l in range(dims.n_layers)], m.forward([5], [n])
    m.reset()
    m.prefill_chunks(toks, 0, chunk)
    got = [m.read_kv(l, 0, n) for l in range(dims.n_layers)], m.forward([5], [n])
    for l in range(dims.n_layers):
        bad += int(not np.array_equal(got[0][l][0], want[0][l][0])) + int(not np.array_equal(got[0][l][1], want[0][l][1]))
    bad += int(not np.array_equal(got[1], want[1]))
m.close()
print("BAD", bad)
"""


@pytest.mark.parametrize("lanes", [1, 3, 4])
def test_prefill_chunks_on_other_numbers_of_lanes(lanes):
    """L2_PREFILL_LANES chooses how many chunks of a prompt are in flight when the library is loaded (default 2).
    With three or four lanes a chunk's rows are needed by chunks that never waited for it directly: the event of
    a chunk is recorded behind its own wait, so it stands for every earlier chunk.  Same bit-for-bit comparison
    with the chunks given to transformer<B> one by one, in a process of its own."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, L2_PREFILL_LANES=str(lanes))
    r = subprocess.run([sys.executable, "-c", _LANES_SNIPPET, os.path.join(root, "llama2.rs_amd"), root],
                       capture_output=True, text=True, env=env, timeout=150)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.strip().endswith("BAD 0"), r.stdout[-500:]


LONG_G128 = ck.Dims(dim=512, hidden_dim=768, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=260,
                    seq_len=330, group_size=128)


@pytest.mark.parametrize("dims,B", [(TINY_GQA, 5), (MID, 33), (MID, 128), (TINY, 37), (GQA8_G64, 5), (GQA8_G64, 64),
                                    (GQA8_G64, 130), (LONG_G128, 256), (LONG_G128, 300)],
                         ids=["gqa_g128_b5", "g32_b33", "g32_b128", "mha_g64_b37", "gqa8_g64_b5", "gqa8_g64_b64",
                              "gqa8_g64_b130", "gqa_g128_b256", "gqa_g128_b300"])
def test_mfma_prefill_operator_and_forward(ops, oracle, dims, B):
    """The dequant->fp16->MFMA form of QLinear::matvec<B> and of transformer<B> (B > 1)."""
    from llama2_rs import _lib
    img = ck.synth_weights_image(dims, seed=5)
    m = ops.Model(img, dims)
    o = oracle.Model(img, dims)
    m.set_prefill_mode(_lib.PREFILL_MFMA)
    rng = np.random.default_rng(B)
    import tests.test_oracle_loop as tol
    W = tol._split_image(img, dims)
    x = rng.standard_normal((B, dims.dim)).astype(np.float32)
    hx = rng.standard_normal((B, dims.hidden_dim)).astype(np.float32)
    for proj, name, xin in ((_lib.WQ, "wq", x), (_lib.WK, "wk", x), (_lib.W1, "w1", x), (_lib.W2, "w2", hx)):
        got = m.qmatvec(0, proj, xin)
        want = (W[name][0] @ xin.astype(np.float64).T).T
        assert nrel(got, want) < REL_MFMA, name
        fp32 = ops.Model(img, dims)
        assert nrel(got, fp32.qmatvec(0, proj, xin)) < REL_MFMA
        fp32.close()
    # a chunk of B positions through the whole layer stack: cache rows and the logits that follow
    n = min(B, dims.seq_len - 2)
    toks = rng.integers(0, dims.vocab_size, size=n).astype(np.int32)
    poss = np.arange(n, dtype=np.int32)
    m.reset()
    m.forward(toks, poss)
    o.new_state()
    o.transformer(toks, poss)
    ko, vo = o.kv_cache()
    for l in range(dims.n_layers):
        k, v = m.read_kv(l, 0, n)
        assert nrel(k, ko[l, :n]) < 2.5 * REL_MFMA
        assert nrel(v, vo[l, :n]) < 2.5 * REL_MFMA
    got = m.forward([7], [n])
    want = o.transformer([7], [n])
    # observed 2e-4 .. 2.5e-3: the whole prompt went through fp16 projections, two or three layers deep
    assert nrel(got, want) < 2.5 * REL_MFMA
    m.close()
    o.close()
