"""Structural pins for the oracle's transformer<B> / generate (src/models.rs:178-298,
src/inference.rs:16-193).  The reference holds no checkpoint and no expected
tokens, so the whole loop is 'parity unpinned' by fixtures; what can be fixed
without one is fixed here: an independent fp64 numpy forward on the dequantised
weights, batched prefill == token by token, and the loop's bookkeeping."""
import numpy as np
import pytest

from llama2_rs import checkpoint as ck

TINY = ck.Dims(dim=256, hidden_dim=512, n_layers=2, n_heads=2, n_kv_heads=2, vocab_size=300,
               seq_len=96, group_size=64)
TINY_GQA = ck.Dims(dim=512, hidden_dim=768, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=260,
                   seq_len=80, group_size=128)


def _split_image(img, d, layers=None, names=None, max_rows=None):
    """Walk the image in struct order and return fp64 dense weights (independent of oracle.c).
    With `layers` / `names` only those layers of those tensors are dequantised (big models); the rest is None.
    With `max_rows` a quantised projection of more than 2 * max_rows outputs gives its first and last max_rows
    rows only; w["rows"][name] holds the row numbers."""
    off = [0]
    rows_of = {}

    def take(n, dt, want=True):
        a = img[off[0]:off[0] + n * 4].view(dt) if want else None
        off[0] += n * 4
        return a

    def wanted(name):
        return names is None or name in names

    def qlin(name, n_in, n_out):
        out = []
        g = ck.groups_of(n_in, d.group_size) if d.group_size else 0
        for l in range(d.n_layers):
            want = wanted(name) and (layers is None or l in layers)
            if d.group_size == 0:  # dense Linear (src/model.rs:11-15)
                a = take(n_out * n_in, np.float32, want)
                out.append(a.reshape(n_out, n_in).astype(np.float64) if want else None)
                continue
            qw = take(n_out * n_in // 8, np.int32, want)
            qz = take(n_out // 8 * g, np.int32, want)
            sc = take(n_out * g, np.float32, want)
            gi = take(n_in, np.int32, want)
            if not want:
                out.append(None)
                continue
            qw, qz, sc = qw.reshape(n_out, n_in // 8), qz.reshape(n_out // 8, g), sc.reshape(n_out, g)
            idx = np.arange(n_out)
            if max_rows and n_out > 2 * max_rows:
                assert max_rows % 8 == 0
                idx = np.concatenate([idx[:max_rows], idx[-max_rows:]])
                qw, sc = qw[idx], sc[idx]
                qz = np.concatenate([qz[:max_rows // 8], qz[-(max_rows // 8):]])
            rows_of[name] = idx
            out.append(ck.dequant_bin(qw, qz, sc, gi, d.group_size))
        return out

    def f64(name, n, shape):
        a = take(n, np.float32, wanted(name))
        return a.reshape(shape).astype(np.float64) if a is not None else None

    w = {"eps": float(take(1, np.float32)[0])}
    w["emb"] = f64("emb", d.vocab_size * d.dim, (d.vocab_size, d.dim))
    w["rms_att"] = f64("rms_att", d.n_layers * d.dim, (d.n_layers, d.dim))
    w["wq"], w["wk"], w["wv"], w["wo"] = (qlin("wq", d.dim, d.dim), qlin("wk", d.dim, d.kv_dim),
                                          qlin("wv", d.dim, d.kv_dim), qlin("wo", d.dim, d.dim))
    w["rms_ffn"] = f64("rms_ffn", d.n_layers * d.dim, (d.n_layers, d.dim))
    w["w1"], w["w2"], w["w3"] = (qlin("w1", d.dim, d.hidden_dim), qlin("w2", d.hidden_dim, d.dim),
                                 qlin("w3", d.dim, d.hidden_dim))
    w["rms_final"] = f64("rms_final", d.dim, (d.dim,))
    take(2 * d.seq_len * (d.head_size // 2), np.float32, False)
    w["wcls"] = f64("wcls", d.vocab_size * d.dim, (d.vocab_size, d.dim))
    assert off[0] == img.nbytes
    w["rows"] = rows_of
    return w


def _forward_fp64(w, d, tokens):
    """Plain fp64 decoder over a token sequence; returns logits of the last position."""
    HS, half = d.head_size, d.head_size // 2
    ag = d.attn_groups
    K = [[] for _ in range(d.n_layers)]
    V = [[] for _ in range(d.n_layers)]

    def norm(x, wt):
        return wt * x / np.sqrt(np.mean(x * x) + w["eps"])

    def rope(vec, nh, pos):
        v = vec.reshape(nh, HS).copy()
        ang = pos / (10000.0 ** (2.0 * np.arange(half) / HS))
        c, s = np.cos(ang), np.sin(ang)
        first = v[:, :half] * c - v[:, half:] * s
        second = v[:, half:] * c + first * s        # src/models.rs:112-116
        return np.concatenate([first, second], 1).reshape(-1)

    logits = None
    for pos, tok in enumerate(tokens):
        x = w["emb"][tok].copy()
        for l in range(d.n_layers):
            xb = norm(x, w["rms_att"][l])
            q, k, v = w["wq"][l] @ xb, w["wk"][l] @ xb, w["wv"][l] @ xb
            q, k = rope(q, d.n_heads, pos), rope(k, d.n_kv_heads, pos)
            K[l].append(k.reshape(d.n_kv_heads, HS))
            V[l].append(v.reshape(d.n_kv_heads, HS))
            Kc, Vc = np.stack(K[l]), np.stack(V[l])
            att = np.zeros(d.dim)
            for h in range(d.n_heads):
                a = Kc[:, h // ag] @ q[h * HS:(h + 1) * HS] / np.sqrt(HS)
                a = np.exp(a - a.max())
                a /= a.sum()
                att[h * HS:(h + 1) * HS] = a @ Vc[:, h // ag]
            x = x + w["wo"][l] @ att
            xb = norm(x, w["rms_ffn"][l])
            a, b = w["w1"][l] @ xb, w["w3"][l] @ xb
            x = x + w["w2"][l] @ (a / (1 + np.exp(-a)) * b)
        logits = w["wcls"] @ norm(x, w["rms_final"])
    return logits


DENSE_GQA = ck.Dims(dim=512, hidden_dim=640, n_layers=2, n_heads=4, n_kv_heads=2, vocab_size=260,
                    seq_len=80, group_size=0)  # the build without quantisation (GROUPSIZE 0)


@pytest.mark.parametrize("dims", [TINY, TINY_GQA, DENSE_GQA], ids=["mha_g64", "gqa_g128", "dense_gqa"])
def test_transformer_against_fp64_numpy(oracle, dims):
    img = ck.synth_weights_image(dims, seed=11)
    m = oracle.Model(img, dims)
    toks = [1, 5, 250, 17, 3, 99]
    m.new_state()
    for pos, t in enumerate(toks):
        logits = m.transformer([t], [pos])
    want = _forward_fp64(_split_image(img, dims), dims, toks)
    scale = np.sqrt(np.mean(want ** 2))
    assert np.max(np.abs(logits - want)) / scale < 2e-4
    assert int(np.argmax(want)) == oracle.argmax(logits)
    m.close()


def test_weights_size_check(oracle):
    img = ck.synth_weights_image(TINY, seed=1)
    assert img.nbytes == ck.weights_bytes(TINY)
    with pytest.raises(ValueError):
        oracle.Model(img[:-4], TINY)


def test_struct_sizes_of_the_three_presets():
    # size_of::<QTransformerWeights>() + header, from the #[repr(C)] field list
    # 7B by hand: 2*524288000 (emb, wcls) + 32*(4*8994816 + 2*24145920 + 24173568) + norms/freq/eps/header
    assert ck.checkpoint_bytes(ck.preset("7B", 128)) == 4_520_919_072
    assert round(ck.checkpoint_bytes(ck.preset("13B", 128)) / 1e9, 3) == 8.110
    assert round(ck.checkpoint_bytes(ck.preset("70B", 64)) / 1e9, 3) == 41.167
    # one q_proj of the 7B preset: the byte count quoted for the standalone matvec
    assert ck.qlinear_bytes(4096, 4096, 128) == 8_388_608 + 65_536 + 524_288 + 16_384
    # size_of::<TransformerWeights>() of the 7B build without quantisation (src/model.rs:36-67), by hand:
    # eps + 2 tables of 32000x4096 + 32 layers of (2 norms + 4 x 4096^2 + 3 x 4096x11008) + final norm + freq tables
    dense = 4 + 2 * 32000 * 4096 * 4 + 32 * (2 * 4096 + 4 * 4096 * 4096 + 3 * 4096 * 11008) * 4 + 4096 * 4 \
        + 2 * 2048 * 64 * 4
    assert ck.weights_bytes(ck.preset("7B", 0)) == dense


@pytest.mark.parametrize("n_prompt", [0, 1, 2, 3, 7, 23, 70])
def test_prefill_ladder_equals_token_by_token(oracle, n_prompt):
    """'Should lead to identical results' (src/inference.rs:12-15): the batched
    ladder fills the same cache and yields the same tokens as the B=1 loop."""
    d = TINY
    img = ck.synth_weights_image(d, seed=2)
    rng = np.random.default_rng(n_prompt)
    prompt = rng.integers(0, d.vocab_size, size=n_prompt).astype(np.int32)
    steps = n_prompt + 6
    m = oracle.Model(img, d)
    a = m.generate_greedy(prompt, steps, use_prefill=True)
    ka, va = (c.copy() for c in m.kv_cache())
    b = m.generate_greedy(prompt, steps, use_prefill=False)
    kb, vb = m.kv_cache()
    # B=1 loop writes every iteration's `next`: steps tokens, the prompt forced first
    assert len(b) == steps
    np.testing.assert_array_equal(b[:n_prompt], prompt)
    # the ladder consumed positions silently: ret.len() == steps - start position
    consumed = steps - len(a)
    assert 0 <= consumed < max(n_prompt, 1) and (consumed == 0 or consumed % 2 == 0)
    np.testing.assert_array_equal(a, b[consumed:])
    np.testing.assert_array_equal(ka, kb)
    np.testing.assert_array_equal(va, vb)
    m.close()


def test_ladder_consumes_expected_positions(oracle):
    # strict `pos + A < len`: 70 prompt tokens -> 64, then 4 (66..69 needs pos+4<70 -> 64+4=68<70),
    # then nothing for 2 (68+2<70 is false)
    d = TINY
    img = ck.synth_weights_image(d, seed=2)
    m = oracle.Model(img, d)
    prompt = np.arange(70, dtype=np.int32) % d.vocab_size
    assert len(m.generate_greedy(prompt, 80, True)) == 80 - 68
    m.close()
