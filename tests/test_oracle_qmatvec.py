"""Pins for the oracle's GPTQ 4-bit matvec (oracle.c:or_qmatvec ~ src/gptq.rs:94-176).

The reference holds no asserted outputs for this function; what it does hold
are two constant-data cases whose answers are closed forms, and the exporter's
transform.  Beyond those the sum itself is pinned by an fp64 brute force on the
UNTRANSFORMED AutoGPTQ tensors, which shares no code with the oracle's packed
layout walk, plus invariants that break under a wrong nibble, sign or index.
"""
import numpy as np
import pytest

from llama2_rs import checkpoint as ck


def test_kat_basic_gptq_test_rs(oracle):
    # src/gptq_test.rs:40-53: qweight words 0x76543210, scales 10, qzeros 0, x 10
    IN, OUT, G = 4096, 2048, 128
    qw = np.full((OUT, IN // 8), 1985229328, np.int32)
    qz = np.zeros((OUT // 8, IN // G), np.int32)
    sc = np.full((OUT, IN // G), 10.0, np.float32)
    gi = np.arange(IN, dtype=np.int32)
    y = oracle.qmatvec(qw, qz, sc, gi, G, np.full(IN, 10.0, np.float32))
    # 10*10*(IN/8)*sum_{k=0..7}(k-1) = 100*512*20
    assert np.all(y == 1024000.0)


def test_kat_kernel_py(oracle):
    # src/kernel.py:100-103 (= src/gptq_test.rs:56-62 defaults): qweight 0, scales -1,
    # qzeros 0x76543210, x 1  ->  y[o] = IN * ((o mod 8) + 1)
    IN, OUT, G = 4096, 4096, 128
    qw = np.zeros((OUT, IN // 8), np.int32)
    qz = np.full((OUT // 8, IN // G), 1985229328, np.int32)
    sc = np.full((OUT, IN // G), -1.0, np.float32)
    gi = np.arange(IN, dtype=np.int32)
    y = oracle.qmatvec(qw, qz, sc, gi, G, np.ones(IN, np.float32))
    assert np.array_equal(y, (IN * ((np.arange(OUT) % 8) + 1)).astype(np.float32))


def test_pack_roundtrip_and_word_order():
    rng = np.random.default_rng(1)
    v = rng.integers(0, 16, size=(64, 24), dtype=np.int32)
    for ax in (0, 1):
        assert np.array_equal(ck.unpack_nibbles(ck.pack_nibbles(v, ax), ax), v)
    # low nibble first: the word the reference's tests use decodes to 0..7
    assert list(ck.unpack_nibbles(np.array([1985229328], np.int32), 0)) == list(range(8))
    # high nibble >= 8 makes the int32 negative; the arithmetic shift + mask still recovers it
    w = ck.pack_nibbles(np.array([1, 2, 3, 4, 5, 6, 7, 15], np.int32))
    assert w[0] < 0 and ck.unpack_nibbles(w)[7] == 15


@pytest.mark.parametrize("n_in,n_out,G,B", [(256, 64, 32, 1), (512, 128, 64, 3), (1024, 256, 128, 2),
                                             (4096, 4096, 128, 1)])
def test_brute_force_autogptq_form(oracle, n_in, n_out, G, B):
    """y[o] = sum_i s[g_idx[i]][o] (q[i][o] - z[g_idx[i]][o] - 1) x[i] in fp64, from the
    AutoGPTQ tensors; the oracle sees only the exporter-transformed arrays."""
    rng = np.random.default_rng(0)
    ag = ck.synth_autogptq_linear(rng, n_in, n_out, G, act_order=True)
    x = rng.standard_normal((B, n_in)).astype(np.float32)
    W = ck.dequant_autogptq(*ag)                      # [IN][OUT] fp64
    want = x.astype(np.float64) @ W
    qw, qz, sc, gi = ck.export_transform(*ag)
    got = oracle.qmatvec(qw, qz, sc, gi, G, x)
    scale = np.maximum(np.abs(want), np.sqrt(np.mean(want ** 2)))
    assert np.max(np.abs(got - want) / scale) < 2e-5
    # the .bin-layout dequant helper tells the same story
    W2 = ck.dequant_bin(qw, qz, sc, gi, G)
    np.testing.assert_allclose(W2.T, W, rtol=0, atol=0)


def test_export_transform_matches_reference_recipe():
    """export.py:51-60 written out literally with numpy broadcasting (no torch):
    extract -> view(IN, OUT)[order] -> shift back -> OR over 8."""
    rng = np.random.default_rng(3)
    n_in, n_out, G = 256, 40, 32
    qweight, qzeros, scales, g_idx = ck.synth_autogptq_linear(rng, n_in, n_out, G)
    offset = np.array([0, 4, 8, 12, 16, 20, 24, 28], np.int32)
    order = np.argsort(g_idx, kind="stable")
    extract = (qweight[:, None, :] >> offset[:, None]) & 15
    extract = extract.reshape(n_in, -1)[order]
    store = extract << np.tile(offset, n_in // 8)[:, None]
    store = store.reshape(n_in // 8, 8, n_out)
    final = np.zeros((n_in // 8, n_out), np.int32)
    for i in range(8):
        final = final | store[:, i]
    qw, qz, sc, gi = ck.export_transform(qweight, qzeros, scales, g_idx)
    assert np.array_equal(qw, final.T)
    assert np.array_equal(qz, qzeros.T) and np.array_equal(sc, scales.T)
    assert np.array_equal(gi, order)
    # sorted rows are grouped: row j of the sorted matrix belongs to group j // G
    assert np.array_equal(g_idx[gi], np.arange(n_in) // G)


def test_invariants(oracle):
    rng = np.random.default_rng(5)
    n_in, n_out, G = 512, 96, 64
    qw, qz, sc, gi = ck.synth_qlinear(rng, n_in, n_out, G)
    W = ck.dequant_bin(qw, qz, sc, gi, G)
    # unit vectors read back single dequantised weights, exactly (one nonzero term)
    for j in (0, 7, 8, 63, 64, 511):
        e = np.zeros(n_in, np.float32)
        e[j] = 1.0
        y = oracle.qmatvec(qw, qz, sc, gi, G, e)
        np.testing.assert_array_equal(y, W[:, j].astype(np.float32))
    # batch columns are independent B=1 calls, bit for bit
    xs = rng.standard_normal((5, n_in)).astype(np.float32)
    yb = oracle.qmatvec(qw, qz, sc, gi, G, xs)
    for b in range(5):
        np.testing.assert_array_equal(yb[b], oracle.qmatvec(qw, qz, sc, gi, G, xs[b]))
    # linearity (to rounding) and zero scales
    a, b = xs[0], xs[1]
    lhs = oracle.qmatvec(qw, qz, sc, gi, G, 2 * a + b)
    rhs = 2 * oracle.qmatvec(qw, qz, sc, gi, G, a) + oracle.qmatvec(qw, qz, sc, gi, G, b)
    assert np.max(np.abs(lhs - rhs)) < 1e-4 * np.max(np.abs(rhs))
    assert not oracle.qmatvec(qw, qz, np.zeros_like(sc), gi, G, a).any()
    # identity permutation == no act-order: permuting g_index and x together changes nothing
    ident = np.arange(n_in, dtype=np.int32)
    inv = np.empty_like(gi)
    inv[gi] = ident
    np.testing.assert_array_equal(oracle.qmatvec(qw, qz, sc, gi, G, a),
                                  oracle.qmatvec(qw, qz, sc, ident, G, a[gi]))


def test_lane_order_is_the_reference_order(oracle):
    """Eight partial sums over j mod 8, rounded mul then rounded add, then an
    ordered horizontal sum (src/gptq.rs:152-168) — restated with numpy scalars."""
    rng = np.random.default_rng(9)
    n_in, n_out, G = 256, 16, 32
    qw, qz, sc, gi = ck.synth_qlinear(rng, n_in, n_out, G)
    x = rng.standard_normal(n_in).astype(np.float32)
    q = ck.unpack_nibbles(qw, axis=1)
    z = ck.unpack_nibbles(qz, axis=0) + 1
    xg = x[gi]
    want = np.zeros(n_out, np.float32)
    for o in range(n_out):
        lanes = np.zeros(8, np.float32)
        for j in range(n_in):
            w = np.float32(sc[o, j // G]) * np.float32(q[o, j] - z[o, j // G])
            lanes[j % 8] = np.float32(lanes[j % 8] + np.float32(w * xg[j]))
        r = np.float32(0.0)
        for k in range(8):
            r = np.float32(r + lanes[k])
        want[o] = r
    np.testing.assert_array_equal(oracle.qmatvec(qw, qz, sc, gi, G, x), want)
