"""Pins for the oracle's per-token blocks (src/models.rs:47-176, src/model.rs:22-31,
src/util.rs:39-46) against what the mathematics fixes: fp64 closed forms, library
routines, and special cases chosen so a dropped term, a wrong sign or a swapped
index fails."""
import numpy as np
import pytest


def test_dense_matvec_is_numpy_dot(oracle):
    rng = np.random.default_rng(0)
    w = rng.standard_normal((37, 129)).astype(np.float32)
    x = rng.standard_normal(129).astype(np.float32)
    y = oracle.dense_matvec(w, x)
    np.testing.assert_allclose(y, w.astype(np.float64) @ x.astype(np.float64), rtol=2e-5, atol=1e-5)
    # a transposed operand would fail this non-square, asymmetric case
    e = np.zeros(129, np.float32)
    e[5] = 1
    np.testing.assert_array_equal(oracle.dense_matvec(w, e), w[:, 5])


def test_rmsnorm_closed_form(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(256).astype(np.float32) * 3
    w = rng.standard_normal(256).astype(np.float32)
    eps = 1e-5
    want = w.astype(np.float64) * x / np.sqrt(np.mean(x.astype(np.float64) ** 2) + eps)
    np.testing.assert_allclose(oracle.rmsnorm(x, w, eps), want, rtol=1e-5, atol=1e-6)
    # eps sits inside the square root, added to the MEAN (not the sum)
    z = np.zeros(16, np.float32)
    z[0] = 4.0  # mean of squares = 1
    got = oracle.rmsnorm(z, np.ones(16, np.float32), 3.0)
    assert abs(got[0] - 4.0 / 2.0) < 1e-6


def test_softmax_invariants(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(100).astype(np.float32) * 5
    p = oracle.softmax(x)
    e = np.exp(x.astype(np.float64) - x.max())
    np.testing.assert_allclose(p, e / e.sum(), rtol=1e-5)
    assert abs(p.sum() - 1) < 1e-5
    np.testing.assert_allclose(oracle.softmax(x + 7.0), p, rtol=1e-4)
    assert oracle.softmax(np.array([1000.0, 1000.0], np.float32)).tolist() == [0.5, 0.5]


def test_silu_gate(oracle):
    rng = np.random.default_rng(3)
    a = rng.standard_normal(64).astype(np.float32) * 4
    b = rng.standard_normal(64).astype(np.float32)
    want = a.astype(np.float64) / (1 + np.exp(-a.astype(np.float64))) * b
    np.testing.assert_allclose(oracle.silu_gate(a, b), want, rtol=1e-5, atol=1e-7)
    # the gate is applied to the FIRST argument only
    assert oracle.silu_gate(np.array([0.0], np.float32), np.array([5.0], np.float32))[0] == 0.0
    assert abs(oracle.silu_gate(np.array([5.0], np.float32), np.array([0.5], np.float32))[0]
               - 5 / (1 + np.exp(-5.0)) * 0.5) < 1e-6


@pytest.mark.parametrize("n_heads,n_kv", [(4, 4), (8, 2)])
def test_rope_in_place_quirk(oracle, n_heads, n_kv):
    """src/models.rs:100-129.  First half of each head is the textbook rotate-half
    rotation; the second half reads the ALREADY ROTATED first half."""
    HS = 128
    rng = np.random.default_rng(4)
    q = rng.standard_normal(n_heads * HS).astype(np.float32)
    k = rng.standard_normal(n_kv * HS).astype(np.float32)
    # pos = 0 is the identity (cos 1, sin 0)
    q0, k0 = oracle.rope(q, k, 0, n_heads, n_kv, HS)
    np.testing.assert_array_equal(q0, q)
    np.testing.assert_array_equal(k0, k)
    pos = 37
    q1, k1 = oracle.rope(q, k, pos, n_heads, n_kv, HS)
    i = np.arange(HS // 2)
    ang = pos / (10000.0 ** (2.0 * i / HS))
    c, s = np.cos(ang), np.sin(ang)
    for vec, out, nh in ((q, q1, n_heads), (k, k1, n_kv)):
        v = vec.reshape(nh, HS).astype(np.float64)
        o = out.reshape(nh, HS)
        first = v[:, :64] * c - v[:, 64:] * s                  # textbook
        second_quirk = v[:, 64:] * c + first * s               # uses rotated first half
        second_textbook = v[:, 64:] * c + v[:, :64] * s
        np.testing.assert_allclose(o[:, :64], first, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(o[:, 64:], second_quirk, rtol=1e-4, atol=1e-5)
        assert np.max(np.abs(o[:, 64:] - second_textbook)) > 1e-2  # and it is NOT the textbook one
    # keys beyond n_kv heads do not exist; k heads use the same angles as q heads
    qq, kk = oracle.rope(np.tile(k[:HS], n_heads), k, pos, n_heads, n_kv, HS)
    np.testing.assert_array_equal(qq[:HS], kk[:HS])
    # table rows are the very same libm values
    ct, st = oracle.rope_table_row(pos, HS)
    np.testing.assert_allclose(ct, c, rtol=0, atol=2e-6)
    np.testing.assert_allclose(st, s, rtol=0, atol=2e-6)


def _attention_fp64(q, kc, vc, pos, n_heads, n_kv, HS):
    out = np.zeros((len(pos), n_heads * HS))
    ag = n_heads // n_kv
    for b, p in enumerate(pos):
        for h in range(n_heads):
            qh = q[b, h * HS:(h + 1) * HS].astype(np.float64)
            K = kc[:p + 1, h // ag].astype(np.float64)
            V = vc[:p + 1, h // ag].astype(np.float64)
            a = K @ qh / np.sqrt(HS)
            a = np.exp(a - a.max())
            a /= a.sum()
            out[b, h * HS:(h + 1) * HS] = a @ V
    return out


@pytest.mark.parametrize("n_heads,n_kv", [(2, 2), (8, 2)])
def test_attention(oracle, n_heads, n_kv):
    HS, T = 128, 40
    rng = np.random.default_rng(6)
    kc = rng.standard_normal((T, n_kv, HS)).astype(np.float32)
    vc = rng.standard_normal((T, n_kv, HS)).astype(np.float32)
    q = rng.standard_normal((3, n_heads * HS)).astype(np.float32)
    pos = [0, 17, 39]
    got = oracle.attention(q, vc, kc, pos, n_heads, n_kv, HS)
    np.testing.assert_allclose(got, _attention_fp64(q, kc, vc, pos, n_heads, n_kv, HS),
                               rtol=2e-4, atol=2e-5)
    # pos = 0: the output is V[0] of the head's kv group, whatever q is
    for h in range(n_heads):
        np.testing.assert_allclose(got[0, h * HS:(h + 1) * HS], vc[0, h // (n_heads // n_kv)],
                                   rtol=1e-6)
    # causal: entries beyond pos are never read
    vc2 = vc.copy()
    vc2[18:] = 1e30
    got2 = oracle.attention(q[1:2], vc2, kc, [17], n_heads, n_kv, HS)
    np.testing.assert_array_equal(got2[0], got[1])
    # uniform keys -> plain mean of the values
    ku = np.ones_like(kc)
    gm = oracle.attention(q[2:3], vc, ku, [39], n_heads, n_kv, HS)
    for h in range(n_heads):
        np.testing.assert_allclose(gm[0, h * HS:(h + 1) * HS],
                                   vc[:, h // (n_heads // n_kv)].mean(0), rtol=1e-4, atol=1e-5)


def test_argmax_last_index_on_ties(oracle):
    assert oracle.argmax(np.array([1, 3, 2, 3, 0], np.float32)) == 3
    assert oracle.argmax(np.array([5, 5, 5], np.float32)) == 2
    assert oracle.argmax(np.array([7, 1, 2], np.float32)) == 0
    assert oracle.argmax(np.array([-1.0], np.float32)) == 0
