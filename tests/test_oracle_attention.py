"""Pins the attention-softmax / attention / gate parts of the oracle."""
import numpy as np

from oracle import mega_oracle as O


def test_softmax_plain_and_right_aligned_causal():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(2, 3, 4, 6))
    y = O.attention_softmax(x, False)
    e = np.exp(x - x.max(-1, keepdims=True))
    assert np.allclose(y, e / e.sum(-1, keepdims=True), atol=1e-14)
    yc = O.attention_softmax(x, True)
    for r in range(4):
        n = 6 - 4 + r + 1
        e = np.exp(x[..., r, :n] - x[..., r, :n].max(-1, keepdims=True))
        assert np.allclose(yc[..., r, :n], e / e.sum(-1, keepdims=True), atol=1e-14)
        assert np.all(yc[..., r, n:] == 0)
    assert np.allclose(yc.sum(-1), 1)


def test_softmax_fully_masked_rows_are_zero():
    x = np.full((1, 2, 3), -np.inf)
    x[0, 1, 0] = 0.5
    y = O.attention_softmax(x, False)
    assert np.all(y[0, 0] == 0) and np.allclose(y[0, 1], [1, 0, 0])
    # outer > inner with the causal mask: the first rows keep no column at all
    y = O.attention_softmax(np.zeros((1, 4, 2)), True)
    assert np.all(y[0, :2] == 0) and np.allclose(y[0, 2], [1, 0]) and np.allclose(y[0, 3], [.5, .5])


def test_attention_matches_loops_and_chunks_are_independent():
    rng = np.random.default_rng(1)
    B, L, Nh, H1, H2 = 2, 5, 2, 3, 4
    q = rng.normal(size=(B, L, Nh, H1)); k = rng.normal(size=(B, L, Nh, H1)); v = rng.normal(size=(B, L, Nh, H2))
    y, w = O.attention(q, k, v, 0.7, True)
    for b in range(B):
        for n in range(Nh):
            for l in range(L):
                s = np.array([0.7 * q[b, l, n] @ k[b, j, n] for j in range(l + 1)])
                p = np.exp(s - s.max()); p /= p.sum()
                assert np.allclose(y[b, l, n], sum(p[j] * v[b, j, n] for j in range(l + 1)), atol=1e-12)
                assert np.allclose(w[b, n, l, :l + 1], p, atol=1e-14) and np.all(w[b, n, l, l + 1:] == 0)
    q2 = q.copy(); q2[1] += 1.0
    y2, _ = O.attention(q2, k, v, 0.7, True)
    assert np.array_equal(y2[0], y[0])


def test_swiglu_and_rotary():
    a = np.array([-2.0, 0.0, 3.0]); b = np.array([1.5, 2.0, -1.0])
    assert np.allclose(O.swiglu(a, b), a / (1 + np.exp(-a)) * b)
    rng = np.random.default_rng(2)
    x = rng.normal(size=(2, 7, 8))
    r = O.rotary(x)
    assert np.allclose(r[:, 0], x[:, 0])                                   # position 0 is not rotated
    assert np.allclose((r ** 2).sum(-1), (x ** 2).sum(-1))                 # rotations keep the norm
    # q.k after rotary depends on the position difference only
    q = rng.normal(size=(1, 1, 8)).repeat(7, 1); k = rng.normal(size=(1, 1, 8)).repeat(7, 1)
    rq, rk = O.rotary(q), O.rotary(k)
    assert np.isclose(rq[0, 5] @ rk[0, 3], rq[0, 4] @ rk[0, 2])


def _layer_params(rng, D, S, E, N):
    from conftest import mega_init_complex
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    return dict(norm_weight=rng.normal(size=D) * 0.1, norm_bias=rng.normal(size=D) * 0.1, p=p, q=q, ema_gamma=g,
                omega=rng.normal(size=D), v_w=rng.normal(size=(E, D)) * 0.2, v_b=rng.normal(size=E) * 0.1,
                mx_w=rng.normal(size=(2 * D + S + E, D)) * 0.2, mx_b=rng.normal(size=2 * D + S + E) * 0.1,
                h_w=rng.normal(size=(D, E)) * 0.2, gamma=rng.normal(size=(2, S)) * 0.1, beta=rng.normal(size=(2, S)) * 0.1)


def test_layer_gate_closed_forms_and_chunk_causality():
    rng = np.random.default_rng(5)
    B, L, D, S, E, N = 2, 12, 8, 4, 6, 4
    P = _layer_params(rng, D, S, E, N)
    x = rng.normal(size=(B, L, D))
    y = O.gated_attention_layer(x, P, chunk=4, num_groups=2)
    # u == 0 (a very negative gate bias) makes the layer the identity
    P0 = dict(P); P0['mx_b'] = P['mx_b'].copy(); P0['mx_b'][:D] = -1e4; P0['mx_w'] = P['mx_w'].copy(); P0['mx_w'][:D] = 0
    assert np.allclose(O.gated_attention_layer(x, P0, chunk=4, num_groups=2), x, atol=1e-12)
    # causal: outputs before t do not see x[t:]
    x2 = x.copy(); x2[:, 7:] += rng.normal(size=(B, 5, D))
    y2 = O.gated_attention_layer(x2, P, chunk=4, num_groups=2)
    assert np.allclose(y2[:, :7], y[:, :7], atol=1e-10) and not np.allclose(y2[:, 7:], y[:, 7:])
    # head split with one head equals the single-head layer; rms variant follows its formula
    assert np.allclose(O.gated_attention_layer(x, P, chunk=4, num_heads=1, num_groups=2), y)
    z = rng.normal(size=(3, 5))
    assert np.allclose(O.rms_norm(z, None, 1e-5), z / np.sqrt((z ** 2).mean(-1, keepdims=True) + 1e-5))
    yh = O.gated_attention_layer(x, P, chunk=4, num_heads=2, num_groups=2)
    assert yh.shape == y.shape and not np.allclose(yh, y)
