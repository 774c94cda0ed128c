"""Pins of the oracle's backward restatements (CPU only):
  * central differences of the oracle's own fp64 forward (a dropped term, a wrong sign or a
    transposed index in the backward fails these);
  * the outputs of the reference's own CPU operators (tests/golden/ref_cpu_vectors.npz)."""
import os

import numpy as np
import pytest

from conftest import mega_init_complex, rel_err
from oracle import mega_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_cpu_vectors.npz")


def _fd(f, arr, idx, unit=1.0, e=1e-6):
    a1, a2 = arr.copy(), arr.copy()
    a1[idx] += e * unit
    a2[idx] -= e * unit
    return (f(a1) - f(a2)) / (2 * e)


@pytest.mark.parametrize("G,masked,prior", [(4, True, 3), (None, True, 2), (2, False, 0), (8, True, 0)])
def test_timestep_norm_bwd_matches_finite_differences(G, masked, prior):
    rng = np.random.default_rng(7)
    B, L, H = 2, 11, 8
    GG = H if G is None else G
    x = rng.normal(size=(B, L, H))
    gamma, beta = rng.normal(size=H) + 1, rng.normal(size=H)
    mask = (rng.random((B, L)) < 0.3) if masked else None      # interior padding included
    pc = np.array([prior, prior + 1]) if prior else np.zeros(B, np.int64)
    pm, pv = rng.normal(size=(B, GG)) * 0.3, rng.random((B, GG)) + 0.5
    wy, wm, wv = rng.normal(size=(B, L, H)), rng.normal(size=(B, GG)), rng.normal(size=(B, GG))

    def loss(x_, pm_, pv_, g_, b_):
        y, _, mu, v = O.timestep_norm(x_, pc, pm_, pv_, g_, b_, mask, G, 1e-5)
        return (y * wy).sum() + (mu * wm).sum() + (v * wv).sum()

    cnt, gm, cm, cr = O.timestep_norm_saved(x, pc, pm, pv, mask, G, 1e-5)
    grads = O.timestep_norm_bwd(wy, wm, wv, x, pm, cnt, gm if G else None, cm, cr, gamma, mask, G)
    args = [x, pm, pv, gamma, beta]
    for which, g in enumerate(grads):
        if which in (1, 2) and prior == 0:
            continue                                           # count 0: the prior has no weight
        for _ in range(8):
            idx = tuple(rng.integers(0, s) for s in args[which].shape)
            f = lambda a: loss(*[a if i == which else args[i] for i in range(5)])
            assert abs(_fd(f, args[which], idx) - g[idx]) < 1e-6


@pytest.mark.parametrize("masked,bidir,shift", [(False, False, True), (True, False, True), (True, True, True),
                                                (False, True, False)])
def test_ema_backward_matches_finite_differences(masked, bidir, shift):
    rng = np.random.default_rng(8)
    D, N, L, B = 3, 4, 13, 2
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, 2 * D if bidir else D, N))
    om = rng.normal(size=D)
    x, wy = rng.normal(size=(B, D, L)), rng.normal(size=(B, D, L))
    mask = (rng.random((B, L)) < 0.3) if masked else None
    loss = lambda x_, p_, q_, g_, o_: (O.ema_forward(x_, p_, q_, g_, o_, mask, bidirectional=bidir,
                                                     shift=shift)[0] * wy).sum()
    dx, dp, dq, dg, dom = O.ema_backward(wy, x, p, q, g, om, mask, bidir, shift)
    for _ in range(6):
        i = tuple(rng.integers(0, s) for s in x.shape)
        j = tuple(rng.integers(0, s) for s in p.shape)
        d = (int(rng.integers(0, D)),)
        assert abs(_fd(lambda a: loss(a, p, q, g, om), x, i) - dx[i]) < 1e-6
        assert abs(_fd(lambda a: loss(x, a, q, g, om), p, j) - dp[j]) < 1e-6
        assert abs(_fd(lambda a: loss(x, p, q, g, a), om, d) - dom[d]) < 1e-6
        # complex gradients: real part = d/dRe, imaginary part = d/dIm
        assert abs(_fd(lambda a: loss(x, p, a, g, om), q, j) - dq[j].real) < 1e-6
        assert abs(_fd(lambda a: loss(x, p, a, g, om), q, j, 1j) - dq[j].imag) < 1e-6
        assert abs(_fd(lambda a: loss(x, p, q, a, om), g, j) - dg[j].real) < 1e-6
        assert abs(_fd(lambda a: loss(x, p, q, a, om), g, j, 1j) - dg[j].imag) < 1e-6


@pytest.mark.parametrize("G,last,masked", [(4, False, True), (None, True, True), (2, True, False)])
def test_sequence_norm_bwd_matches_finite_differences(G, last, masked):
    rng = np.random.default_rng(10)
    B, L, H = 2, 9, 8
    x = rng.normal(size=(B, H, L) if last else (B, L, H))
    wy = rng.normal(size=x.shape)
    gamma, beta = rng.normal(size=H) + 1, rng.normal(size=H)
    mask = (rng.random((B, L)) < 0.3) if masked else None
    loss = lambda x_, g_, b_: (O.sequence_norm(x_, g_, b_, mask, G, 1e-5, last)[0] * wy).sum()
    dx, dg, db = O.sequence_norm_bwd(wy, x, gamma, mask, G, 1e-5, last)
    for _ in range(10):
        i = tuple(rng.integers(0, s) for s in x.shape)
        c = (int(rng.integers(0, H)),)
        assert abs(_fd(lambda a: loss(a, gamma, beta), x, i) - dx[i]) < 1e-6
        assert abs(_fd(lambda a: loss(x, a, beta), gamma, c) - dg[c]) < 1e-6
        assert abs(_fd(lambda a: loss(x, gamma, a), beta, c) - db[c]) < 1e-6


@pytest.mark.parametrize("causal", [True, False])
def test_attention_bwd_matches_finite_differences(causal):
    rng = np.random.default_rng(9)
    B, L, Nh, H1, H2 = 2, 7, 2, 4, 5
    q, k = rng.normal(size=(B, L, Nh, H1)), rng.normal(size=(B, L, Nh, H1))
    v, wy = rng.normal(size=(B, L, Nh, H2)), rng.normal(size=(B, L, Nh, H2))
    loss = lambda q_, k_, v_: (O.attention(q_, k_, v_, 0.7, causal)[0] * wy).sum()
    dq, dk, dv = O.attention_bwd(wy, q, k, v, 0.7, causal)
    for _ in range(8):
        i = tuple(rng.integers(0, s) for s in q.shape)
        j = tuple(rng.integers(0, s) for s in v.shape)
        assert abs(_fd(lambda a: loss(a, k, v), q, i) - dq[i]) < 1e-6
        assert abs(_fd(lambda a: loss(q, a, v), k, i) - dk[i]) < 1e-6
        assert abs(_fd(lambda a: loss(q, k, a), v, j) - dv[j]) < 1e-6
    # the softmax step alone: derivative of sum(softmax(x) * w)
    x, w = rng.normal(size=(3, 5, 9)), rng.normal(size=(3, 5, 9))
    y = O.attention_softmax(x, causal)
    dx = O.attention_softmax_bwd(w, y)
    for _ in range(8):
        i = tuple(rng.integers(0, s) for s in x.shape)
        assert abs(_fd(lambda a: (O.attention_softmax(a, causal) * w).sum(), x, i) - dx[i]) < 1e-6


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def _case(gold, tag):
    return {k[len(tag) + 1:]: gold[k] for k in gold.files if k.startswith(tag + ".")}


@pytest.mark.parametrize("tag", ["gtsn_bwd_a", "gtsn_bwd_b", "tsn_bwd"])
def test_timestep_norm_bwd_matches_reference_vectors(gold, tag):
    c = _case(gold, tag)
    G = int(c["groups"]) or None
    mask = c.get("mask")
    cnt, gm, cm, cr = O.timestep_norm_saved(c["x"], c["prev_count"], c["prev_mean"], c["prev_var"], mask, G, 1e-5)
    got = O.timestep_norm_bwd(c["y_grad"], c["mean_grad"], c["var_grad"], c["x"], c["prev_mean"], cnt,
                              gm if G else None, cm, cr, c["gamma"], mask, G)
    for a, name in zip(got, ("x_grad", "prev_mean_grad", "prev_var_grad", "gamma_grad", "beta_grad")):
        assert rel_err(a, c[name]) < 5e-5, name            # the vectors are fp32 results


def test_ema_kernel_bwd_matches_reference_vectors(gold):
    c = _case(gold, "ema_bwd")
    dp, dq, dg = O.ema_kernel_bwd(c["kernel_grad"], c["p"], c["q"], c["gamma"])
    assert rel_err(dp, c["p_grad"]) < 5e-5
    for a, b in ((dq, c["q_grad"]), (dg, c["gamma_grad"])):
        assert rel_err(a.real, b.real) < 5e-5 and rel_err(a.imag, b.imag) < 5e-5


@pytest.mark.parametrize("tag", ["gsn_bwd_a", "gsn_bwd_b", "sn_bwd"])
def test_sequence_norm_bwd_matches_reference_vectors(gold, tag):
    c = _case(gold, tag)
    G = int(c["groups"]) or None
    dx, dg, db = O.sequence_norm_bwd(c["y_grad"], c["x"], c["gamma"], c.get("mask"), G, 1e-5, bool(c["length_last"]))
    assert rel_err(dx, c["x_grad"]) < 5e-5 and rel_err(dg, c["gamma_grad"]) < 5e-5 and rel_err(db, c["beta_grad"]) < 5e-5


def test_ema_bias_bwd_matches_finite_differences_and_reference_vectors(gold):
    rng = np.random.default_rng(11)
    D, N, L, B = 3, 4, 9, 2
    _, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    h = rng.normal(size=(B, D, N)) + 1j * rng.normal(size=(B, D, N))
    wb = rng.normal(size=(B, D, L))
    loss = lambda q_, g_, h_: (O.ema_bias(q_, g_, h_, L) * wb).sum()
    dq, dg, dh = O.ema_bias_bwd(wb, q, g, h)
    for _ in range(6):
        j = tuple(rng.integers(0, s) for s in q.shape)
        i = tuple(rng.integers(0, s) for s in h.shape)
        for unit, part in ((1.0, "real"), (1j, "imag")):
            assert abs(_fd(lambda a: loss(a, g, h), q, j, unit) - getattr(dq[j], part)) < 1e-6
            assert abs(_fd(lambda a: loss(q, a, h), g, j, unit) - getattr(dg[j], part)) < 1e-6
            assert abs(_fd(lambda a: loss(q, g, a), h, i, unit) - getattr(dh[i], part)) < 1e-6
    c = _case(gold, "ema_bwd")
    dp, dq, dg = O.ema_kernel_bwd(c["kernel_grad"], c["p"], c["q"], c["gamma"])
    bq, bg, bh = O.ema_bias_bwd(c["bias_grad"], c["q"], c["gamma"], c["h"])
    assert rel_err(dp, c["p_grad_b"]) < 5e-5
    for a, b in ((dq + bq, c["q_grad_b"]), (dg + bg, c["gamma_grad_b"]), (bh, c["h_grad_b"])):
        assert rel_err(a.real, b.real) < 5e-5 and rel_err(a.imag, b.imag) < 5e-5


def test_ema_hidden_bwd_matches_finite_differences_and_reference_vectors(gold):
    rng = np.random.default_rng(12)
    D, N, L, B = 3, 4, 10, 2
    p, q, _ = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    x = rng.normal(size=(B, D, L))
    h = rng.normal(size=(B, D, N)) + 1j * rng.normal(size=(B, D, N))
    w = rng.normal(size=(B, D, N)) + 1j * rng.normal(size=(B, D, N))      # loss = Re sum conj(w) h'
    loss = lambda x_, p_, q_, h_: np.real(np.conj(w) * O.ema_hidden(x_, p_, q_, h_)).sum()
    dx, dp, dq, dh = O.ema_hidden_bwd(w, x, p, q, h)
    for _ in range(6):
        i = tuple(rng.integers(0, s) for s in x.shape)
        j = tuple(rng.integers(0, s) for s in p.shape)
        k = tuple(rng.integers(0, s) for s in h.shape)
        assert abs(_fd(lambda a: loss(a, p, q, h), x, i) - dx[i]) < 1e-6
        assert abs(_fd(lambda a: loss(x, a, q, h), p, j) - dp[j]) < 1e-6
        for unit, part in ((1.0, "real"), (1j, "imag")):
            assert abs(_fd(lambda a: loss(x, p, a, h), q, j, unit) - getattr(dq[j], part)) < 1e-6
            assert abs(_fd(lambda a: loss(x, p, q, a), h, k, unit) - getattr(dh[k], part)) < 1e-6
    c = _case(gold, "hid_bwd")
    dx, dp, dq, dh = O.ema_hidden_bwd(c["y_grad"], c["x"], c["p"], c["q"], c["h"])
    assert rel_err(dx, c["x_grad"]) < 5e-5 and rel_err(dp, c["p_grad"]) < 5e-5
    for a, b in ((dq, c["q_grad"]), (dh, c["h_grad"])):
        assert rel_err(a.real, b.real) < 5e-5 and rel_err(a.imag, b.imag) < 5e-5
