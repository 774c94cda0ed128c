"""Pins the TimestepNorm part of the oracle: the literal Welford recurrences against the
textbook statement (mean / biased variance of every element seen so far) and numpy."""
import numpy as np
import pytest

from conftest import rel_err
from oracle import mega_oracle as O


def _run(x, G, mask=None, count=None, mean=None, var=None, gamma=None, beta=None, eps=1e-5):
    B, L, H = x.shape
    Gs = H if G is None else G
    count = np.zeros(B, np.int64) if count is None else count
    mean = np.zeros((B, Gs)) if mean is None else mean
    var = np.ones((B, Gs)) if var is None else var
    gamma = np.ones(H) if gamma is None else gamma
    beta = np.zeros(H) if beta is None else beta
    return O.timestep_norm(x, count, mean, var, gamma, beta, mask, G, eps)


def test_group_matches_prefix_statistics():
    rng = np.random.default_rng(0)
    B, L, H, G = 2, 9, 12, 3
    x = rng.normal(size=(B, L, H)) * 2 + 1
    y, c, mu, v = _run(x, G)
    for b in range(B):
        for t in range(L):
            for g in range(G):
                seen = x[b, :t + 1, g * 4:(g + 1) * 4]
                exp = (x[b, t, g * 4:(g + 1) * 4] - seen.mean()) / np.sqrt(seen.var() + 1e-5)
                assert np.allclose(y[b, t, g * 4:(g + 1) * 4], exp, atol=1e-10)
    assert np.all(c == L)
    assert np.allclose(mu, x.reshape(B, L, G, 4).mean(axis=(1, 3)), atol=1e-12)
    assert np.allclose(v, x.reshape(B, L, G, 4).transpose(0, 2, 1, 3).reshape(B, G, -1).var(-1), atol=1e-12)


@pytest.mark.parametrize("G", [4, None])
def test_closed_form_with_mask_gamma_beta(G):
    rng = np.random.default_rng(1)
    B, L, H = 3, 31, 16
    x = rng.normal(size=(B, L, H))
    mask = rng.random((B, L)) < 0.3
    mask[:, 0] = False
    gamma = rng.normal(size=H) + 1; beta = rng.normal(size=H)
    if G is None:
        # the per-feature variant needs a prior with count > 1: use 2 pseudo-steps of (0, 1)
        y, c, mu, v = _run(x, None, mask, np.full(B, 2, np.int64), np.zeros((B, H)), np.ones((B, H)), gamma, beta)
        # 2 pseudo-steps with mean 0 and variance 1 == two extra samples -1, +1 per feature
        xx = np.concatenate([-np.ones((B, 1, H)), np.ones((B, 1, H)), x], 1)
        mm = np.concatenate([np.zeros((B, 2), bool), mask], 1)
        yc, _, _ = O.timestep_norm_closed_form(xx, mm, None, 1e-5, gamma, beta)
        assert rel_err(y, yc[:, 2:]) < 1e-9
        assert np.all(c == 2 + (~mask).sum(1))
    else:
        y, c, mu, v = _run(x, G, mask, gamma=gamma, beta=beta)
        yc, muc, vc = O.timestep_norm_closed_form(x, mask, G, 1e-5, gamma, beta)
        assert rel_err(y, yc) < 1e-9
        assert np.all(y[mask] == 0)
        assert np.allclose(mu, muc[:, -1], atol=1e-11) and np.allclose(v, vc[:, -1], atol=1e-11)
        assert np.all(c == (~mask).sum(1))


def test_chunk_split_and_prior():
    rng = np.random.default_rng(2)
    B, L, H, G = 2, 20, 8, 2
    x = rng.normal(size=(B, L, H))
    mask = rng.random((B, L)) < 0.2
    y, c, mu, v = _run(x, G, mask)
    y1, c1, m1, v1 = _run(x[:, :7], G, mask[:, :7])
    y2, c2, m2, v2 = _run(x[:, 7:], G, mask[:, 7:], c1, m1, v1)
    assert np.allclose(np.concatenate([y1, y2], 1), y, atol=1e-11)
    assert np.all(c2 == c) and np.allclose(m2, mu, atol=1e-12) and np.allclose(v2, v, atol=1e-12)
    # a prior (count c0, mean m, var s2) acts like c0 earlier steps whose group moments were (m, s2)
    c0 = 3
    pm = rng.normal(size=(B, G)); pv = rng.random((B, G)) + 0.5
    yp, cp, _, _ = _run(x, G, None, np.full(B, c0, np.int64), pm, pv)
    # build c0 synthetic steps with exactly those group moments: values m +- sqrt(s2)
    Dg = H // G
    pre = np.zeros((B, c0, H))
    for g in range(G):
        half = Dg // 2
        pre[:, :, g * Dg:g * Dg + half] = (pm[:, g] - np.sqrt(pv[:, g]))[:, None, None]
        pre[:, :, g * Dg + half:(g + 1) * Dg] = (pm[:, g] + np.sqrt(pv[:, g]))[:, None, None]
    yq, cq, _, _ = _run(np.concatenate([pre, x], 1), G)
    assert np.allclose(yq[:, c0:], yp, atol=1e-10) and np.all(cq == cp)


def test_constant_input_and_group_equals_feature():
    B, L, H = 1, 6, 4
    x = np.full((B, L, H), 3.0)
    beta = np.arange(H, dtype=float)
    y, _, _, v = _run(x, 2, beta=beta)
    assert np.allclose(y, beta) and np.allclose(v, 0)
    rng = np.random.default_rng(3)
    x = rng.normal(size=(2, 10, 5))
    cnt = np.full(2, 2, np.int64)
    # groups of one feature: the group operator must agree with the per-feature operator
    ya, ca, ma, va = _run(x, 5, None, cnt, np.zeros((2, 5)), np.ones((2, 5)))
    yb, cb, mb, vb = _run(x, None, None, cnt, np.zeros((2, 5)), np.ones((2, 5)))
    assert np.allclose(ya, yb, atol=1e-11) and np.allclose(ma, mb, atol=1e-12) and np.allclose(va, vb, atol=1e-12)
