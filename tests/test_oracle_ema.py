"""Pins the EMA part of the oracle without the reference's code: closed forms, brute force
and library routines chosen so that a dropped term, a wrong sign / index or a transposed
operand fails at least one of them."""
import math

import numpy as np
import pytest

from conftest import mega_init_complex, mega_init_real, rel_err
from oracle import mega_oracle as O


def _coeffs(rng, K, N, cplx):
    if cplx:
        a, d, t, g = mega_init_complex(rng, K, N)
        return O.ema_coeffs_complex(a, d, t, g)
    a, d, b, g = mega_init_real(rng, K, N)
    return O.ema_coeffs_real(a, d, b, g)


def test_coeffs_real_closed_form():
    rng = np.random.default_rng(0)
    a, d, b, g = mega_init_real(rng, 5, 4)
    p, q, gm = O.ema_coeffs_real(a, d, b, g)
    for k in range(5):
        for n in range(4):
            sa = 1 / (1 + math.exp(-a[k, n, 0]))
            sd = 1 / (1 + math.exp(-d[k, n, 0]))
            assert q[k, n] == pytest.approx(1 - sa * sd, rel=1e-14)
            assert p[k, n] == pytest.approx(sa * b[k, n, 0], rel=1e-14)
            assert gm[k, n] == pytest.approx(g[k, n] * 0.5, rel=1e-14)
    assert np.all((q > 0) & (q < 1))


def test_coeffs_complex_invariants():
    rng = np.random.default_rng(1)
    K, N = 6, 16
    a, d, t, g = mega_init_complex(rng, K, N)
    p, q, gm = O.ema_coeffs_complex(a, d, t, g)
    assert np.all(np.abs(q) < 1) and np.all(np.abs(q) > 0)
    ang = np.angle(q)
    phi = (1 / (1 + np.exp(-t.reshape(K)))) * 2 * math.pi / N
    # theta_{d,n} = (n+1) theta_{d,0}: compare on the unit circle (angles wrap)
    for n in range(N):
        assert np.allclose(np.exp(1j * ang[:, n]), np.exp(1j * (n + 1) * phi), atol=1e-12)
    assert np.allclose(np.abs(q), 1 - p * (1 / (1 + np.exp(-d.reshape(K, N)))), atol=1e-14)
    assert np.all(gm.imag == 0)                     # imaginary part of gamma starts at 0
    assert np.allclose(gm.real, g[..., 0] / 4.0)


@pytest.mark.parametrize("cplx", [False, True])
def test_kernel_bruteforce_powers(cplx):
    """exp(l log q) against repeated multiplication, term by term."""
    rng = np.random.default_rng(2)
    K, N, L = 4, 8, 50
    p, q, g = _coeffs(rng, K, N, cplx)
    w = O.ema_kernel(p, q, g, L)
    ref = np.zeros((K, L))
    for d in range(K):
        for n in range(N):
            pw = 1.0 + 0j
            for l in range(L):
                ref[d, l] += (p[d, n] * g[d, n] * pw).real
                pw = pw * q[d, n]
    assert rel_err(w, ref) < 1e-12


def test_kernel_geometric_closed_form():
    """N = 1, gamma' = 1: k[l] = p q^l and sum_l k[l] -> p / (1 - q)."""
    p = np.array([[0.3]]); q = np.array([[0.9]]); g = np.array([[1.0]])
    w = O.ema_kernel(p, q, g, 400)
    assert np.allclose(w[0], 0.3 * 0.9 ** np.arange(400), rtol=1e-12)
    assert w.sum() == pytest.approx(0.3 / (1 - 0.9), rel=1e-10)
    assert O.ema_kernel(p, q, g, 1)[0, 0] == pytest.approx(0.3)      # L = 1: Re sum p gamma


def test_bias_is_shifted_kernel():
    """With h = p e_n summed over n the bias is the kernel advanced by one lag."""
    rng = np.random.default_rng(3)
    K, N, L = 3, 4, 20
    p, q, g = _coeffs(rng, K, N, True)
    h = np.broadcast_to(p[None].astype(np.complex128), (2, K, N))
    b = O.ema_bias(q, g, h, L)
    w = O.ema_kernel(p, q, g, L + 1)
    assert rel_err(b[0], w[:, 1:]) < 1e-12 and rel_err(b[1], w[:, 1:]) < 1e-12


def test_causal_conv_against_direct_and_numpy():
    rng = np.random.default_rng(4)
    for L in (1, 7, 32, 33, 100):
        x = rng.normal(size=(2, 3, L)); k = rng.normal(size=(3, L))
        y = O.causal_conv(x, k)
        assert rel_err(y, O.causal_conv_direct(x, k)) < 1e-11
        for b in range(2):
            for d in range(3):
                assert np.allclose(y[b, d], np.convolve(x[b, d], k[d])[:L], atol=1e-10)


def test_causal_conv_impulse_causality_linearity():
    rng = np.random.default_rng(5)
    L = 40
    k = rng.normal(size=(2, L))
    x = np.zeros((1, 2, L)); x[0, :, 9] = 1.0
    y = O.causal_conv(x, k)
    assert np.allclose(y[0, :, :9], 0, atol=1e-12) and np.allclose(y[0, :, 9:], k[:, :L - 9], atol=1e-12)
    x1 = rng.normal(size=(1, 2, L)); x2 = x1.copy(); x2[..., 20:] += rng.normal(size=(1, 2, 20))
    assert np.allclose(O.causal_conv(x1, k)[..., :20], O.causal_conv(x2, k)[..., :20], atol=1e-11)
    assert np.allclose(O.causal_conv(2 * x1 - 3 * x2, k), 2 * O.causal_conv(x1, k) - 3 * O.causal_conv(x2, k), atol=1e-10)


@pytest.mark.parametrize("shift", [True, False])
@pytest.mark.parametrize("Lk", [12, 5])
def test_bidirectional_conv_lag_formulas(shift, Lk):
    rng = np.random.default_rng(6)
    B, D, L = 2, 3, 12
    x = rng.normal(size=(B, D, L)); k = rng.normal(size=(2 * D, Lk))
    assert rel_err(O.bidirectional_conv(x, k, shift), O.bidirectional_conv_direct(x, k, shift)) < 1e-11


def test_bidirectional_time_reversal_symmetry():
    """Reversing x and swapping the halves (shift = False) reverses y."""
    rng = np.random.default_rng(7)
    D, L = 2, 9
    x = rng.normal(size=(1, D, L)); k = rng.normal(size=(2 * D, L))
    y = O.bidirectional_conv(x, k, False)
    ks = np.concatenate([k[D:], k[:D]])
    yr = O.bidirectional_conv(x[..., ::-1].copy(), ks, False)
    assert np.allclose(yr[..., ::-1], y, atol=1e-11)
    # shift=False minus shift=True: + k2[0] x[t] + sum_{m>=1} (k2[m] - k2[m-1]) x[t+m]
    diff = O.bidirectional_conv(x, k, False) - O.bidirectional_conv(x, k, True)
    k2 = k[D:]
    exp = np.zeros_like(x)
    for t in range(L):
        exp[0, :, t] = k2[:, 0] * x[0, :, t]
        for m in range(1, L - t):
            exp[0, :, t] += (k2[:, m] - k2[:, m - 1]) * x[0, :, t + m]
    assert np.allclose(diff, exp, atol=1e-11)


@pytest.mark.parametrize("cplx", [False, True])
def test_forward_mask_and_residual(cplx):
    rng = np.random.default_rng(8)
    B, D, N, L = 2, 3, 4, 17
    p, q, g = _coeffs(rng, D, N, cplx)
    om = rng.normal(size=D)
    x = rng.normal(size=(B, D, L))
    mask = np.zeros((B, L), bool); mask[0, 11:] = True; mask[1, :] = True
    y, _ = O.ema_forward(x, p, q, g, om, mask)
    assert np.allclose(y[1], om[:, None] * x[1], atol=1e-12)         # all masked: only the residual
    x2 = x.copy(); x2[0, :, 11:] = 0
    y2, _ = O.ema_forward(x2, p, q, g, om, None)
    assert np.allclose(y[0, :, :11], y2[0, :, :11], atol=1e-12)
    assert np.allclose(y[0, :, 11:] - om[:, None] * x[0, :, 11:], y2[0, :, 11:], atol=1e-12)


@pytest.mark.parametrize("cplx", [False, True])
def test_recurrence_equals_parallel_and_chunk_split(cplx):
    rng = np.random.default_rng(9)
    B, D, N, L = 2, 3, 4, 23
    p, q, g = _coeffs(rng, D, N, cplx)
    om = rng.normal(size=D)
    x = rng.normal(size=(B, D, L))
    y, hL = O.ema_forward(x, p, q, g, om, incremental=True)
    h = None
    ys = []
    for t in range(L):
        yt, h = O.ema_one_step(x[:, :, t], p, q, g, om, h)
        ys.append(yt)
    assert rel_err(np.stack(ys, -1), y) < 1e-11
    assert rel_err(np.abs(h - hL), np.zeros_like(np.abs(h))) < 1e-11 or np.allclose(h, hL, atol=1e-11)
    # split 0:9 | 9:23 with the carried state
    y1, h1 = O.ema_forward(x[..., :9], p, q, g, om, incremental=True)
    y2, h2 = O.ema_forward(x[..., 9:], p, q, g, om, h=h1)
    assert np.allclose(np.concatenate([y1, y2], -1), y, atol=1e-11)
    assert np.allclose(h2, hL, atol=1e-11)
    # x = 0: the state only decays
    hz = O.ema_hidden(np.zeros((B, D, 5)), p, q, h1)
    assert np.allclose(hz, q[None] ** 5 * h1, atol=1e-12)


def test_truncated_bidirectional_layer_matches_lags():
    rng = np.random.default_rng(10)
    B, D, N, L, T = 1, 2, 4, 14, 5
    p, q, g = _coeffs(rng, 2 * D, N, True)
    om = rng.normal(size=D)
    x = rng.normal(size=(B, D, L))
    y, _ = O.ema_forward(x, p, q, g, om, bidirectional=True, truncation=T, shift=True)
    k = O.ema_kernel(p, q, g, T)
    assert rel_err(y, O.bidirectional_conv_direct(x, k, True) + om[None, :, None] * x) < 1e-11
