"""The plain-C oracle (the timed CPU baseline) against the numpy oracle."""
import numpy as np
import pytest

import oracle_c_api as OC
from conftest import mega_init_complex, mega_init_real, rel_err
from oracle import mega_oracle as O


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("dt,tol", [(np.float64, 1e-11), (np.float32, 2e-5)])
def test_kernel_bias_hidden(cplx, dt, tol):
    rng = np.random.default_rng(0)
    K, N, L, B = 6, 16, 70, 3
    if cplx:
        p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    else:
        p, q, g = O.ema_coeffs_real(*mega_init_real(rng, K, N))
    h = rng.normal(size=(B, K, N)) + (1j * rng.normal(size=(B, K, N)) if cplx else 0)
    x = rng.normal(size=(B, K, L))
    assert rel_err(OC.ema_kernel(p, q, g, L, dt), O.ema_kernel(p, q, g, L)) < tol
    assert rel_err(OC.ema_bias(q, g, h, L, dt), O.ema_bias(q, g, h, L)) < tol
    hh = OC.ema_hidden(x, p, q, h, dt)
    ref = O.ema_hidden(x, p, q, h)
    assert rel_err(hh.real, ref.real) < tol and rel_err(hh.imag, np.asarray(ref).imag) < 10 * tol + 1e-9
    h0 = OC.ema_hidden(x, p, q, None, dt)
    assert rel_err(h0.real, O.ema_hidden(x, p, q).real) < tol


def test_direct_conv():
    rng = np.random.default_rng(1)
    x = rng.normal(size=(2, 3, 40)); k = rng.normal(size=(3, 25))
    assert rel_err(OC.causal_conv_direct(x, k), O.causal_conv_direct(x, k)) < 1e-12
    assert rel_err(OC.causal_conv_direct(x, k), O.causal_conv(x, np.pad(k, ((0, 0), (0, 15))))) < 1e-11


@pytest.mark.parametrize("G", [4, 1, None])
@pytest.mark.parametrize("dt,tol", [(np.float64, 1e-10), (np.float32, 3e-5)])
def test_timestep_norm(G, dt, tol):
    rng = np.random.default_rng(2)
    B, L, H = 3, 37, 40          # groups of 10 / 40: exercises the chunk-of-16 cascade and its tail
    x = rng.normal(size=(B, L, H)) + 0.5
    mask = rng.random((B, L)) < 0.25
    Gs = H if G is None else G
    pc = np.array([2, 5, 3], np.int64)
    pm = rng.normal(size=(B, Gs)) * 0.1; pv = rng.random((B, Gs)) + 0.5
    gamma = rng.normal(size=H) + 1; beta = rng.normal(size=H)
    a = OC.timestep_norm(x, pc, pm, pv, gamma, beta, mask, G, 1e-5, dt)
    b = O.timestep_norm(x, pc, pm, pv, gamma, beta, mask, G, 1e-5)
    assert rel_err(a[0], b[0]) < tol
    assert np.array_equal(a[1], b[1])
    assert rel_err(a[2], b[2]) < tol and rel_err(a[3], b[3]) < tol


def test_softmax():
    rng = np.random.default_rng(3)
    x = rng.normal(size=(2, 5, 9)); x[0, 1, :] = -np.inf
    for causal in (False, True):
        assert np.allclose(OC.attention_softmax(x, causal), O.attention_softmax(x, causal), atol=1e-14)
    x = rng.normal(size=(1, 6, 3))
    assert np.allclose(OC.attention_softmax(x, True), O.attention_softmax(x, True), atol=1e-14)
