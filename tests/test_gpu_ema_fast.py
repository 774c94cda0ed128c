"""The matrix-core EMA path (bf16 activations, ndim <= 16, L >= 256) against the fp64 oracle:
both memory layouts, every feature the path claims (mask, carried state, bidirectional with
and without shift, real / complex, ragged sizes, idle channel lanes)."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, mega_init_real, rel_err
from gpu_util import DEV, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _coeffs(rng, K, N, cplx):
    if cplx:
        return O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    return O.ema_coeffs_real(*mega_init_real(rng, K, N))


def _check(y, yo, tol=2e-2, med=3e-3):
    e = np.abs(host(y) - yo)
    rms = np.sqrt(np.mean(yo ** 2))
    assert rel_err(host(y), yo) < tol
    # the typical error must look like bf16 output rounding (2^-9 relative), not like bf16 arithmetic
    assert np.median(e) < med * rms, (np.median(e), rms)


@pytest.mark.parametrize("out_layout", ["rows", "input"])
@pytest.mark.parametrize("time_major", [False, True])
@pytest.mark.parametrize("cplx", [True, False])
@pytest.mark.parametrize("B,D,N,L", [(2, 32, 16, 2048), (1, 24, 16, 1000), (2, 16, 7, 5000), (3, 40, 2, 256),
                                     (1, 8, 16, 4352)])
def test_causal(out_layout, time_major, cplx, B, D, N, L):
    print(f"case out={out_layout} time_major={time_major} cplx={cplx} B={B} D={D} N={N} L={L}", flush=True)
    rng = np.random.default_rng(31)
    p, q, g = _coeffs(rng, D, N, cplx)
    om = rng.normal(size=D)
    if time_major:
        xt, x64t = rounded(rng.normal(size=(B, L, D)), BF)
        x, x64 = xt.transpose(1, 2), x64t.transpose(0, 2, 1)
    else:
        x, x64 = rounded(rng.normal(size=(B, D, L)), BF)
    mask = np.zeros((B, L), bool)
    mask[0, L - L // 5:] = True
    mask[-1, 3] = True
    y, _ = M.ops.ema_forward(x, dev(p), dev(q), dev(g), dev(om), padding_mask=dev(mask, torch.bool),
                             out_layout=out_layout)
    torch.cuda.synchronize()
    assert y.stride() == (x.stride() if out_layout == "input" else (D * L, L, 1))
    yo, _ = O.ema_forward(x64, p, q, g, om, mask)
    _check(y, yo)
    y2, _ = M.ops.ema_forward(x, dev(p), dev(q), dev(g), dev(om), out_layout=out_layout)
    yo2, _ = O.ema_forward(x64, p, q, g, om)
    _check(y2, yo2)


@pytest.mark.parametrize("time_major", [False, True])
@pytest.mark.parametrize("L1,L2", [(1024, 512), (1000, 1048), (288, 300), (2048, 4096)])
def test_carried_state(time_major, L1, L2):
    rng = np.random.default_rng(32)
    B, D, N = 2, 32, 16
    L = L1 + L2
    p, q, g = _coeffs(rng, D, N, True)
    om = rng.normal(size=D)
    if time_major:
        xt, x64t = rounded(rng.normal(size=(B, L, D)), BF)
        x, x64 = xt.transpose(1, 2), x64t.transpose(0, 2, 1)
    else:
        x, x64 = rounded(rng.normal(size=(B, D, L)), BF)
    yo, ho = O.ema_forward(x64, p, q, g, om, incremental=True)
    a = x[..., :L1] if time_major else x[..., :L1].contiguous()
    c = x[..., L1:] if time_major else x[..., L1:].contiguous()
    y1, h1 = M.ops.ema_forward(a, dev(p), dev(q), dev(g), dev(om), want_state=True)
    y2, h2 = M.ops.ema_forward(c, dev(p), dev(q), dev(g), dev(om), h=h1)
    torch.cuda.synchronize()
    _check(torch.cat([y1, y2], -1), yo)
    assert rel_err(np.real(host(h2)), np.real(ho)) < 2e-3 and rel_err(np.imag(host(h2)), np.imag(ho)) < 2e-3


@pytest.mark.parametrize("time_major", [False, True])
@pytest.mark.parametrize("shift", [True, False])
@pytest.mark.parametrize("cplx", [True, False])
def test_bidirectional(time_major, shift, cplx):
    rng = np.random.default_rng(33)
    B, D, N, L = 2, 32, 16, 1536
    p, q, g = _coeffs(rng, 2 * D, N, cplx)
    om = rng.normal(size=D)
    if time_major:
        xt, x64t = rounded(rng.normal(size=(B, L, D)), BF)
        x, x64 = xt.transpose(1, 2), x64t.transpose(0, 2, 1)
    else:
        x, x64 = rounded(rng.normal(size=(B, D, L)), BF)
    mask = np.zeros((B, L), bool); mask[1, 1200:] = True
    y, _ = M.ops.ema_forward(x, dev(p), dev(q), dev(g), dev(om), padding_mask=dev(mask, torch.bool),
                             bidirectional=True, shift=shift)
    torch.cuda.synchronize()
    yo, _ = O.ema_forward(x64, p, q, g, om, mask, bidirectional=True, shift=shift)
    _check(y, yo)


def test_slowly_decaying_poles():
    """|q| close to 1 (trained-model regime): states stay large over many tiles."""
    rng = np.random.default_rng(34)
    B, D, N, L = 1, 16, 16, 8192
    mag = 1 - 10 ** rng.uniform(-4, -1.5, size=(D, N))
    q = mag * np.exp(1j * rng.uniform(0, np.pi, size=(D, N)))
    p = rng.random((D, N)) * 0.5
    g = (rng.normal(size=(D, N)) + 1j * rng.normal(size=(D, N))) / 4
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), BF)
    y, h = M.ops.ema_forward(x, dev(p), dev(q), dev(g), dev(om), want_state=True)
    torch.cuda.synchronize()
    yo, ho = O.ema_forward(x64, p, q, g, om, incremental=True)
    _check(y, yo)
    assert rel_err(np.real(host(h)), np.real(ho)) < 2e-3
