"""HIP moving-average layer (kernel generation + long convolution + residual, fused) against
the fp64 oracle, which follows the reference's torch.fft path."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, mega_init_real, rel_err
from gpu_util import DEV, TOL, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu


def _coeffs(rng, K, N, cplx):
    if cplx:
        return O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    return O.ema_coeffs_real(*mega_init_real(rng, K, N))


def _run(x, p, q, g, om, **kw):
    y, h = M.ops.ema_forward(x, dev(p), dev(q), dev(g), dev(om), **kw)
    torch.cuda.synchronize()
    return y, h


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("B,D,N,L", [(2, 8, 16, 100), (1, 5, 2, 33), (3, 64, 16, 1000), (2, 16, 32, 64), (1, 3, 1, 1),
                                     (2, 7, 5, 257)])
def test_causal_matches_oracle(dtype, cplx, B, D, N, L):
    print(f"case dtype={dtype} cplx={cplx} B={B} D={D} N={N} L={L}", flush=True)
    rng = np.random.default_rng(11)
    p, q, g = _coeffs(rng, D, N, cplx)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    y, _ = _run(x, p, q, g, om)
    yo, _ = O.ema_forward(x64, p, q, g, om)
    assert y.shape == x.shape and y.dtype == dtype
    assert rel_err(host(y), yo) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_time_major_layout_and_mask(dtype):
    """x handed over as the transposed view of a [B, L, D] tensor (how the layer calls it)."""
    rng = np.random.default_rng(12)
    B, D, N, L = 2, 96, 16, 300
    p, q, g = _coeffs(rng, D, N, True)
    om = rng.normal(size=D)
    xt, x64t = rounded(rng.normal(size=(B, L, D)), dtype)
    mask = np.zeros((B, L), bool); mask[0, 250:] = True; mask[1, 17] = True
    y, _ = _run(xt.transpose(1, 2), p, q, g, om, padding_mask=dev(mask, torch.bool))
    assert y.shape == (B, D, L) and y.is_contiguous()      # the reference's convolution output layout
    yo, _ = O.ema_forward(x64t.transpose(0, 2, 1), p, q, g, om, mask)
    assert rel_err(host(y), yo) < TOL[dtype]


@pytest.mark.parametrize("cplx", [False, True])
def test_incremental_chunks_and_state(cplx):
    rng = np.random.default_rng(13)
    B, D, N, L = 2, 24, 16, 200
    p, q, g = _coeffs(rng, D, N, cplx)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), torch.float32)
    yo, ho = O.ema_forward(x64, p, q, g, om, incremental=True)
    h = None
    ys = []
    for a, b in ((0, 64), (64, 65), (65, 200)):
        y, h = _run(x[..., a:b].contiguous(), p, q, g, om, h=h, want_state=True)
        ys.append(y)
    assert rel_err(host(torch.cat(ys, -1)), yo) < 1e-4
    hh = host(h)
    assert rel_err(np.real(hh), np.real(ho)) < 1e-4
    if cplx:
        assert rel_err(np.imag(hh), np.imag(ho)) < 1e-4


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("B,D,L", [(2, 24, 3000), (16, 256, 4100)])
def test_long_rows_with_state_and_mask(cplx, B, D, L):
    """fp32 [B, D, L] rows on the vector-ALU path: 3000 steps is the single-kernel form with 64-step
    chunks; 16 x 256 rows of 4100 steps is the three-pass form with chunks of several sub-tiles (the
    last one partial), one-sided with a carried state in and out, and two-sided with a mask."""
    rng = np.random.default_rng(15)
    N = 16
    p, q, g = _coeffs(rng, 2 * D, N, cplx)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), torch.float32)
    # the carried state goes in only at the small shape (its bias term is a [B, D, N, L] array in the oracle)
    h0 = None
    if B * D < 100:
        h0 = (rng.normal(size=(B, D, N)) + (1j * rng.normal(size=(B, D, N)) if cplx else 0)).astype(np.complex64)
    mask = np.zeros((B, L), bool); mask[0, L - 77:] = True; mask[B - 1, 5] = True
    y, h = _run(x, p[:D], q[:D], g[:D], om, padding_mask=dev(mask, torch.bool), h=None if h0 is None else dev(h0),
                want_state=True)
    yo, ho = O.ema_forward(x64, p[:D], q[:D], g[:D], om, mask, h=h0, incremental=True)
    assert rel_err(host(y), yo) < 1e-4
    assert rel_err(np.real(host(h)), np.real(ho)) < 1e-4
    if cplx:
        assert rel_err(np.imag(host(h)), np.imag(ho)) < 1e-4
    y2, _ = _run(x, p, q, g, om, padding_mask=dev(mask, torch.bool), bidirectional=True, shift=False)
    yo2, _ = O.ema_forward(x64, p, q, g, om, mask, bidirectional=True, shift=False)
    assert rel_err(host(y2), yo2) < 1e-4


@pytest.mark.parametrize("shift", [True, False])
@pytest.mark.parametrize("trunc", [None, 40])
@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("L", [150, 256, 1000])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bidirectional(shift, trunc, cplx, L, dtype):
    rng = np.random.default_rng(14)
    B, D, N = 2, 12, 16
    p, q, g = _coeffs(rng, 2 * D, N, cplx)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    mask = np.zeros((B, L), bool); mask[1, L - 30:] = True
    y, _ = _run(x, p, q, g, om, padding_mask=dev(mask, torch.bool), bidirectional=True, truncation=trunc, shift=shift)
    yo, _ = O.ema_forward(x64, p, q, g, om, mask, bidirectional=True, truncation=trunc, shift=shift)
    assert rel_err(host(y), yo) < TOL[dtype]


@pytest.mark.parametrize("shift", [True, False])
@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("L", [1024, 3072])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_bidirectional_whole_blocks(shift, cplx, L, dtype):
    """Whole blocks of 1024 tokens: the two directions of a block are formed by one wave and meet before y is
    written; masked tokens in the middle of the rows, not only at their ends."""
    rng = np.random.default_rng(15)
    B, D, N = 2, 10, 16
    p, q, g = _coeffs(rng, 2 * D, N, cplx)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    mask = rng.random((B, L)) < 0.05
    mask[1, L - 100:] = True
    y, _ = _run(x, p, q, g, om, padding_mask=dev(mask, torch.bool), bidirectional=True, shift=shift)
    yo, _ = O.ema_forward(x64, p, q, g, om, mask, bidirectional=True, shift=shift)
    assert rel_err(host(y), yo) < TOL[dtype]
    y2, _ = _run(x, p, q, g, om, bidirectional=True, shift=shift)
    yo2, _ = O.ema_forward(x64, p, q, g, om, None, bidirectional=True, shift=shift)
    assert rel_err(host(y2), yo2) < TOL[dtype]


def test_modules_forward():
    torch.manual_seed(3)
    B, D, N, L = 2, 32, 16, 128
    for cls, kw in ((M.MultiHeadComplexEMA, {}), (M.MultiHeadEMA, {}), (M.MultiHeadEMA, {"bidirectional": True})):
        m = cls(D, ndim=N, **kw).to(DEV).eval()
        x = torch.randn(B, D, L, device=DEV)
        with torch.no_grad():
            y = m(x)
        p, q, g = m.coeffs()
        yo, _ = O.ema_forward(host(x), host(p.squeeze(-1)), host(q.squeeze(-1)), host(g), host(m.omega).reshape(-1),
                              bidirectional=kw.get("bidirectional", False))
        assert rel_err(host(y), yo) < 1e-4


def test_config0_real_ema_b2_l1024_d512():
    rng = np.random.default_rng(1234)
    B, D, N, L = 2, 512, 16, 1024
    p, q, g = _coeffs(rng, D, N, False)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), torch.float32)
    y, _ = _run(x, p, q, g, om)
    yo, _ = O.ema_forward(x64, p, q, g, om)
    assert rel_err(host(y), yo) < 1e-4


def test_config1_bidirectional_b1_l16384_d256():
    rng = np.random.default_rng(1235)
    B, D, N, L = 1, 256, 16, 16384
    p, q, g = _coeffs(rng, 2 * D, N, False)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), torch.float32)
    mask = np.zeros((B, L), bool); mask[0, L - int(rng.integers(0, L // 4)):] = True
    y, _ = _run(x, p, q, g, om, padding_mask=dev(mask, torch.bool), bidirectional=True)
    yo, _ = O.ema_forward(x64, p, q, g, om, mask, bidirectional=True)
    assert rel_err(host(y), yo) < 1e-4


def test_config2_cema_b4_l4096_d1024_bf16():
    rng = np.random.default_rng(1236)
    B, D, N, L = 4, 1024, 16, 4096
    p, q, g = _coeffs(rng, D, N, True)
    om = rng.normal(size=D)
    xt, x64t = rounded(rng.normal(size=(B, L, D)), torch.bfloat16)
    y, _ = _run(xt.transpose(1, 2), p, q, g, om)
    yo, _ = O.ema_forward(x64t.transpose(0, 2, 1), p, q, g, om)
    assert rel_err(host(y), yo) < TOL[torch.bfloat16]
    assert np.median(np.abs(host(y) - yo)) < 5e-3 * np.sqrt(np.mean(yo ** 2))


def test_decode_steps_agree_with_parallel_path():
    """Recurrent single-step updates against the parallel path on the concatenation, fp32:
    the two HIP paths within 1e-5 of each other and within 1e-4 of the oracle."""
    rng = np.random.default_rng(1237)
    B, D, N, T = 8, 64, 16, 256
    p, q, g = _coeffs(rng, D, N, True)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, T)), torch.float32)
    tp, tq, tg, to = dev(p), dev(q), dev(g), dev(om)
    h = None
    ys = []
    for t in range(T):
        yt, h = M.ops.ema_step(x[:, :, t].contiguous(), tp, tq, tg, to, h)
        ys.append(yt)
    ystep = torch.stack(ys, -1)
    ypar, hpar = M.ops.ema_forward(x, tp, tq, tg, to, want_state=True)
    torch.cuda.synchronize()
    yo, ho = O.ema_forward(x64, p, q, g, om, incremental=True)
    assert rel_err(host(ystep), host(ypar)) < 1e-5
    assert rel_err(host(ystep), yo) < 1e-4
    assert np.abs(host(h) - host(hpar)).max() < 1e-5 * max(1.0, float(np.abs(ho).max()))
    assert rel_err(np.real(host(h)), np.real(ho)) < 1e-4


def test_errors():
    x = torch.zeros(1, 4, 8, device=DEV)
    with pytest.raises(RuntimeError, match="ndim"):
        M.ops.ema_forward(x, torch.zeros(4, 40, device=DEV), torch.zeros(4, 40, device=DEV),
                          torch.zeros(4, 40, device=DEV), torch.zeros(4, device=DEV))
    with pytest.raises(RuntimeError, match="kernel_dim"):
        M.ops.ema_forward(x, torch.zeros(4, 2, device=DEV), torch.zeros(4, 2, device=DEV),
                          torch.zeros(4, 2, device=DEV), torch.zeros(4, device=DEV), bidirectional=True)
