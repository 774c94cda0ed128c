"""The moving average on [B, D, L] rows on the matrix cores for every activation type (blocks of 1024 tokens
with the end-state kernel in front, fp32 as two fp16 terms): carried state in and out on whole blocks, partial
last blocks, rows and masks that are not aligned for four tokens per access, few states, the two-pass form of
the two-sided layer, against the fp64 oracle (BaseMovingLayer.forward, fairseq/modules/base_moving_average.py:120-172)."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, mega_init_real, rel_err
from gpu_util import DEV, TOL, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16]


def _coeffs(rng, K, N, cplx):
    if cplx:
        return O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    return O.ema_coeffs_real(*mega_init_real(rng, K, N))


def _run(x, p, q, g, om, **kw):
    y, h = M.ops.ema_forward(x, dev(p), dev(q), dev(g), dev(om), **kw)
    torch.cuda.synchronize()
    return y, h


def _state_close(h, ho, cplx, tol):
    hh = host(h)
    assert rel_err(np.real(hh), np.real(ho)) < tol
    if cplx:
        assert rel_err(np.imag(hh), np.imag(ho)) < tol


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("N", [16, 7, 2])
@pytest.mark.parametrize("dtype", DTYPES)
def test_state_in_and_out_on_whole_blocks(dtype, N, cplx):
    """Three calls of 1024, 2048 and 1024 tokens with the state carried between them equal one call of 4096."""
    rng = np.random.default_rng(31)
    B, D, L = 2, 12, 4096
    p, q, g = _coeffs(rng, D, N, cplx)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    mask = np.zeros((B, L), bool); mask[1, 1500:1520] = True; mask[0, L - 40:] = True
    yo, ho = O.ema_forward(x64, p, q, g, om, mask, incremental=True)
    tm = dev(mask, torch.bool)
    h, ys = None, []
    for a, b in ((0, 1024), (1024, 3072), (3072, 4096)):
        y, h = _run(x[..., a:b].contiguous(), p, q, g, om, padding_mask=tm[:, a:b].contiguous(), h=h, want_state=True)
        ys.append(y)
    assert rel_err(host(torch.cat(ys, -1)), yo) < TOL[dtype]
    # the state is fp32 whatever the activations are; its error is that of the rounded products that built it
    _state_close(h, ho, cplx, 1e-4 if dtype is torch.float32 else 2e-3)
    y1, h1 = _run(x, p, q, g, om, padding_mask=tm, want_state=True)
    assert rel_err(host(y1), yo) < TOL[dtype]
    _state_close(h1, ho, cplx, 1e-4 if dtype is torch.float32 else 2e-3)


@pytest.mark.parametrize("bidir", [False, True])
@pytest.mark.parametrize("L", [1030, 2049, 5000, 16384])
@pytest.mark.parametrize("dtype", DTYPES)
def test_partial_blocks_and_odd_lengths(dtype, L, bidir):
    """Lengths that end inside a block and are not multiples of four (1030, 2049: one token at a time), a
    multiple of four that is no whole block (5000: the two-sided layer runs its directions one after the
    other with partial sums between them) and the longest row the path takes (16 blocks)."""
    rng = np.random.default_rng(32)
    B, D, N = 2, 6, 16
    p, q, g = _coeffs(rng, 2 * D if bidir else D, N, True)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    mask = rng.random((B, L)) < 0.03
    y, _ = _run(x, p, q, g, om, padding_mask=dev(mask, torch.bool), bidirectional=bidir)
    yo, _ = O.ema_forward(x64, p, q, g, om, mask, bidirectional=bidir)
    assert rel_err(host(y), yo) < TOL[dtype]


@pytest.mark.parametrize("bidir", [False, True])
@pytest.mark.parametrize("dtype", DTYPES)
def test_rows_that_start_off_the_vector_boundary(dtype, bidir):
    """x is a slice that starts one element into its buffer and has a row pitch that is no multiple of four:
    the kernel falls back to one token per access; the output goes into a caller's tensor."""
    rng = np.random.default_rng(33)
    B, D, N, L = 2, 5, 16, 2048
    p, q, g = _coeffs(rng, 2 * D if bidir else D, N, False)
    om = rng.normal(size=D)
    big, big64 = rounded(rng.normal(size=(B, D, L + 3)), dtype)
    x, x64 = big[..., 1:L + 1], big64[..., 1:L + 1]
    assert x.stride(1) % 4 != 0 and not x.is_contiguous()
    y, _ = _run(x, p, q, g, om, bidirectional=bidir)
    yo, _ = O.ema_forward(x64, p, q, g, om, None, bidirectional=bidir)
    assert rel_err(host(y), yo) < TOL[dtype]


def test_slow_poles_reach_across_all_blocks():
    """|q| close to one: every earlier block still matters at the end of the row (16 terms of the block sum)."""
    rng = np.random.default_rng(34)
    B, D, N, L = 1, 8, 16, 16384
    # coefficients that fp32 holds exactly: q^16384 moves by 16384 times the rounding of q, and the oracle must
    # start from the same q as the library
    p = (np.abs(rng.normal(size=(D, N))) * 0.05).astype(np.float32).astype(np.float64)
    q = (1.0 - 10.0 ** rng.uniform(-4.5, -2.0, size=(D, N))).astype(np.float32).astype(np.float64)
    g = (rng.normal(size=(D, N)) * 0.25).astype(np.float32).astype(np.float64)
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, D, L)), torch.float32)
    y, h = _run(x, p, q, g, om, want_state=True)
    yo, ho = O.ema_forward(x64, p, q, g, om, incremental=True)
    assert rel_err(host(y), yo) < 1e-4
    assert rel_err(np.real(host(h)), np.real(ho)) < 1e-4


@pytest.mark.parametrize("dtype,B,D,layout", [(torch.float32, 2, 24, "rows"), (torch.float16, 1, 8, "rows"),
                                              (torch.bfloat16, 1, 16, "rows"), (torch.bfloat16, 2, 64, "time_major")])
def test_kernel_generation_inside_the_call(dtype, B, D, layout):
    """Without a prepared image the call generates the operands its own kernel reads (the fp16 terms for fp32 /
    fp16 rows, the bf16 terms for bf16 on either kernel): the same result as with the prepared image."""
    rng = np.random.default_rng(35)
    N, L = 16, 2048
    p, q, g = _coeffs(rng, D, N, True)
    om = rng.normal(size=D)
    if layout == "rows":
        x, _ = rounded(rng.normal(size=(B, D, L)), dtype)
    else:
        xt, _ = rounded(rng.normal(size=(B, L, D)), dtype)
        x = xt.transpose(1, 2)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    y0, h0 = layer(x, None, None, want_state=True)
    saved, layer.image = layer.image, None
    y1, h1 = layer(x, None, None, want_state=True)
    layer.image = saved
    torch.cuda.synchronize()
    assert torch.equal(y0, y1) and torch.equal(torch.view_as_real(h0), torch.view_as_real(h1))
