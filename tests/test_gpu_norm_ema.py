"""TimestepNorm -> moving average in one call (mega_norm_ema_fwd) against the fp64 oracle and against
the two operators run one after the other: the one-kernel envelope (bf16, 64 or 128 channels per group, padding
masks, rows of any length), carried state in and out, both output layouts, slowly decaying poles, prior
statistics, and shapes outside the envelope (which take the two-operator route inside the call)."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, mega_init_real, rel_err
from gpu_util import DEV, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


def _setup(rng, D, N, cplx=True):
    if cplx:
        p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    else:
        p, q, g = O.ema_coeffs_real(*mega_init_real(rng, D, N))
    om = rng.normal(size=D)
    nw = rng.normal(size=D) * 0.1
    nb = rng.normal(size=D) * 0.1
    return p, q, g, om, nw, nb


def _check_y(y, yo, tol=2e-2, med=3e-3):
    e = np.abs(host(y) - yo)
    rms = np.sqrt(np.mean(yo ** 2))
    assert rel_err(host(y), yo) < tol
    assert np.median(e) < med * rms, (np.median(e), rms)


def _run(layer, x, G, nw, nb, prior=None, **kw):
    B = x.shape[0]
    if prior is None:
        pc = torch.zeros(B, dtype=torch.int64, device=DEV)
        pm = torch.zeros(B, G, device=DEV)
        pv = torch.ones(B, G, device=DEV)
    else:
        pc, pm, pv = prior
    out = layer.norm_forward(x, pc, pm, pv, dev(nw + 1), dev(nb), G, 1e-5, **kw)
    torch.cuda.synchronize()
    assert M.ops.timestep_norm_status() == 0
    return out


@pytest.mark.parametrize("out_layout", ["rows", "input"])
@pytest.mark.parametrize("B,L,G,N,cplx,cpg", [(2, 1024, 2, 16, True, 64), (1, 4096, 8, 16, True, 64),
                                             (3, 2048, 1, 7, False, 64), (1, 3072, 16, 16, True, 64),
                                             (2, 2048, 2, 16, True, 128), (1, 3072, 8, 9, False, 128),
                                             (3, 1024, 1, 16, True, 128)])
def test_one_kernel_envelope_against_oracle(out_layout, B, L, G, N, cplx, cpg):
    """cpg: channels per norm group; groups of 128 channels are shared by two workgroups."""
    print(f"case out={out_layout} B={B} L={L} G={G} N={N} cplx={cplx} cpg={cpg}", flush=True)
    D = cpg * G
    rng = np.random.default_rng(51)
    p, q, g, om, nw, nb = _setup(rng, D, N, cplx)
    x, x64 = rounded(rng.normal(size=(B, L, D)) * 1.5 + 0.3, BF)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    xn, y, cnt, mean, var, _ = _run(layer, x, G, nw, nb, out_layout=out_layout)
    assert y.shape == (B, D, L)
    assert y.stride() == ((D * L, L, 1) if out_layout == "rows" else (L * D, 1, D))
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, None, G)
    assert rel_err(host(xn), xno) < 2e-2
    assert cnt.tolist() == c.tolist()
    assert rel_err(host(mean), mu) < 1e-4 and rel_err(host(var), v) < 1e-4
    # the layer sees the rounded xn, as with two modules
    yo, _ = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om)
    _check_y(y, yo)
    # the same call as two operators
    xn2, _, mean2, var2, _, _, _ = M.ops.group_timestep_norm_fwd(x, torch.zeros(B, dtype=torch.int64, device=DEV),
                                                                 torch.zeros(B, G, device=DEV), torch.ones(B, G, device=DEV),
                                                                 dev(nw + 1), dev(nb), None, G, 1e-5, need_stats=False)
    y2, _ = layer(xn2.transpose(1, 2))
    torch.cuda.synchronize()
    assert rel_err(host(xn), host(xn2)) < 1e-2          # one bf16 step where the fp32 statistics differ in the last bits
    assert (xn != xn2).float().mean().item() < 0.02
    assert rel_err(host(y), host(y2)) < 2e-2
    assert rel_err(host(mean), host(mean2)) < 1e-5 and rel_err(host(var), host(var2)) < 1e-5


def test_config2_headline_shape():
    """B = 4, L = 4096, D = 1024, N = 16, 16 groups, bf16: the block of configs[2] as one kernel; the norm
    against the closed form in fp64, the moving average against the FFT oracle on sampled channels."""
    B, L, D, N, G = 4, 4096, 1024, 16, 16
    rng = np.random.default_rng(1236)
    p, q, g, om, nw, nb = _setup(rng, D, N)
    gen = torch.Generator().manual_seed(1236)
    x = torch.randn(B, L, D, generator=gen).to(BF).to(DEV)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    xn, y, cnt, mean, var, h = _run(layer, x, G, np.zeros(D), np.zeros(D), want_state=True)
    x64 = x.double().cpu().numpy()
    xno, mu, v = O.timestep_norm_closed_form(x64, None, G)
    assert rel_err(host(xn), xno) < 2e-2
    assert cnt.tolist() == [L] * B
    sel = np.r_[0:4, 60:68, 500:504, 1020:1024]
    xs = host(xn)[:, :, sel].transpose(0, 2, 1)
    yo, ho = O.ema_forward(xs, p[sel], q[sel], g[sel], om[sel], incremental=True)
    _check_y(y[:, sel], yo)
    assert rel_err(np.real(host(h)[:, sel]), np.real(ho)) < 2e-3
    assert rel_err(np.imag(host(h)[:, sel]), np.imag(ho)) < 2e-3
    # every channel against the two-operator route
    y2, h2 = layer(xn.transpose(1, 2), want_state=True)
    torch.cuda.synchronize()
    assert rel_err(host(y), host(y2)) < 2e-2
    assert rel_err(np.real(host(h)), np.real(host(h2))) < 2e-3


@pytest.mark.parametrize("B,L,G,cpg,out_layout,masked", [(8, 2048, 16, 64, "input", False), (4, 3072, 8, 128, "rows", True),
                                                        (4, 4000, 16, 64, "input", True), (4, 4096, 16, 64, "rows", False)])
def test_held_back_starts_change_nothing(B, L, G, cpg, out_layout, masked):
    """A launch of one round of workgroups (192 to 256 of them on 256 compute units, two to four blocks a row) holds
    back the start of every row's later blocks.  A row's result does not depend on the other rows, so the same rows
    in a call of half the batch (too few workgroups for the held-back starts) must come out bit for bit the same."""
    print(f"case B={B} L={L} G={G} cpg={cpg} out={out_layout} masked={masked}", flush=True)
    D = cpg * G
    rng = np.random.default_rng(57)
    p, q, g, om, nw, nb = _setup(rng, D, 16)
    x = torch.randn(B, L, D, generator=torch.Generator().manual_seed(57)).to(BF).to(DEV)
    mask = None
    if masked:
        mask = torch.zeros(B, L, dtype=torch.bool, device=DEV)
        for b in range(B):
            mask[b, L - 37 * (b + 1):] = True
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    h0 = torch.view_as_complex(torch.randn(B, D, 16, 2, generator=torch.Generator().manual_seed(58)).to(DEV)) if L % 1024 == 0 and not masked else None
    run = lambda xs, ms, hs: _run(layer, xs, G, nw, nb, out_layout=out_layout, padding_mask=ms, h=hs, want_state=not masked)
    full = run(x, mask, h0)
    h = B // 2
    half = run(x[:h].contiguous(), None if mask is None else mask[:h].contiguous(), None if h0 is None else h0[:h].contiguous())
    for a, b_, name in zip(full, half, ("xn", "y", "count", "mean", "var", "h")):
        if a is None:
            continue
        a = torch.view_as_real(a) if a.is_complex() else a
        b_ = torch.view_as_real(b_) if b_.is_complex() else b_
        assert torch.equal(a[:h], b_), name
    # and against the oracle on a few channels of the last row
    xn, y = full[0], full[1]
    sel = np.r_[0:3, D - 3:D]
    m = None if mask is None else host(mask)[B - 1:]
    xs = host(xn)[B - 1:, :, sel].transpose(0, 2, 1)
    hs = None if h0 is None else host(h0)[B - 1:, sel]
    yo, _ = O.ema_forward(xs, p[sel], q[sel], g[sel], om[sel], padding_mask=m, h=hs)
    _check_y(y[B - 1:, sel], yo)


@pytest.mark.parametrize("cpg", [64, 128])
@pytest.mark.parametrize("L1,L2", [(1024, 2048), (2048, 1024), (1024, 1000)])
def test_carried_state_and_prior_statistics(L1, L2, cpg):
    """Two chunks with the norm statistics and the moving-average state carried from the first call to the
    second equal one call on the whole sequence (the second chunk of the last case leaves the one-kernel
    envelope and runs as two operators out of the same workspace)."""
    B, G, N = 2, 4, 16
    D, L = cpg * G, L1 + L2
    rng = np.random.default_rng(52)
    p, q, g, om, nw, nb = _setup(rng, D, N)
    x, x64 = rounded(rng.normal(size=(B, L, D)) + 0.5, BF)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    xn1, y1, c1, m1, v1, h1 = _run(layer, x[:, :L1].contiguous(), G, nw, nb, want_state=True)
    xn2, y2, c2, m2, v2, h2 = _run(layer, x[:, L1:].contiguous(), G, nw, nb, prior=(c1, m1, v1), h=h1)
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, None, G)
    xn = torch.cat([xn1, xn2], 1)
    assert rel_err(host(xn), xno) < 2e-2
    assert c2.tolist() == [L] * B
    assert rel_err(host(m2), mu) < 1e-4 and rel_err(host(v2), v) < 1e-4
    yo, ho = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, incremental=True)
    _check_y(torch.cat([y1, y2], -1), yo)
    assert rel_err(np.real(host(h2)), np.real(ho)) < 2e-3 and rel_err(np.imag(host(h2)), np.imag(ho)) < 2e-3


@pytest.mark.parametrize("mixed", [False, True])
def test_slowly_decaying_poles_across_blocks(mixed):
    """|q| close to 1: the state a block inherits from the earlier blocks stays large (8 blocks).  `mixed`:
    every second channel decays fast instead (|q| <= 0.9)."""
    rng = np.random.default_rng(53)
    B, G, N, L = 1, 1, 16, 8192
    D = 64
    mag = 1 - 10 ** rng.uniform(-4, -1.5, size=(D, N))
    if mixed:
        mag[::2] = rng.uniform(0.5, 0.9, size=(D // 2, N))
    q = mag * np.exp(1j * rng.uniform(0, np.pi, size=(D, N)))
    p = rng.random((D, N)) * 0.5
    g = (rng.normal(size=(D, N)) + 1j * rng.normal(size=(D, N))) / 4
    om = rng.normal(size=D)
    x, x64 = rounded(rng.normal(size=(B, L, D)), BF)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    xn, y, _, _, _, h = _run(layer, x, G, np.zeros(D), np.zeros(D), want_state=True)
    yo, ho = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, incremental=True)
    # With poles this close to 1 the states are two orders of magnitude above y and cancel in the sum over the
    # states; both kernels carry them into the output product as two bf16 terms (one term left the worst element of
    # 5e5 at 2.1e-2, 2.5e-2 in the mixed case; two terms: 1.3e-2 / 1.7e-2), the rms error is 2.3e-3 of rms(y).
    _check_y(y, yo, tol=2e-2)
    e = host(y) - yo
    assert np.sqrt(np.mean(e ** 2)) < 3e-3 * np.sqrt(np.mean(yo ** 2))
    y2, _ = layer(xn.transpose(1, 2))
    torch.cuda.synchronize()
    assert rel_err(host(y2), yo) < 2e-2
    assert rel_err(host(y), host(y2)) < 2e-2
    assert rel_err(np.real(host(h)), np.real(ho)) < 2e-3


@pytest.mark.parametrize("dtype,B,L,D,G,masked", [(BF, 2, 700, 128, 2, False), (BF, 2, 1000, 128, 2, True),
                                                  (torch.float32, 1, 1024, 64, 1, False), (BF, 1, 2048, 96, 3, False)])
def test_outside_the_envelope_runs_two_operators(dtype, B, L, D, G, masked):
    rng = np.random.default_rng(54)
    N = 16
    p, q, g, om, nw, nb = _setup(rng, D, N)
    x, x64 = rounded(rng.normal(size=(B, L, D)), dtype)
    mask = None
    if masked:
        mask = np.zeros((B, L), bool)
        mask[0, L - 100:] = True
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    tm = None if mask is None else dev(mask, torch.bool)
    xn, y, cnt, mean, var, _ = _run(layer, x, G, nw, nb, padding_mask=tm)
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, mask, G)
    tol = M_TOL[dtype]
    assert rel_err(host(xn), xno) < tol
    assert cnt.tolist() == c.tolist()
    yo, _ = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, mask)
    assert rel_err(host(y), yo) < tol


M_TOL = {torch.float32: 1e-4, BF: 2e-2}


@pytest.mark.parametrize("L,out_layout,masked", [(1000, "rows", False), (1032, "rows", True), (2056, "input", False),
                                                 (3001, "input", True), (300, "input", False), (8, "rows", False),
                                                 (1, "input", False), (5000, "rows", False)])
@pytest.mark.parametrize("cpg", [64, 128])
def test_one_kernel_rows_of_any_length(L, out_layout, masked, cpg):
    """Rows that are not whole blocks of 1024 tokens: the block grid is aligned to the end of the row (the first block
    starts before the row), so the state handed back is the state after the last token -- what a prompt of any length
    needs before decoding continues from it.  Statistics carried in, state out, both layouts (rows in time need a length
    that is a multiple of 8), with and without padding; the continuation of the row by a second call (two operators:
    it carries a state in) agrees with one call on the whole."""
    print(f"case L={L} out={out_layout} masked={masked} cpg={cpg}", flush=True)
    B, G, N = 2, 2, 16
    D = cpg * G
    rng = np.random.default_rng(58)
    p, q, g, om, nw, nb = _setup(rng, D, N)
    L2 = 64
    x, x64 = rounded(rng.normal(size=(B, L + L2, D)) * 1.2 + 0.4, BF)
    mask = None
    if masked:
        mask = np.zeros((B, L + L2), bool)
        mask[0, max(L - 40, 0):L] = True
        mask[1, :min(10, L)] = True
        mask[1, L // 2] = True
    pc = np.array([5, 0])
    pm = rng.normal(size=(B, G)).astype(np.float32).astype(np.float64)
    pv = (rng.random((B, G)) + 0.5).astype(np.float32).astype(np.float64)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    tm = None if mask is None else dev(mask[:, :L], torch.bool)
    xn, y, cnt, mean, var, h = _run(layer, x[:, :L].contiguous(), G, nw, nb,
                                    prior=(dev(pc, torch.int64), dev(pm), dev(pv)), padding_mask=tm,
                                    out_layout=out_layout, want_state=True)
    assert y.shape == (B, D, L)
    xno, c, mu, v = O.timestep_norm(x64, pc, pm, pv, nw + 1, nb, mask, G)
    assert rel_err(host(xn), xno[:, :L]) < 2e-2
    m1 = None if mask is None else mask[:, :L]
    _, c1, mu1, v1 = O.timestep_norm(x64[:, :L], pc, pm, pv, nw + 1, nb, m1, G)
    assert cnt.tolist() == c1.tolist()
    assert rel_err(host(mean), mu1) < 1e-4 and rel_err(host(var), v1) < 1e-4
    yo, ho = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, m1, incremental=True)
    _check_y(y, yo)
    assert rel_err(np.real(host(h)), np.real(ho)) < 2e-3 and rel_err(np.imag(host(h)), np.imag(ho)) < 2e-3
    # the row continues: statistics and state carried into a second call
    tm2 = None if mask is None else dev(mask[:, L:], torch.bool)
    xn2, y2, c2, _, _, _ = _run(layer, x[:, L:].contiguous(), G, nw, nb, prior=(cnt, mean, var), h=h, padding_mask=tm2,
                                out_layout=out_layout)
    assert rel_err(host(xn2), xno[:, L:]) < 2e-2 and c2.tolist() == c.tolist()
    yo2, _ = O.ema_forward(host(torch.cat([xn, xn2], 1)).transpose(0, 2, 1), p, q, g, om, mask)
    _check_y(y2, yo2[:, :, L:])


@pytest.mark.parametrize("out_layout", ["rows", "input"])
@pytest.mark.parametrize("B,L,G,cpg,affine", [(3, 3072, 2, 64, True), (2, 2048, 1, 128, False), (4, 1024, 8, 64, True)])
def test_one_kernel_with_padding_mask(out_layout, B, L, G, cpg, affine):
    """Padding inside the one-kernel envelope: masked tokens take no part in the running statistics and leave the norm
    as zeros (timestep_norm.cc:283-311), the moving average sees those zeros.  The masks: a padded tail, a row that
    starts padded, a whole block of 1024 padded tokens in the middle of a row, single tokens, a row of nothing but
    padding, and a row without padding."""
    print(f"case out={out_layout} B={B} L={L} G={G} cpg={cpg} affine={affine}", flush=True)
    D, N = cpg * G, 16
    rng = np.random.default_rng(57)
    p, q, g, om, nw, nb = _setup(rng, D, N)
    if not affine:
        nw, nb = np.zeros(D), np.zeros(D)
    x, x64 = rounded(rng.normal(size=(B, L, D)) * 1.3 - 0.2, BF)
    mask = np.zeros((B, L), bool)
    mask[0, L - 300:] = True
    mask[1, :70] = True
    mask[1, 500:503] = True
    if B > 2 and L >= 3072:
        mask[2, 1024:2048] = True
    mask[-1, ::97] |= B > 3
    if B > 3:
        mask[2, :] = True                                  # a row of nothing but padding: the prior statistics come back
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    xn, y, cnt, mean, var, h = _run(layer, x, G, nw, nb, padding_mask=dev(mask, torch.bool), out_layout=out_layout,
                                    want_state=True)
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, mask, G)
    assert rel_err(host(xn), xno) < 2e-2
    assert np.array_equal(host(xn)[mask], np.zeros_like(host(xn)[mask]))
    assert cnt.tolist() == c.tolist()
    assert rel_err(host(mean), mu) < 1e-4 and rel_err(host(var), v) < 1e-4
    yo, ho = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, mask, incremental=True)
    _check_y(y, yo)
    assert rel_err(np.real(host(h)), np.real(ho)) < 2e-3 and rel_err(np.imag(host(h)), np.imag(ho)) < 2e-3
    # and the two operators on the same input
    xn2 = M.ops.group_timestep_norm_fwd(x, torch.zeros(B, dtype=torch.int64, device=DEV), torch.zeros(B, G, device=DEV),
                                        torch.ones(B, G, device=DEV), dev(nw + 1), dev(nb), dev(mask, torch.bool), G, 1e-5,
                                        need_stats=False)[0]
    y2, _ = layer(xn2.transpose(1, 2), dev(mask, torch.bool))
    torch.cuda.synchronize()
    assert rel_err(host(xn), host(xn2)) < 1e-2 and rel_err(host(y), host(y2)) < 2e-2


def test_kernel_generation_inside_the_call():
    """image = NULL: the operand images are generated into the workspace by the same call."""
    B, L, G, N = 2, 2048, 2, 16
    D = 64 * G
    rng = np.random.default_rng(55)
    p, q, g, om, nw, nb = _setup(rng, D, N)
    x, x64 = rounded(rng.normal(size=(B, L, D)), BF)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    ref = _run(layer, x, G, nw, nb)
    saved, layer.image = layer.image, None
    got = _run(layer, x, G, nw, nb)
    layer.image = saved
    assert torch.equal(ref[0], got[0]) and torch.equal(ref[1], got[1])


def test_module_pair_keeps_both_incremental_states():
    """norm_then_move(norm, move, x, ...) equals the two modules called one after the other, chunk by chunk with
    incremental state (1024 tokens in one kernel, then 300 as two operators, then a single token)."""
    B, G, N = 2, 2, 16
    D = 64 * G
    torch.manual_seed(56)
    norm = M.TimestepNorm(D, G).to(DEV).eval()
    move = M.MultiHeadComplexEMA(D, ndim=N).to(DEV).eval()
    with torch.no_grad():
        norm.weight.normal_(0, 0.1)
        norm.bias.normal_(0, 0.1)
    x = torch.randn(B, 1325, D, device=DEV).to(BF)
    inc_a, inc_b = {}, {}
    with torch.no_grad():
        for lo, hi in ((0, 1024), (1024, 1324), (1324, 1325)):
            xc = x[:, lo:hi].contiguous()
            xn_a, y_a = M.norm_then_move(norm, move, xc, None, inc_a, out_layout="input")
            xn_b = norm(xc, incremental_state=inc_b)
            y_b = move(xn_b.transpose(1, 2), None, inc_b, out_layout="input")
            torch.cuda.synchronize()
            assert y_a.shape == y_b.shape == (B, D, hi - lo)
            assert rel_err(host(xn_a), host(xn_b)) < 1e-2
            assert rel_err(host(y_a), host(y_b)) < 2e-2
    sa, sb = norm._get_input_buffer(inc_a), norm._get_input_buffer(inc_b)
    assert sa['prev_count'].tolist() == sb['prev_count'].tolist() == [1325] * B
    assert rel_err(host(sa['prev_mean']), host(sb['prev_mean'])) < 1e-5
    assert rel_err(host(sa['prev_var']), host(sb['prev_var'])) < 1e-5
    ha, hb = move._get_input_buffer(inc_a)['prev_state'], move._get_input_buffer(inc_b)['prev_state']
    assert rel_err(np.real(host(ha)), np.real(host(hb))) < 2e-3
    # with autograd the pair is one differentiable operator
    xg = x[:, :64].float().requires_grad_(True)
    xn_g, y_g = M.norm_then_move(norm, move, xg)
    assert y_g.requires_grad and xn_g.requires_grad


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.float16, 4e-3)])
@pytest.mark.parametrize("out_layout,masked", [("rows", False), ("input", True)])
def test_fp32_fp16_two_slices_with_state(dtype, tol, out_layout, masked):
    """fp32 / fp16 activations: the norm, then the moving average on rows in time through a transposition each way.
    Two slices of a row (1024 + 2048 tokens, the state of both operators carried across) against the oracle on the
    whole row, in both output layouts, with padded tails."""
    print(f"case dtype={dtype} out={out_layout} masked={masked}", flush=True)
    B, G, N, D, L1, L2 = 2, 4, 16, 256, 1024, 2048
    L = L1 + L2
    rng = np.random.default_rng(57)
    p, q, g, om, nw, nb = _setup(rng, D, N)
    x, x64 = rounded(rng.normal(size=(B, L, D)) + 0.5, dtype)
    mask = tm = None
    if masked:
        mask = np.zeros((B, L), bool)
        mask[1, L - 300:] = True
        tm = dev(mask, torch.bool)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    m1 = None if tm is None else tm[:, :L1].contiguous()
    m2 = None if tm is None else tm[:, L1:].contiguous()
    xn1, y1, c1, mu1, v1, h1 = _run(layer, x[:, :L1].contiguous(), G, nw, nb, want_state=True, out_layout=out_layout,
                                    padding_mask=m1)
    xn2, y2, c2, mu2, v2, h2 = _run(layer, x[:, L1:].contiguous(), G, nw, nb, prior=(c1, mu1, v1), h=h1,
                                    out_layout=out_layout, padding_mask=m2)
    assert y2.shape == (B, D, L2)
    assert y2.stride() == ((D * L2, L2, 1) if out_layout == "rows" else (L2 * D, 1, D))
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, mask, G)
    xn = torch.cat([xn1, xn2], 1)
    assert rel_err(host(xn), xno) < tol
    assert c2.tolist() == c.tolist()
    assert rel_err(host(mu2), mu) < 1e-4 and rel_err(host(v2), v) < 1e-4
    yo, ho = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, mask, incremental=True)
    assert rel_err(host(torch.cat([y1, y2], -1)), yo) < tol
    assert rel_err(np.real(host(h2)), np.real(ho)) < 1e-3 and rel_err(np.imag(host(h2)), np.imag(ho)) < 1e-3


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-4), (torch.float16, 4e-3)])
def test_fp32_fp16_ragged_row_and_training_statistics(dtype, tol):
    """A row that is no whole number of blocks (no state asked for) with the statistics a training forward keeps."""
    B, G, N, D, L = 2, 2, 16, 128, 1500
    rng = np.random.default_rng(58)
    p, q, g, om, nw, nb = _setup(rng, D, N)
    x, x64 = rounded(rng.normal(size=(B, L, D)) * 1.2 - 0.2, dtype)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
    xn, y, cnt, mean, var, h, cm, cr = _run(layer, x, G, nw, nb, want_stats=True)
    assert h is None and cm.shape == (B, L, G) and cr.shape == (B, L, G)
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, None, G)
    assert rel_err(host(xn), xno) < tol
    assert cnt.tolist() == c.tolist()
    assert rel_err(host(cm)[:, -1], mu) < 1e-4
    assert rel_err(host(cr)[:, -1], 1.0 / np.sqrt(v + 1e-5)) < 1e-4
    yo, _ = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om)
    assert rel_err(host(y), yo) < tol
