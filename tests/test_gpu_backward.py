"""Backward kernels on the GPU against the fp64 oracle's backward restatements (which the CPU
suite pins by finite differences of the oracle's forward and by the reference's own CPU
operators' outputs in tests/golden)."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, rel_err
from gpu_util import DEV, TOL, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu


def _tsn_case(rng, B, L, H, G, masked, prior, dtype):
    GG = H if G is None else G
    x, x64 = rounded(rng.normal(size=(B, L, H)) * 1.3 + 0.2, dtype)
    dy, dy64 = rounded(rng.normal(size=(B, L, H)), dtype)
    mask = (rng.random((B, L)) < 0.25) if masked else None
    pc = rng.integers(1, 5, B).astype(np.int64) if prior else np.zeros(B, np.int64)
    pm = (rng.normal(size=(B, GG)) * 0.2 * prior).astype(np.float32).astype(np.float64)
    pv = (rng.random((B, GG)) + 0.5 if prior else np.ones((B, GG))).astype(np.float32).astype(np.float64)
    gamma = (rng.normal(size=H) * 0.3 + 1).astype(np.float32).astype(np.float64)
    beta = rng.normal(size=H).astype(np.float32).astype(np.float64)
    dm = rng.normal(size=(B, GG)).astype(np.float32).astype(np.float64)
    dv = rng.normal(size=(B, GG)).astype(np.float32).astype(np.float64)
    return x, x64, dy, dy64, mask, pc, pm, pv, gamma, beta, dm, dv


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,H,G,masked,prior", [
    (2, 37, 64, 4, True, True),        # ragged tile, interior padding, carried statistics
    (3, 130, 128, 16, False, False),   # several tiles per row, 8 channels per group
    (1, 96, 1024, 16, False, False),   # the headline geometry (64 channels per group)
    (2, 50, 48, 2, True, False),       # 24 channels per group: three vectors per lane
    (2, 33, 30, 5, True, True),        # 6 channels per group: element-wise path
    (2, 45, 24, None, True, True),     # per-feature statistics
    (2, 300, 1100, None, True, True),  # per-feature, three blocks of 512 channels (the last partial), five tiles of 64 tokens
    (1, 130, 25, None, False, False),  # per-feature with an odd number of channels: the group form with one channel a group
])
def test_timestep_norm_bwd(dtype, B, L, H, G, masked, prior):
    rng = np.random.default_rng(51)
    x, x64, dy, dy64, mask, pc, pm, pv, gamma, beta, dm, dv = _tsn_case(rng, B, L, H, G, masked, prior, dtype)
    tm = None if mask is None else torch.from_numpy(mask).to(DEV)
    if G is None:
        y, cnt, mu, var, cm, cr = M.ops.timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma),
                                                          dev(beta), tm, 1e-5)
        got = M.ops.timestep_norm_bwd(dy, dev(dm), dev(dv), x, dev(pm), cnt, cm, cr, dev(gamma), tm)
    else:
        y, cnt, mu, var, gm, cm, cr = M.ops.group_timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv),
                                                                    dev(gamma), dev(beta), tm, G, 1e-5)
        got = M.ops.group_timestep_norm_bwd(dy, dev(dm), dev(dv), x, dev(pm), cnt, gm, cm, cr, dev(gamma), tm, G)
        # without the saved group means the kernel recomputes them
        got2 = M.ops.group_timestep_norm_bwd(dy, dev(dm), dev(dv), x, dev(pm), cnt, None, cm, cr, dev(gamma), tm, G)
        assert rel_err(host(got2[0]), host(got[0])) < 1e-5
    ocnt, ogm, ocm, ocr = O.timestep_norm_saved(x64, pc, pm, pv, mask, G, 1e-5)
    assert np.array_equal(host(cnt), ocnt)
    ref = O.timestep_norm_bwd(dy64, dm, dv, x64, pm, ocnt, ogm if G else None, ocm, ocr, gamma, mask, G)
    tol = TOL[dtype]
    assert rel_err(host(got[0]), ref[0]) < tol                       # dx, rounded once to the activation type
    for a, b in zip(got[1:], ref[1:]):                                # fp32 sums over tokens / channels
        assert rel_err(host(a), b) < 2e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,H,G,masked,prior,saved_gm", [
    (4, 4096, 1024, 16, False, False, True),    # the headline geometry: 128 tiles a row, block records of 16 tiles
    (2, 2000, 1024, 16, True, True, False),     # ragged last tile, padding, carried statistics, group means formed again
    (1, 8192, 2048, 16, False, True, True),     # 128 channels per group: tiles of 16 tokens, 512 tiles a row
    (3, 700, 128, 16, True, False, True),       # one vector per group, 22 tiles: look-back over the tiles themselves
    (2, 1030, 256, 2, True, True, False),       # two groups of 128 channels
    (5, 31, 64, 1, False, True, True),          # a single partial tile
])
def test_timestep_norm_bwd_one_launch(dtype, B, L, H, G, masked, prior, saved_gm):
    """The one-launch form (every tile composes the maps of the tiles behind it) against the three-pass form on the
    same inputs, and against the oracle where that is quick."""
    print(f"case {dtype} B={B} L={L} H={H} G={G} masked={masked} prior={prior} saved_gm={saved_gm}", flush=True)
    rng = np.random.default_rng(53)
    x, x64, dy, dy64, mask, pc, pm, pv, gamma, beta, dm, dv = _tsn_case(rng, B, L, H, G, masked, prior, dtype)
    tm = None if mask is None else torch.from_numpy(mask).to(DEV)
    y, cnt, mu, var, gm, cm, cr = M.ops.group_timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma),
                                                                dev(beta), tm, G, 1e-5)
    run = lambda: M.ops.group_timestep_norm_bwd(dy, dev(dm), dev(dv), x, dev(pm), cnt, gm if saved_gm else None, cm, cr,
                                                dev(gamma), tm, G)
    lib = M._lib.load()
    one = run()
    torch.cuda.synchronize()
    assert M.ops.lookback_status() == 0
    lib.mega_test_timestep_norm_bwd_onepass(0)
    try:
        three = run()
        torch.cuda.synchronize()
    finally:
        lib.mega_test_timestep_norm_bwd_onepass(1)
    assert not torch.isnan(one[0].float()).any()
    # fp32 walks composed in another order, dx rounded once to the activation type: the odd last-bit difference
    assert rel_err(host(one[0]), host(three[0])) < 1e-2
    assert (one[0] != three[0]).float().mean().item() < 0.02
    for a, b_ in zip(one[1:], three[1:]):
        assert rel_err(host(a), host(b_)) < 1e-4
    if B * L * H <= 2 * 2000 * 1024:
        ocnt, ogm, ocm, ocr = O.timestep_norm_saved(x64, pc, pm, pv, mask, G, 1e-5)
        ref = O.timestep_norm_bwd(dy64, dm, dv, x64, pm, ocnt, ogm, ocm, ocr, gamma, mask, G)
        assert rel_err(host(one[0]), ref[0]) < TOL[dtype]
        for a, b_ in zip(one[1:], ref[1:]):
            assert rel_err(host(a), b_) < 3e-4


def test_timestep_norm_bwd_zero_upstream_state_grads():
    rng = np.random.default_rng(52)
    x, x64, dy, dy64, mask, pc, pm, pv, gamma, beta, _, _ = _tsn_case(rng, 2, 40, 32, 4, False, True, torch.float32)
    y, cnt, mu, var, gm, cm, cr = M.ops.group_timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma),
                                                                dev(beta), None, 4, 1e-5)
    got = M.ops.group_timestep_norm_bwd(dy, None, None, x, dev(pm), cnt, gm, cm, cr, dev(gamma), None, 4)
    ocnt, ogm, ocm, ocr = O.timestep_norm_saved(x64, pc, pm, pv, None, 4, 1e-5)
    ref = O.timestep_norm_bwd(dy64, None, None, x64, pm, ocnt, ogm, ocm, ocr, gamma, None, 4)
    for a, b in zip(got, ref):
        assert rel_err(host(a), b) < 2e-4


@pytest.mark.parametrize("groups,prior_count", [(8, 0), (None, 2), (4, 3)])
def test_timestep_norm_module_autograd(groups, prior_count):
    """loss = sum(y * w): gradients of x, weight, bias (and the prior when it is a parameter)."""
    rng = np.random.default_rng(53)
    B, L, H = 2, 70, 32
    mod = M.TimestepNorm(H, groups, prior_count=prior_count).to(DEV).train()
    with torch.no_grad():
        mod.weight.normal_(0, 0.2); mod.bias.normal_(0, 0.2)
        if prior_count > 0:
            mod.prior_mean.normal_(0, 0.2); mod.prior_logv.normal_(0, 0.2)
    x64 = rng.normal(size=(B, L, H)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, L, H)).astype(np.float32).astype(np.float64)
    x = dev(x64).requires_grad_(True)
    y = mod(x)
    (y * dev(w64)).sum().backward()
    G = H if groups is None else groups
    pc = np.full(B, prior_count, np.int64)
    pm = np.broadcast_to(host(mod.prior_mean), (B, G)).copy()
    pv = np.broadcast_to(np.exp(host(mod.prior_logv)), (B, G)).copy()
    gamma = host(mod.weight) + 1.0
    ocnt, ogm, ocm, ocr = O.timestep_norm_saved(x64, pc, pm, pv, None, groups, 1e-5)
    dx, dpm, dpv, dg, db = O.timestep_norm_bwd(w64, None, None, x64, pm, ocnt, ogm if groups else None, ocm, ocr,
                                               gamma, None, groups)
    assert rel_err(host(x.grad), dx) < 2e-4
    assert rel_err(host(mod.weight.grad), dg) < 2e-4 and rel_err(host(mod.bias.grad), db) < 2e-4
    if prior_count > 0:
        assert rel_err(host(mod.prior_mean.grad), dpm.sum(0)) < 2e-4
        assert rel_err(host(mod.prior_logv.grad), (dpv * pv).sum(0)) < 2e-4


@pytest.mark.parametrize("dtype,B,L,D,G,N,masked,layout", [
    (torch.bfloat16, 2, 1024, 128, 2, 16, False, "rows"),      # one kernel, one block
    (torch.bfloat16, 1, 2048, 256, 2, 16, False, "input"),     # groups of 128 channels, two blocks
    (torch.bfloat16, 2, 1000, 64, 1, 8, True, "input"),        # ragged row with padding
    (torch.float32, 2, 70, 32, 4, 4, True, "rows"),            # outside the one-kernel envelope
])
def test_norm_then_move_trains_as_one_operator(dtype, B, L, D, G, N, masked, layout):
    """norm_then_move under autograd is one operator whose forward is the one-kernel block (with the norm's
    running statistics kept); gradients of x and of every parameter of both modules against the two modules'
    own operators one after the other, and the kept statistics against the fp64 oracle."""
    rng = np.random.default_rng(71)
    torch.manual_seed(17)
    norm = M.TimestepNorm(D, G, prior_count=2).to(DEV).train()
    move = M.MultiHeadComplexEMA(D, ndim=N).to(DEV).train()
    with torch.no_grad():
        norm.weight.normal_(0, 0.2); norm.bias.normal_(0, 0.2)
        norm.prior_mean.normal_(0, 0.2); norm.prior_logv.normal_(0, 0.2)
    x0 = torch.randn(B, L, D, device=DEV).mul_(1.3).add_(0.2).to(dtype)
    w1 = torch.randn(B, L, D, device=DEV).to(dtype)
    w2 = torch.randn(B, D, L, device=DEV).to(dtype)
    mask = None
    if masked:
        mask = torch.from_numpy(rng.random((B, L)) < 0.2).to(DEV)
    params = list(norm.parameters()) + list(move.parameters())

    def run(enabled):
        for q in params:
            q.grad = None
        x = x0.clone().requires_grad_(True)
        M.modules.NormThenMoveFunc.ENABLED = enabled
        try:
            xn, y = M.norm_then_move(norm, move, x, mask, None, out_layout=layout)
        finally:
            M.modules.NormThenMoveFunc.ENABLED = True
        assert y.shape == (B, D, L) and (layout == "rows") == y.is_contiguous()
        ((xn * w1).sum() + (y * w2).sum()).backward()
        torch.cuda.synchronize()
        return xn.detach(), y.detach(), x.grad, [None if q.grad is None else q.grad.clone() for q in params]

    xn_a, y_a, dx_a, g_a = run(True)
    xn_b, y_b, dx_b, g_b = run(False)
    tol = 2e-4 if dtype == torch.float32 else 3e-2
    assert rel_err(host(xn_a), host(xn_b)) < tol and rel_err(host(y_a), host(y_b)) < tol
    assert rel_err(host(dx_a), host(dx_b)) < tol
    for (name, _), ga, gb in zip(list(norm.named_parameters()) + list(move.named_parameters()), g_a, g_b):
        assert (ga is None) == (gb is None), name
        if ga is not None:
            assert rel_err(host(ga), host(gb)) < tol, name

    # the statistics the one call keeps for the backward pass
    layer = move._prepared_layer()
    pc, pm, pv = norm._prior_state(B)
    with torch.no_grad():
        out = layer.norm_forward(x0, pc, pm, pv, norm.weight.float() + 1.0, norm.bias.float(), G, norm.eps, mask,
                                 None, want_stats=True)
    x64 = host(x0)
    m64 = None if mask is None else host(mask).astype(bool)
    ocnt, _, ocm, ocr = O.timestep_norm_saved(x64, host(pc).astype(np.int64), host(pm), host(pv), m64, G, norm.eps)
    assert host(out[2]).tolist() == ocnt.tolist()
    assert rel_err(host(out[6]), ocm) < 1e-4 and rel_err(host(out[7]), ocr) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("cplx,K,N,D", [(True, 24, 16, 24), (True, 10, 3, 5), (True, 6, 80, 6), (True, 2048, 16, 2048),
                                         (False, 12, 4, 12), (False, 8, 2, 4)])
def test_coefficient_kernels(dtype, cplx, K, N, D):
    """The layer's coefficients from its parameters in one launch, forwards against the fp64 oracle's formulas and
    backwards against torch's autograd of the same formulas in fp64 on the CPU (random upstream gradients)."""
    rng = np.random.default_rng(77)
    alpha, a64 = rounded(rng.normal(0, 0.4, (K, N, 1)), dtype)
    delta, d64 = rounded(rng.normal(0, 0.4, (K, N, 1)), dtype)
    omega, o64 = rounded(rng.normal(size=(D, 1) if cplx else (D,)), dtype)
    if cplx:
        third, t64 = rounded(rng.normal(0, 1.5, (K, 1, 1)), dtype)
        gamma, g64 = rounded(rng.normal(size=(K, N, 2)), dtype)
        po, qo, go = O.ema_coeffs_complex(a64, d64, t64, g64)
    else:
        third, t64 = rounded(rng.normal(0, 1.0, (K, N, 1)), dtype)
        gamma, g64 = rounded(rng.normal(size=(K, N)), dtype)
        po, qo, go = O.ema_coeffs_real(a64, d64, t64, g64)
    p, q2, g2, om = M.ops.ema_coeffs_fwd(alpha, delta, third, gamma, omega, cplx)
    assert p.dtype == q2.dtype == g2.dtype == om.dtype == torch.float32
    assert rel_err(host(p), po.reshape(K, N)) < 2e-6
    qo, go = np.asarray(qo, np.complex128).reshape(K, N), np.asarray(go, np.complex128).reshape(K, N)
    assert rel_err(host(q2), np.stack([qo.real, qo.imag], -1)) < 2e-6
    assert rel_err(host(g2), np.stack([go.real, go.imag], -1)) < 2e-6
    assert np.array_equal(host(om), o64.reshape(-1))
    # backward: arbiter = autograd of the formulas in fp64
    ta, td, tt, tg = (torch.from_numpy(v).requires_grad_(True) for v in (a64, d64, t64, g64))
    sa, sd = torch.sigmoid(ta), torch.sigmoid(td)
    up = [rng.normal(size=(K, N)), rng.normal(size=(K, N, 2)), rng.normal(size=(K, N, 2)), rng.normal(size=D)]
    up = [u.astype(np.float32).astype(np.float64) for u in up]
    if cplx:
        ang = torch.arange(1, N + 1, dtype=torch.float64).view(1, N, 1) * torch.sigmoid(tt) * (2 * np.pi / N)
        r = 1 - sa * sd
        qre, qim = (r * torch.cos(ang)).squeeze(-1), (r * torch.sin(ang)).squeeze(-1)
        gs = tg / np.sqrt(N)
        loss = (sa.squeeze(-1) * torch.from_numpy(up[0])).sum() + (qre * torch.from_numpy(up[1][..., 0])).sum() + \
            (qim * torch.from_numpy(up[1][..., 1])).sum() + (gs * torch.from_numpy(up[2])).sum()
        gq, gg = dev(up[1]), dev(up[2])
    else:
        loss = ((sa * tt).squeeze(-1) * torch.from_numpy(up[0])).sum() + \
            ((1 - sa * sd).squeeze(-1) * torch.from_numpy(up[1][..., 0])).sum() + \
            (tg / np.sqrt(N) * torch.from_numpy(up[2][..., 0])).sum()
        gq, gg = dev(up[1][..., 0].copy()), dev(up[2][..., 0].copy())
    loss.backward()
    da, dd, dt, dg, dom = M.ops.ema_coeffs_bwd(dev(up[0]), gq, gg, dev(up[3]), alpha, delta, third, gamma, omega, cplx)
    assert da.dtype == dd.dtype == dt.dtype == dg.dtype == dom.dtype == dtype
    assert da.shape == alpha.shape and dt.shape == third.shape and dg.shape == gamma.shape and dom.shape == omega.shape
    tol = TOL[dtype] if dtype != torch.float32 else 1e-5
    for got, ref in ((da, ta.grad), (dd, td.grad), (dt, tt.grad), (dg, tg.grad)):
        assert rel_err(host(got), ref.numpy()) < tol
    assert rel_err(host(dom).reshape(-1), up[3]) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,B,learned", [(64, 4, 3, True), (40, 40, 2, True), (32, 8, 1, False)])
def test_norm_parameter_kernels(dtype, H, G, B, learned):
    """weight + 1, bias, the prior over the batch: values, and parameter gradients with the sums over the batch."""
    rng = np.random.default_rng(78)
    w, w64 = rounded(rng.normal(0, 0.3, H), dtype)
    b, b64 = rounded(rng.normal(0, 0.3, H), dtype)
    pm, pm64 = rounded(rng.normal(0, 0.3, G), dtype)
    pl, pl64 = rounded(rng.normal(0, 0.3, G), dtype)
    gamma, beta, mean, var = M.ops.norm_params_fwd(w, b, pm, pl, B)
    assert np.allclose(host(gamma), w64 + 1, rtol=1e-6, atol=0) and np.array_equal(host(beta), b64)
    assert np.array_equal(host(mean), np.broadcast_to(pm64, (B, G)))
    assert rel_err(host(var), np.broadcast_to(np.exp(pl64), (B, G))) < 1e-6
    up = [rng.normal(size=s).astype(np.float32).astype(np.float64) for s in ((H,), (H,), (B, G), (B, G))]
    dw, db, dpm, dpl = M.ops.norm_params_bwd(dev(up[0]), dev(up[1]), dev(up[2]), dev(up[3]), w, pm, pl, B, learned)
    tol = 1e-6 if dtype == torch.float32 else TOL[dtype]
    assert dw.dtype == dtype and rel_err(host(dw), up[0]) < tol and rel_err(host(db), up[1]) < tol
    if learned:
        assert rel_err(host(dpm), up[2].sum(0)) < tol
        assert rel_err(host(dpl), up[3].sum(0) * np.exp(pl64)) < tol
    else:
        assert dpm is None and dpl is None


# ----------------------------------------------------------------------------------------------
# moving-average layer
# ----------------------------------------------------------------------------------------------
def _ema_coeffs(rng, D, N, cplx):
    if cplx:
        return O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    alpha, delta = rng.normal(size=(D, N)) * 0.2, rng.normal(size=(D, N)) * 0.2
    beta = rng.normal(size=(D, N)) * 0.02 + np.where(np.arange(N) % 2 == 0, 1.0, -1.0)
    return O.ema_coeffs_real(alpha, delta, beta, rng.normal(size=(D, N)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,D,N,L,cplx,layout,masked", [
    (2, 32, 16, 2048, True, "bld", False),    # matrix-core path backwards in time, channels contiguous
    (1, 16, 16, 1024, True, "bdl", False),    # rows in time: flipped through a copy
    (2, 24, 16, 300, True, "bld", True),      # generic path, padding
    (3, 20, 2, 77, False, "bdl", True),       # real layer, two states
    (2, 40, 7, 129, True, "bld", False),      # odd state count
    (2, 16, 16, 1544, True, "mixed", False),  # x with channels contiguous, dy with rows in time; a partial last step
    (1, 8, 16, 520, False, "bdl", False),     # real coefficients on the matrix-core sums
])
def test_ema_backward(dtype, B, D, N, L, cplx, layout, masked):
    rng = np.random.default_rng(61)
    p, q, g = _ema_coeffs(rng, D, N, cplx)
    p, g = p.astype(np.float32).astype(np.float64), (g.astype(np.complex64).astype(np.complex128) if cplx else
                                                      g.astype(np.float32).astype(np.float64))
    q = q.astype(np.complex64).astype(np.complex128) if cplx else q.astype(np.float32).astype(np.float64)
    om = rng.normal(size=D).astype(np.float32).astype(np.float64)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    dy, dy64 = rounded(rng.normal(size=(B, D, L)), dtype)
    if layout in ("bld", "mixed"):
        x = x.transpose(1, 2).contiguous().transpose(1, 2)
    if layout == "bld":
        dy = dy.transpose(1, 2).contiguous().transpose(1, 2)
    mask = (rng.random((B, L)) < 0.2) if masked else None
    tm = None if mask is None else torch.from_numpy(mask).to(DEV)
    got = M.ops.ema_backward(dy, x, dev(p), dev(q), dev(g), dev(om), tm)
    ref = O.ema_backward(dy64, x64, p, q, g, om, mask)
    assert got[0].stride() == dy.stride()
    # dx is one moving average of dy: same bound as the forward layer
    assert rel_err(host(got[0]), ref[0]) < TOL[dtype]
    for a, b, name in zip(got[1:], ref[1:], ("dp", "dq", "dgamma", "domega")):
        a = host(a)
        if np.iscomplexobj(b):
            assert rel_err(a.real, b.real) < 5e-4 and rel_err(a.imag, b.imag) < 5e-4, name
        else:
            assert rel_err(a, np.real(b)) < 5e-4, name


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,D,N,L,shift,layout,masked", [
    (2, 32, 16, 2048, True, "bld", False),    # matrix-core path, both directions
    (2, 24, 16, 300, True, "bld", True),
    (1, 16, 4, 150, False, "bdl", True),      # backward kernel with its lag-0 tap
    (2, 32, 16, 1100, False, "bld", False),   # lag-0 tap, no padding: the reversed half on the matrix-core sums
])
def test_ema_backward_two_sided(dtype, B, D, N, L, shift, layout, masked):
    rng = np.random.default_rng(63)
    p, q, g = _ema_coeffs(rng, 2 * D, N, True)
    p, q, g = p.astype(np.float32).astype(np.float64), q.astype(np.complex64).astype(np.complex128), \
        g.astype(np.complex64).astype(np.complex128)
    om = rng.normal(size=D).astype(np.float32).astype(np.float64)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    dy, dy64 = rounded(rng.normal(size=(B, D, L)), dtype)
    if layout == "bld":
        x = x.transpose(1, 2).contiguous().transpose(1, 2)
        dy = dy.transpose(1, 2).contiguous().transpose(1, 2)
    mask = (rng.random((B, L)) < 0.2) if masked else None
    tm = None if mask is None else torch.from_numpy(mask).to(DEV)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om), True, None, shift)
    got = M.ops.ema_backward(dy, x, dev(p), dev(q), dev(g), dev(om), tm, layer=layer)
    ref = O.ema_backward(dy64, x64, p, q, g, om, mask, True, shift)
    assert rel_err(host(got[0]), ref[0]) < TOL[dtype]
    for a, b, name in zip(got[1:], ref[1:], ("dp", "dq", "dgamma", "domega")):
        a = host(a)
        if np.iscomplexobj(b):
            assert rel_err(a.real, b.real) < 5e-4 and rel_err(a.imag, b.imag) < 5e-4, name
        else:
            assert rel_err(a, np.real(b)) < 5e-4, name


def test_two_sided_module_autograd():
    rng = np.random.default_rng(64)
    B, D, N, L = 2, 16, 8, 80
    torch.manual_seed(6)
    mod = M.MultiHeadComplexEMA(D, ndim=N, bidirectional=True).to(DEV).train()
    x64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    x = dev(x64).requires_grad_(True)
    (mod(x) * dev(w64)).sum().backward()
    P = {n: host(getattr(mod, n)) for n in ("alpha", "delta", "theta", "gamma", "omega")}

    def loss(Pd):
        p, q, g = O.ema_coeffs_complex(Pd["alpha"], Pd["delta"], Pd["theta"], Pd["gamma"])
        return (O.ema_forward(x64, p, q, g, Pd["omega"].reshape(-1), bidirectional=True)[0] * w64).sum()

    eps = 1e-5
    for n in P:
        grad = host(getattr(mod, n).grad)
        scale = np.abs(grad).max() + 1e-6
        for _ in range(4):
            idx = tuple(rng.integers(0, s) for s in P[n].shape)
            Pp = {k: v.copy() for k, v in P.items()}; Pp[n][idx] += eps
            Pm = {k: v.copy() for k, v in P.items()}; Pm[n][idx] -= eps
            fd = (loss(Pp) - loss(Pm)) / (2 * eps)
            assert abs(fd - grad[idx]) < 2e-3 * scale, (n, idx, fd, grad[idx])


@pytest.mark.parametrize("cls,N", [("cema", 16), ("ema", 2)])
def test_moving_average_module_autograd(cls, N):
    """Gradients of the raw parameters (alpha, delta, theta | beta, gamma, omega) and of x through
    autograd of the coefficient formulas + the backward operator, against central differences of
    the fp64 oracle."""
    rng = np.random.default_rng(62)
    B, D, L = 2, 16, 96
    torch.manual_seed(5)
    mod = (M.MultiHeadComplexEMA if cls == "cema" else M.MultiHeadEMA)(D, ndim=N).to(DEV).train()
    x64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    x = dev(x64).requires_grad_(True)
    (mod(x) * dev(w64)).sum().backward()

    names = ["alpha", "delta", "theta" if cls == "cema" else "beta", "gamma", "omega"]
    P = {n: host(getattr(mod, n)) for n in names}

    def loss(Pd, xx):
        if cls == "cema":
            p, q, g = O.ema_coeffs_complex(Pd["alpha"], Pd["delta"], Pd["theta"], Pd["gamma"])
        else:
            p, q, g = O.ema_coeffs_real(Pd["alpha"], Pd["delta"], Pd["beta"], Pd["gamma"])
        return (O.ema_forward(xx, p, q, g, Pd["omega"].reshape(-1))[0] * w64).sum()

    eps = 1e-5
    for n in names:
        grad = host(getattr(mod, n).grad)
        scale = np.abs(grad).max() + 1e-6
        for _ in range(4):
            idx = tuple(rng.integers(0, s) for s in P[n].shape)
            Pp = {k: v.copy() for k, v in P.items()}; Pp[n][idx] += eps
            Pm = {k: v.copy() for k, v in P.items()}; Pm[n][idx] -= eps
            fd = (loss(Pp, x64) - loss(Pm, x64)) / (2 * eps)
            assert abs(fd - grad[idx]) < 2e-3 * scale, (n, idx, fd, grad[idx])
    dxo = O.ema_backward(w64, x64, *_module_coeffs(mod, cls), host(mod.omega).reshape(-1))[0]
    assert rel_err(host(x.grad), dxo) < 1e-4


def _fd_check(rng, names, P, grads, loss, eps=1e-5, tol=2e-3, picks=4):
    for n in names:
        grad = grads[n]
        scale = np.abs(grad).max() + 1e-6
        for _ in range(picks):
            idx = tuple(rng.integers(0, s) for s in P[n].shape)
            Pp = {k: v.copy() for k, v in P.items()}; Pp[n][idx] += eps
            Pm = {k: v.copy() for k, v in P.items()}; Pm[n][idx] -= eps
            fd = (loss(Pp) - loss(Pm)) / (2 * eps)
            assert abs(fd - grad[idx]) < tol * scale, (n, idx, fd, grad[idx])


@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("cls,N", [("cema", 16), ("ema", 4)])
def test_training_with_carried_state(cls, N, masked):
    """Two chunks in training mode with the state carried between them (base_moving_average.py:139-160: kernel and
    bias from ema_parameters, ema_hidden for the next state): outputs against the oracle on the whole sequence,
    gradients of the raw parameters and of x (through both chunks and the state) against central differences of
    the fp64 oracle."""
    rng = np.random.default_rng(71)
    B, D, L1, L2 = 2, 8, 40, 56
    torch.manual_seed(6)
    mod = (M.MultiHeadComplexEMA if cls == "cema" else M.MultiHeadEMA)(D, ndim=N).to(DEV).train()
    x64 = rng.normal(size=(B, D, L1 + L2)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, D, L1 + L2)).astype(np.float32).astype(np.float64)
    mask = None
    if masked:
        mask = np.zeros((B, L1 + L2), bool); mask[0, 30:35] = True; mask[1, L1 + 20:] = True
    x = dev(x64).requires_grad_(True)
    state = {}
    tm = None if mask is None else dev(mask, torch.bool)
    y1 = mod(x[:, :, :L1], None if tm is None else tm[:, :L1], incremental_state=state)
    y2 = mod(x[:, :, L1:], None if tm is None else tm[:, L1:], incremental_state=state)
    y = torch.cat([y1, y2], dim=-1)
    names = ["alpha", "delta", "theta" if cls == "cema" else "beta", "gamma", "omega"]
    P = {n: host(getattr(mod, n)) for n in names}
    P["x"] = x64

    def run(Pd):
        if cls == "cema":
            p, q, g = O.ema_coeffs_complex(Pd["alpha"], Pd["delta"], Pd["theta"], Pd["gamma"])
        else:
            p, q, g = O.ema_coeffs_real(Pd["alpha"], Pd["delta"], Pd["beta"], Pd["gamma"])
        return O.ema_forward(Pd["x"], p, q, g, Pd["omega"].reshape(-1), mask)[0]

    assert rel_err(host(y), run(P)) < 1e-4          # the chunked call equals the whole sequence
    (y * dev(w64)).sum().backward()
    grads = {n: host(getattr(mod, n).grad) for n in names}
    grads["x"] = host(x.grad)
    _fd_check(rng, names + ["x"], P, grads, lambda Pd: (run(Pd) * w64).sum())


@pytest.mark.parametrize("shift", [True, False])
@pytest.mark.parametrize("cls,N", [("cema", 16), ("ema", 4)])
def test_training_with_truncated_kernel(cls, N, shift):
    """A two-sided layer whose kernel is cut to `truncation` lags, in training mode: output against the oracle,
    gradients against its central differences."""
    rng = np.random.default_rng(72)
    B, D, L, trunc = 2, 6, 90, 24
    torch.manual_seed(7)
    mod = (M.MultiHeadComplexEMA if cls == "cema" else M.MultiHeadEMA)(D, ndim=N, bidirectional=True, truncation=trunc,
                                                                      shift=shift).to(DEV).train()
    x64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    mask = np.zeros((B, L), bool); mask[1, L - 17:] = True
    x = dev(x64).requires_grad_(True)
    y = mod(x, dev(mask, torch.bool))
    names = ["alpha", "delta", "theta" if cls == "cema" else "beta", "gamma", "omega"]
    P = {n: host(getattr(mod, n)) for n in names}
    P["x"] = x64

    def run(Pd):
        if cls == "cema":
            p, q, g = O.ema_coeffs_complex(Pd["alpha"], Pd["delta"], Pd["theta"], Pd["gamma"])
        else:
            p, q, g = O.ema_coeffs_real(Pd["alpha"], Pd["delta"], Pd["beta"], Pd["gamma"])
        return O.ema_forward(Pd["x"], p, q, g, Pd["omega"].reshape(-1), mask, bidirectional=True, truncation=trunc,
                             shift=shift)[0]

    assert rel_err(host(y), run(P)) < 1e-4
    with torch.no_grad():
        assert rel_err(host(mod(x.detach(), dev(mask, torch.bool))), run(P)) < 1e-4   # the inference kernels agree
    (y * dev(w64)).sum().backward()
    grads = {n: host(getattr(mod, n).grad) for n in names}
    grads["x"] = host(x.grad)
    _fd_check(rng, names + ["x"], P, grads, lambda Pd: (run(Pd) * w64).sum())


def _module_coeffs(mod, cls):
    p, q, g = mod.coeffs()
    return host(p.squeeze(-1)), host(q.squeeze(-1)), host(g)


# ----------------------------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,causal", [((3, 40, 40), True), ((2, 3, 17, 50), True), ((4, 64, 256), False),
                                          ((2, 33, 33), False)])
def test_attention_softmax_bwd(dtype, shape, causal):
    rng = np.random.default_rng(71)
    x, x64 = rounded(rng.normal(size=shape) * 2, dtype)
    dy, dy64 = rounded(rng.normal(size=shape), dtype)
    y = M.ops.attention_softmax_fwd(x, 0.0, causal)
    y64 = host(y)                                          # the weights the backward is handed
    dx = M.ops.attention_softmax_bwd(dy, y, causal)
    assert rel_err(host(dx), O.attention_softmax_bwd(dy64, y64)) < TOL[dtype]
    # module-level autograd
    xg = x.clone().requires_grad_(True)
    (M.AttentionSoftmax(0.0, causal)(xg) * dy).sum().backward()
    assert rel_err(host(xg.grad), host(dx)) < 1e-6


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 2e-2), (torch.float16, 4e-3)])
@pytest.mark.parametrize("B,L,Nh,H1,H2", [(2, 64, 2, 16, 32), (1, 256, 4, 32, 64), (3, 50, 1, 8, 24)])
def test_attention_autograd(dtype, tol, B, L, Nh, H1, H2):
    """q, k, v gradients through AttentionFunc.  As in the reference (attention_kernel.cu:148, 195-203)
    the weight gradient dy v^T is stored in the activation type before its row mean under the weights
    is subtracted, so q and k gradients carry that rounding amplified by the cancellation: the
    per-op bound applies to their root-mean-square error and 4x the bound to the worst element."""
    rng = np.random.default_rng(72)
    q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    dy, dy64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    y = M.EfficientAttention(scale=0.5)(q, k, v)
    (y * dy).sum().backward()
    assert rel_err(host(y), O.attention(q64, k64, v64, 0.5, True)[0]) < TOL[dtype]
    for got, ref in zip((q.grad, k.grad, v.grad), O.attention_bwd(dy64, q64, k64, v64, 0.5, True)):
        e = host(got) - ref
        rms = np.sqrt((ref ** 2).mean())
        assert np.sqrt((e ** 2).mean()) < tol * rms and np.abs(e).max() < 4 * tol * max(rms, np.abs(ref).max())


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2), (torch.float16, 4e-3)])
@pytest.mark.parametrize("B,L,Nh,H1,H2,causal", [
    (1, 300, 2, 64, 136, True),      # several key tiles, v columns not a multiple of 64
    (2, 77, 3, 8, 24, True),         # rows of the weights that are not a multiple of 8 long
    (1, 640, 1, 128, 256, True),     # row tiles of 256 in the v gradient, reductions that start past the first K step
    (2, 130, 2, 16, 40, False),      # no mask: whole products
    (1, 1030, 2, 64, 64, True),      # more than one row tile of every product, ragged last tile
    (2, 264, 2, 72, 136, False),     # rows of whole 16-byte pieces: operands read in place (K-major), no mask
    (1, 1024, 2, 64, 320, True),     # the same with the mask: several row tiles, reductions that start at the diagonal
    (3, 72, 1, 8, 8, True),          # in place, smallest head sizes
])
def test_attention_bwd_entry_point(dtype, tol, B, L, Nh, H1, H2, causal):
    """mega_attention_bwd (the four products on the library's own matrix-core kernel, operands read head-strided in
    place, the causal half skipped) against the oracle's fp64 gradients (attention_kernel.cu:133-255), from the
    weights the forward returned.  The weight gradient stays in fp32 here (the reference rounds it to the activation
    type), so the bound of the per-op tolerance holds for the root-mean-square error and 4x for the worst element."""
    rng = np.random.default_rng(1000 + L)
    q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    dy, dy64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    scale = 1.0 / np.sqrt(H1)
    lib = M._lib.load()
    assert lib.mega_attention_bwd_workspace_bytes(M.ops._dtype_code(q), B, L, Nh, H1, H2) > 0
    y, w = M.ops.attention_fwd(q, k, v, scale, 0.0, causal, need_weights=True)
    want = O.attention_bwd(dy64, q64, k64, v64, scale, causal)
    # without and with the forward's output (the second lets the entry point take the row sums from y_grad . y)
    for with_y in (False, True):
        got = M.ops.attention_bwd(dy, q, k, v, w, scale, causal, y=y if with_y else None)
        for name, g, ref in zip("qkv", got, want):
            tag = f"{name} with_y={with_y}"
            assert g.shape == ref.shape and g.dtype == dtype
            e = host(g) - ref
            rms = np.sqrt((ref ** 2).mean())
            assert np.isfinite(host(g)).all(), tag
            assert np.sqrt((e ** 2).mean()) < tol * rms and np.abs(e).max() < 4 * tol * max(rms, np.abs(ref).max()), tag


def test_attention_bwd_entry_point_refuses_what_it_does_not_cover():
    """fp32 and head sizes that are not multiples of 8 take the batched library products in ops.attention_bwd; the
    entry point itself says so instead of computing something else."""
    lib = M._lib.load()
    assert lib.mega_attention_bwd_workspace_bytes(0, 1, 64, 1, 16, 16) == 0        # fp32
    assert lib.mega_attention_bwd_workspace_bytes(1, 1, 64, 1, 12, 16) == 0        # bf16, H1 = 12
    rng = np.random.default_rng(5)
    q = dev(rng.normal(size=(1, 64, 1, 12))).to(torch.bfloat16)
    v = dev(rng.normal(size=(1, 64, 1, 16))).to(torch.bfloat16)
    y, w = M.ops.attention_fwd(q, q, v, 0.3, 0.0, True, need_weights=True)
    gq, gk, gv = M.ops.attention_bwd(torch.ones_like(v), q, q, v, w, 0.3, True)       # library products
    ref = O.attention_bwd(np.ones((1, 64, 1, 16)), host(q), host(q), host(v), 0.3, True)
    assert rel_err(host(gv), ref[2]) < 2e-2
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=q.device)
    rc = lib.mega_attention_bwd(M.ops._ptr(v), M.ops._ptr(q), M.ops._ptr(q), M.ops._ptr(v), M.ops._ptr(w), None,
                                M.ops._ptr(gq), M.ops._ptr(gk), M.ops._ptr(gv), 1, 1, 64, 1, 12, 16, 0.3, 1,
                                M.ops._ptr(ws), ws.numel(), None)
    assert rc == -2                                     # MEGA_ERR_UNSUPPORTED


@pytest.mark.parametrize("heads,act,moving,bidir", [(1, 'rmsnorm', 'cema', False), (2, 'silu', 'ema', False),
                                                    (1, 'silu', 'cema', True), (2, 'rmsnorm', 'cema', "padded")])
def test_gated_attention_layer_trains(heads, act, moving, bidir):
    """The whole layer under autograd (fp32), causal and bidirectional (also with padding):
    parameter and input gradients against central differences of the fp64 layer oracle."""
    from test_gpu_layer import _params
    rng = np.random.default_rng(73)
    B, L, D, S, E, N, C = 2, 32, 16, 8, 24, 4, 16
    torch.manual_seed(11)
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_layer=moving, moving_act=act,
                                          norm_num_groups=4, num_heads=heads, bidirectional=bool(bidir)).to(DEV).train()
    mask = None
    if bidir == "padded":
        mask = np.zeros((B, L), bool)
        mask[0, 27:] = True
        mask[1, 12:] = True                    # the second chunk of row 1 is padding only
    with torch.no_grad():
        for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
            prm.normal_(0, 0.3)
        layer.gamma.normal_(0, 0.3); layer.beta.normal_(0, 0.3)
        layer.norm.weight.normal_(0, 0.2); layer.norm.bias.normal_(0, 0.2)
    x64 = rng.normal(size=(B, L, D)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, L, D)).astype(np.float32).astype(np.float64)
    if mask is not None:
        w64 = w64 * (~mask)[..., None]         # padded positions carry no loss
    x = dev(x64).requires_grad_(True)
    out, _ = layer(x, None if mask is None else torch.from_numpy(mask).to(DEV))
    in_place = M.modules.SplitGrads.taken
    (out * dev(w64)).sum().backward()
    # the gradients of the four slices of the mx_proj output were written into one buffer (no concatenation)
    assert M.modules.SplitGrads.taken == in_place + 1
    P = _params(layer)
    okw = dict(chunk=C, num_heads=heads, moving_act=act, num_groups=4, bidirectional=bool(bidir), padding_mask=mask)
    loss = lambda Pd, xx: (O.gated_attention_layer(xx, Pd, **okw) * w64).sum()
    keep = np.ones((B, L), bool) if mask is None else ~mask
    assert rel_err(host(out)[keep], O.gated_attention_layer(x64, P, **okw)[keep]) < 1e-4
    eps = 1e-5
    checks = [("v_w", layer.v_proj.weight), ("mx_w", layer.mx_proj.weight), ("mx_b", layer.mx_proj.bias),
              ("h_w", layer.h_proj.weight), ("gamma", layer.gamma), ("beta", layer.beta),
              ("norm_weight", layer.norm.weight), ("norm_bias", layer.norm.bias)]
    for name, prm in checks:
        grad = host(prm.grad)
        scale = np.abs(grad).max() + 1e-6
        for _ in range(3):
            idx = tuple(rng.integers(0, s) for s in P[name].shape)
            Pp = dict(P); Pp[name] = P[name].copy(); Pp[name][idx] += eps
            Pm = dict(P); Pm[name] = P[name].copy(); Pm[name][idx] -= eps
            fd = (loss(Pp, x64) - loss(Pm, x64)) / (2 * eps)
            assert abs(fd - grad[idx]) < 3e-3 * scale, (name, idx, fd, grad[idx])
    gx = host(x.grad)
    for _ in range(4):
        idx = tuple(rng.integers(0, s) for s in x64.shape)
        xp, xm = x64.copy(), x64.copy()
        xp[idx] += eps; xm[idx] -= eps
        fd = (loss(P, xp) - loss(P, xm)) / (2 * eps)
        assert abs(fd - gx[idx]) < 3e-3 * (np.abs(gx).max() + 1e-6), (idx, fd, gx[idx])
    # the moving-average parameters get gradients as well
    for prm in (layer.move.alpha, layer.move.delta, layer.move.gamma, layer.move.omega):
        assert prm.grad is not None and torch.isfinite(prm.grad).all() and prm.grad.abs().max() > 0


def test_mega2_block_trains_bf16():
    """One Mega2 block (gated attention + TimestepNorm + SwiGLU) forward and backward in bf16 at a
    shape that takes the matrix-core paths (EMA forwards and backwards in time, MFMA attention):
    every parameter receives a finite gradient, and the input gradient agrees with the same block
    evaluated in fp32 (same weights) to the chained bf16 bound."""
    torch.manual_seed(12)
    B, L, D, S, E, N, C, Hf = 2, 2048, 128, 64, 256, 16, 1024, 320
    blk32 = M.Mega2Layer(D, S, E, N, Hf, C, norm_num_groups=8, num_heads=2, moving_act='silu').to(DEV).train()
    import copy
    blk16 = copy.deepcopy(blk32).to(torch.bfloat16)
    with torch.no_grad():                      # both copies hold exactly the bf16-representable weights
        for p32, p16 in zip(blk32.parameters(), blk16.parameters()):
            p32.copy_(p16.float())
    x = torch.randn(B, L, D, device=DEV).to(torch.bfloat16)
    w = torch.randn(B, L, D, device=DEV).to(torch.bfloat16)
    x16 = x.clone().requires_grad_(True)
    x32 = x.float().requires_grad_(True)
    (blk16(x16) * w).sum().backward()
    (blk32(x32) * w.float()).sum().backward()
    for (name, p16), p32 in zip(blk16.named_parameters(), blk32.parameters()):
        assert p16.grad is not None and torch.isfinite(p16.grad).all(), name
    e = host(x16.grad) - host(x32.grad)
    rms = np.sqrt((host(x32.grad) ** 2).mean())
    assert np.sqrt((e ** 2).mean()) < 3e-2 * rms, np.sqrt((e ** 2).mean()) / rms
    # the large matrices' gradients agree as well (sums over B * L tokens in fp32 inside the GEMMs)
    for n16, n32 in ((blk16.attn.mx_proj.weight, blk32.attn.mx_proj.weight), (blk16.ffn.w2.weight, blk32.ffn.w2.weight)):
        e = host(n16.grad) - host(n32.grad)
        rms = np.sqrt((host(n32.grad) ** 2).mean())
        assert np.sqrt((e ** 2).mean()) < 3e-2 * rms


# ----------------------------------------------------------------------------------------------
# SequenceNorm
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,H,G,last,masked", [(2, 256, 64, 8, True, True), (2, 77, 40, 4, True, True),
                                                 (3, 50, 24, None, True, False), (2, 60, 32, 4, False, True)])
def test_sequence_norm_bwd(dtype, B, L, H, G, last, masked):
    rng = np.random.default_rng(91)
    x, x64 = rounded(rng.normal(size=(B, H, L) if last else (B, L, H)) * 1.4 + 0.5, dtype)
    dy, dy64 = rounded(rng.normal(size=x64.shape), dtype)
    gamma = (rng.normal(size=H) * 0.3 + 1).astype(np.float32).astype(np.float64)
    beta = rng.normal(size=H).astype(np.float32).astype(np.float64)
    mask = (rng.random((B, L)) < 0.25) if masked else None
    tm = None if mask is None else torch.from_numpy(mask).to(DEV)
    GG = H if G is None else G
    y, n, mu, r = M.ops.group_sequence_norm_fwd(x, dev(gamma), dev(beta), tm, GG, 1e-5, last)
    dx, dg, db = M.ops.group_sequence_norm_bwd(dy, x, n, mu, r, dev(gamma), tm, GG, last)
    rx, rg, rb = O.sequence_norm_bwd(dy64, x64, gamma, mask, G, 1e-5, last)
    assert rel_err(host(dx), rx) < TOL[dtype]
    assert rel_err(host(dg), rg) < 2e-4 and rel_err(host(db), rb) < 2e-4


def test_sequence_norm_module_autograd_and_golden():
    rng = np.random.default_rng(92)
    B, H, L = 2, 32, 70
    mod = M.SequenceNorm(H, 4).to(DEV).train()
    with torch.no_grad():
        mod.weight.normal_(0, 0.2); mod.bias.normal_(0, 0.2)
    x64 = rng.normal(size=(B, H, L)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, H, L)).astype(np.float32).astype(np.float64)
    x = dev(x64).requires_grad_(True)
    (mod(x) * dev(w64)).sum().backward()
    rx, rg, rb = O.sequence_norm_bwd(w64, x64, host(mod.weight) + 1, None, 4, 1e-5, True)
    assert rel_err(host(x.grad), rx) < 1e-4
    assert rel_err(host(mod.weight.grad), rg) < 2e-4 and rel_err(host(mod.bias.grad), rb) < 2e-4
    # the reference's own backward outputs
    import os
    gold = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_cpu_vectors.npz"))
    for tag in ("gsn_bwd_a", "gsn_bwd_b", "sn_bwd"):
        c = {k[len(tag) + 1:]: gold[k] for k in gold.files if k.startswith(tag + ".")}
        last = bool(c["length_last"])
        G = int(c["groups"]) or c["gamma"].shape[0]
        tm = None if "mask" not in c else torch.from_numpy(c["mask"]).to(DEV)
        y, n, mu, r = M.ops.group_sequence_norm_fwd(dev(c["x"]), dev(c["gamma"]), dev(c["beta"]), tm, G, 1e-5, last)
        dx, dg, db = M.ops.group_sequence_norm_bwd(dev(c["y_grad"]), dev(c["x"]), n, mu, r, dev(c["gamma"]), tm, G, last)
        assert rel_err(host(dx), c["x_grad"]) < 1e-4, tag
        assert rel_err(host(dg), c["gamma_grad"]) < 1e-4 and rel_err(host(db), c["beta_grad"]) < 1e-4, tag


# ----------------------------------------------------------------------------------------------
# element-wise gates
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,width,off", [((2, 50, 512), 1100, 80), ((4, 9, 35), 35, 0)])
def test_gate_backwards(dtype, shape, width, off):
    """gate_mul, gate_out and swiglu backward against the closed-form derivatives in fp64
    (silu'(a) = s (1 + a (1 - s)), s = sigmoid(a)); operands that are slices of a wider row."""
    from test_gpu_ops import _wide
    rng = np.random.default_rng(95)
    sg = O._sigmoid
    dsilu = lambda a_: sg(a_) * (1 + a_ * (1 - sg(a_)))
    a, a64 = rounded(rng.normal(size=shape), dtype)
    r, r64 = _wide(rng, shape, width, off, dtype)
    dy, dy64 = rounded(rng.normal(size=shape), dtype)
    da, dr = M.ops.gate_mul_bwd(dy, a, r)
    assert rel_err(host(da), dy64 * O._silu(r64)) < TOL[dtype]
    assert rel_err(host(dr), dy64 * a64 * dsilu(r64)) < TOL[dtype]
    u, u64 = _wide(rng, shape, width, 0, dtype)
    hx, hx64 = _wide(rng, shape, width, off, dtype)
    hp, hp64 = rounded(rng.normal(size=shape), dtype)
    res, res64 = rounded(rng.normal(size=shape), dtype)
    dres, du, dh = M.ops.gate_out_bwd(dy, res, u, hx, hp)
    s, aa = sg(u64), hx64 + hp64
    assert rel_err(host(dres), dy64 * (1 - s)) < TOL[dtype]
    assert rel_err(host(du), dy64 * (O._silu(aa) - res64) * s * (1 - s)) < TOL[dtype]
    assert rel_err(host(dh), dy64 * s * dsilu(aa)) < TOL[dtype]
    # the same gradients written into slices of one wider buffer (row stride = its width): the values next to
    # the slices stay as they were
    W = 3 * shape[-1] + 8
    buf = torch.full(shape[:-1] + (W,), 7.0, dtype=dtype, device=DEV)
    s0, s1, s2 = buf.narrow(-1, 0, shape[-1]), buf.narrow(-1, shape[-1] + 8, shape[-1]), buf.narrow(-1, 2 * shape[-1] + 8, shape[-1])
    _, dr2 = M.ops.gate_mul_bwd(dy, a, r, r_grad_out=s0)
    _, du2, dh2 = M.ops.gate_out_bwd(dy, res, u, hx, hp, u_grad_out=s1, h_grad_out=s2)
    torch.cuda.synchronize()
    if (shape[-1] * dy.element_size()) % 16 == 0:
        assert dr2.data_ptr() == s0.data_ptr() and du2.data_ptr() == s1.data_ptr() and dh2.data_ptr() == s2.data_ptr()
        assert bool((buf.narrow(-1, shape[-1], 8) == 7.0).all())
    assert torch.equal(dr2, dr) and torch.equal(du2, du) and torch.equal(dh2, dh)
    b, b64 = rounded(rng.normal(size=shape), dtype)
    ga, gb = M.ops.swiglu_bwd(dy, a, b)
    assert rel_err(host(ga), dy64 * b64 * dsilu(a64)) < TOL[dtype]
    assert rel_err(host(gb), dy64 * O._silu(a64)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_silu_backward_and_column_sums(dtype):
    """silu backward against the closed form; column sums (bias gradients) of contiguous and row-strided matrices
    against fp64 sums, the same bits on a second run; LinearFunc against torch's own backward of F.linear."""
    rng = np.random.default_rng(97)
    sg = O._sigmoid
    x, x64 = rounded(rng.normal(size=(3, 37, 24)) * 2, dtype)
    dy, dy64 = rounded(rng.normal(size=(3, 37, 24)), dtype)
    assert rel_err(host(M.ops.silu_bwd(dy, x)), dy64 * sg(x64) * (1 + x64 * (1 - sg(x64)))) < TOL[dtype]
    for T, W, width, off in ((200, 48, 48, 0), (1000, 64, 160, 32), (63, 8, 8, 0), (8192, 520, 1048, 8)):
        wide, w64 = rounded(rng.normal(size=(T, width)), dtype)
        sl = wide.narrow(-1, off, W)
        got = M.ops.colsum(sl, torch.float32)
        ref = w64[:, off:off + W].sum(0)
        assert rel_err(host(got), ref) < 1e-5 and torch.equal(got, M.ops.colsum(sl, torch.float32))
        assert M.ops.colsum(sl).dtype == dtype
    assert rel_err(host(M.ops.colsum(x, torch.float32)), x64.reshape(-1, 24).sum(0)) < 1e-5      # leading axes fold
    odd, o64 = rounded(rng.normal(size=(50, 7)), dtype)                                          # torch's route
    assert rel_err(host(M.ops.colsum(odd, torch.float32)), o64.sum(0)) < 1e-5
    lin = torch.nn.Linear(24, 40).to(DEV).to(dtype)
    up = torch.randn(3, 37, 40, device=DEV).to(dtype)
    xa, xb = x.clone().requires_grad_(True), x.clone().requires_grad_(True)
    (M.modules.linear(lin, xa) * up).sum().backward()
    ga = [xa.grad, lin.weight.grad.clone(), lin.bias.grad.clone()]
    lin.zero_grad()
    (lin(xb) * up).sum().backward()
    tol = 1e-5 if dtype == torch.float32 else TOL[dtype]
    for a, b in zip(ga, [xb.grad, lin.weight.grad, lin.bias.grad]):
        assert a.dtype == b.dtype and a.shape == b.shape and rel_err(host(a), host(b)) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,S,heads,chunk,width,off", [(2, 64, 128, 1, 64, 128, 0), (1, 96, 64, 4, 32, 200, 72),
                                                         (3, 40, 40, 2, 40, 56, 8), (1, 4096, 512, 4, 2048, 512, 0),
                                                         (2, 300, 512, 2, 100, 1024, 512)])
def test_gate_qk_bwd(dtype, B, L, S, heads, chunk, width, off):
    """Backward of the q / k map against fp64 autograd through normalize -> affine -> rotation written
    with torch operations on the CPU; z a slice of a wider row, one all-zero row (clamped norm)."""
    from test_gpu_ops import _wide
    rng = np.random.default_rng(97)
    z, z64 = _wide(rng, (B, L, S), width, off, dtype)
    with torch.no_grad():
        z[0, 1].zero_()
    z64[0, 1] = 0
    g = rng.normal(size=(2, S)) * 0.3 + 1
    b = rng.normal(size=(2, S)) * 0.3
    Hd = S // heads
    freqs = (1.0 / (10000.0 ** (np.arange(0, Hd, 2) / Hd))).astype(np.float32)
    up = rng.normal(size=(2, B, L, S))
    up[:, 0, 1] *= 1e-2                    # the clamped row scales its gradient by 1 / eps: keep it inside fp16
    dq, dq64 = rounded(up[0], dtype)
    dk, dk64 = rounded(up[1], dtype)
    dz, dg, db = M.ops.gate_qk_bwd(dq, dk, z, dev(g), dev(freqs), heads, chunk)
    # the same gradient written into a slice of a wider buffer
    wide = torch.full((B, L, S + 24), 3.0, dtype=dtype, device=DEV)
    dz2, dg2, db2 = M.ops.gate_qk_bwd(dq, dk, z, dev(g), dev(freqs), heads, chunk, z_grad_out=wide.narrow(-1, 16, S))
    torch.cuda.synchronize()
    assert dz2.data_ptr() == wide.narrow(-1, 16, S).data_ptr() and torch.equal(dz2, dz)
    assert torch.equal(dg2, dg) and torch.equal(db2, db)
    assert bool((wide[..., :16] == 3.0).all()) and bool((wide[..., 16 + S:] == 3.0).all())
    # arbiter
    tz = torch.from_numpy(z64).requires_grad_(True)
    tg = torch.from_numpy(g).requires_grad_(True)
    tb = torch.from_numpy(b).requires_grad_(True)
    zn = tz / tz.norm(dim=-1, keepdim=True).clamp_min(1e-5)
    ang = torch.arange(chunk, dtype=torch.float64)[:, None] * torch.from_numpy(freqs.astype(np.float64))[None, :]
    cs, sn = torch.cos(ang)[None, :, None, :], torch.sin(ang)[None, :, None, :]
    loss = 0
    for i, up in ((0, dq64), (1, dk64)):
        a = (zn * tg[i] + tb[i]).reshape(B * (L // chunk), chunk, heads, Hd // 2, 2)
        a0, a1 = a[..., 0], a[..., 1]
        rot = torch.stack([a0 * cs - a1 * sn, a0 * sn + a1 * cs], dim=-1).reshape(B, L, S)
        loss = loss + (rot * torch.from_numpy(up)).sum()
    loss.backward()
    # a clamped row has gradient dzn / eps = 1e5 dzn: compare it apart from the others
    ref = tz.grad.numpy()
    got = host(dz)
    keep = np.ones((B, L), bool); keep[0, 1] = False
    tol = max(TOL[dtype], 5e-4)
    assert rel_err(got[keep], ref[keep]) < tol
    assert rel_err(got[0, 1], ref[0, 1]) < tol
    # sums over all tokens of bf16-rounded products: fp32 accumulation, inputs exact
    assert rel_err(host(dg), tg.grad.numpy()) < 5e-4 and rel_err(host(db), tb.grad.numpy()) < 5e-4


def test_gate_qk_bwd_rejects_bad_arguments():
    z = torch.zeros(2, 4, 36, device=DEV, dtype=torch.bfloat16)
    g = torch.ones(2, 36, device=DEV)
    with pytest.raises(RuntimeError):                                   # rows of 36 bf16 are not whole vectors
        M.ops.gate_qk_bwd(z, z, z, g, torch.ones(9, device=DEV), 2, 4)
    z = torch.zeros(2, 4, 2048, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):                                   # more than two vectors per lane
        M.ops.gate_qk_bwd(z, z, z, torch.ones(2, 2048, device=DEV), torch.ones(1024, device=DEV), 1, 4)
    z = torch.zeros(0, 64, device=DEV)
    dz, dg, db = M.ops.gate_qk_bwd(z, z, z, torch.ones(2, 64, device=DEV), torch.ones(32, device=DEV), 1, 4)
    assert dz.shape == (0, 64) and float(dg.abs().sum()) == 0 and float(db.abs().sum()) == 0


def test_backward_edge_shapes():
    """Single-token and single-row inputs, channel counts that are not multiples of the tile sizes."""
    rng = np.random.default_rng(99)
    # TimestepNorm backward, one token
    x, x64 = rounded(rng.normal(size=(1, 1, 8)), torch.float32)
    dy, dy64 = rounded(rng.normal(size=(1, 1, 8)), torch.float32)
    gamma, beta = np.ones(8), np.zeros(8)
    pc, pm, pv = np.array([2], np.int64), rng.normal(size=(1, 2)) * 0.1, np.ones((1, 2))
    y, cnt, mu, var, gm, cm, cr = M.ops.group_timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma),
                                                                dev(beta), None, 2, 1e-5)
    got = M.ops.group_timestep_norm_bwd(dy, None, None, x, dev(pm), cnt, gm, cm, cr, dev(gamma), None, 2)
    ocnt, ogm, ocm, ocr = O.timestep_norm_saved(x64, pc, pm.astype(np.float32).astype(np.float64), pv, None, 2, 1e-5)
    ref = O.timestep_norm_bwd(dy64, None, None, x64, pm.astype(np.float32).astype(np.float64), ocnt, ogm, ocm, ocr,
                              gamma, None, 2)
    for a, b in zip(got, ref):
        assert rel_err(host(a), b) < 2e-4
    # moving-average backward: one token, then a tile boundary plus one, 5 channels, 3 states
    for L in (1, 129):
        p, q, g = _ema_coeffs(rng, 5, 3, True)
        p, q, g = p.astype(np.float32).astype(np.float64), q.astype(np.complex64).astype(np.complex128), \
            g.astype(np.complex64).astype(np.complex128)
        om = rng.normal(size=5).astype(np.float32).astype(np.float64)
        x, x64 = rounded(rng.normal(size=(2, 5, L)), torch.float32)
        dy, dy64 = rounded(rng.normal(size=(2, 5, L)), torch.float32)
        got = M.ops.ema_backward(dy, x, dev(p), dev(q), dev(g), dev(om))
        ref = O.ema_backward(dy64, x64, p, q, g, om)
        assert rel_err(host(got[0]), ref[0]) < 1e-4
        for a, b in zip(got[1:], ref[1:]):
            a = host(a)
            assert rel_err(np.real(a), np.real(b)) < 5e-4 and rel_err(np.imag(a), np.imag(b)) < 5e-4
    # SequenceNorm forward + backward, one token per row
    x, x64 = rounded(rng.normal(size=(2, 6, 1)), torch.float32)
    dy, dy64 = rounded(rng.normal(size=(2, 6, 1)), torch.float32)
    gam = rng.normal(size=6) + 1
    y, n, mu, r = M.ops.group_sequence_norm_fwd(x, dev(gam), dev(np.zeros(6)), None, 2, 1e-5, True)
    assert rel_err(host(y), O.sequence_norm(x64, gam.astype(np.float32), np.zeros(6), None, 2, 1e-5, True)[0]) < 1e-4
    dx, dg, db = M.ops.group_sequence_norm_bwd(dy, x, n, mu, r, dev(gam), None, 2, True)
    rx, rg, rb = O.sequence_norm_bwd(dy64, x64, gam.astype(np.float32).astype(np.float64), None, 2, 1e-5, True)
    assert rel_err(host(dx), rx) < 1e-4 and rel_err(host(dg), rg) < 2e-4 and rel_err(host(db), rb) < 2e-4
    # softmax backward on a single column
    yv = M.ops.attention_softmax_fwd(dev(rng.normal(size=(3, 1, 1))), 0.0, True)
    assert float(M.ops.attention_softmax_bwd(dev(rng.normal(size=(3, 1, 1))), yv, True).abs().max()) < 1e-6


def test_explicit_kernel_convolution_autograd():
    """ops.fftconv(x, k) under autograd against the oracle's correlations (dk restricted to Lk lags)."""
    rng = np.random.default_rng(97)
    B, D, L, Lk = 2, 6, 70, 40
    x64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    k64 = rng.normal(size=(D, Lk)).astype(np.float32).astype(np.float64)
    w64 = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64)
    x = dev(x64).requires_grad_(True)
    k = dev(k64).requires_grad_(True)
    y = M.ops.fftconv(x, k)
    assert rel_err(host(y), O.causal_conv_direct(x64, k64)) < 1e-4
    (y * dev(w64)).sum().backward()
    dx = np.zeros_like(x64)
    dk = np.zeros_like(k64)
    for l in range(Lk):
        dx[:, :, :L - l] += w64[:, :, l:] * k64[None, :, l:l + 1]
        dk[:, l] = (w64[:, :, l:] * x64[:, :, :L - l]).sum(axis=(0, 2))
    assert rel_err(host(x.grad), dx) < 1e-4 and rel_err(host(k.grad), dk) < 1e-4


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 2e-2)])
def test_attention_dropkey_autograd(dtype, tol):
    """Training with DropKey: the backward runs on the saved weights, which hold zeros at the dropped
    keys, so the gradients are those of the oracle with the same mask."""
    rng = np.random.default_rng(74)
    B, L, Nh, H1, H2 = 2, 64, 2, 16, 32
    q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    dy, dy64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    p, seed = 0.25, 424242
    drop = O.dropkey_draws(seed, (B, Nh, L, L)) < p
    q, k, v = (t.requires_grad_(True) for t in (q, k, v))
    y = M.modules.attention(q, k, v, 0.5, p, True, True, seed)
    (y * dy).sum().backward()
    assert rel_err(host(y), O.attention(q64, k64, v64, 0.5, True, drop)[0]) < TOL[dtype]
    for got, ref in zip((q.grad, k.grad, v.grad), O.attention_bwd(dy64, q64, k64, v64, 0.5, True, drop)):
        e = host(got) - ref
        rms = np.sqrt((ref ** 2).mean())
        assert np.sqrt((e ** 2).mean()) < tol * rms and np.abs(e).max() < 4 * tol * max(rms, np.abs(ref).max())
    # the softmax op alone
    x, x64 = rounded(rng.normal(size=(3, 20, 20)) * 2, dtype)
    g, g64 = rounded(rng.normal(size=(3, 20, 20)), dtype)
    xg = x.clone().requires_grad_(True)
    yy = M.modules.attention_softmax(xg, p, False, True, seed)
    (yy * g).sum().backward()
    ref = O.attention_softmax_bwd(g64, host(yy))
    assert rel_err(host(xg.grad), ref) < TOL[dtype]
    assert np.all(host(xg.grad)[O.dropkey_draws(seed, (3, 20, 20)) < p] == 0)


@pytest.mark.parametrize("B,L,Nh,H1,H2,causal", [(2, 256, 2, 64, 128, True), (1, 520, 1, 32, 64, True),
                                                 (2, 128, 4, 16, 24, False)])
def test_attention_backward_without_kept_weights(B, L, Nh, H1, H2, causal):
    """Training through the fused attention without keeping the L x L weights between the passes (the forward is
    the one-kernel attention, the backward forms the weights again): same output and same gradients as with the
    reference's kept weights, to the rounding of the 16-bit output; and the saved tensors hold no L x L array."""
    torch.manual_seed(77)
    q, k = (torch.randn(B, L, Nh, H1, device=DEV).to(torch.bfloat16) for _ in range(2))
    v = torch.randn(B, L, Nh, H2, device=DEV).to(torch.bfloat16)
    dy = torch.randn(B, L, Nh, H2, device=DEV).to(torch.bfloat16)
    outs = {}
    for keep in (True, False):
        M.modules.AttentionFunc.KEEP_WEIGHTS = keep
        try:
            qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
            y = M.modules.attention(qq, kk, vv, 0.125, 0.0, causal, True)
            saved = [t.shape for t in y.grad_fn.saved_tensors]
            y.backward(dy)
            outs[keep] = (y.detach(), qq.grad, kk.grad, vv.grad, saved)
        finally:
            M.modules.AttentionFunc.KEEP_WEIGHTS = False
    torch.cuda.synchronize()
    assert any(len(s) == 4 and s[-1] == L and s[-2] == L for s in outs[True][4])
    assert not any(len(s) == 4 and s[-1] == L and s[-2] == L for s in outs[False][4])
    def close(got, ref, tol=2e-2):           # the bound of test_attention_autograd: rms error and worst element
        e = host(got) - np.asarray(ref)
        rms = np.sqrt((np.asarray(ref) ** 2).mean())
        return np.sqrt((e ** 2).mean()) < tol * rms and np.abs(e).max() < 4 * tol * max(rms, np.abs(ref).max())

    for a, b in zip(outs[True][:4], outs[False][:4]):      # two 16-bit paths against each other
        assert close(b, host(a))
    # and against the fp64 oracle
    yo, _ = O.attention(host(q), host(k), host(v), 0.125, causal)
    assert rel_err(host(outs[False][0]), yo) < 2e-2
    dq, dk, dv = O.attention_bwd(host(dy), host(q), host(k), host(v), 0.125, causal)
    for got, want in zip(outs[False][1:4], (dq, dk, dv)):
        assert close(got, want)
