"""Seeded random sweeps across the shape boundaries where the library changes kernels: every case is one call
of a public operator checked against the fp64 oracle.  The moving average draws its type, layout, lengths around
64 / 256 / 1024 / 4096 tokens, channel counts around the 16-channel blocks, 1..16 (or 32) states, mask, carried
state, direction and truncation; the TimestepNorm draws group and per-feature variants, masks, priors and tile
boundaries; the norm -> moving-average call draws shapes inside and outside its one-kernel envelope."""
import os

import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, mega_init_real, rel_err
from gpu_util import DEV, TOL, dev, host, rounded
from oracle import mega_oracle as O

# MEGA_SWEEP_SEED_SHIFT=k moves every generator of this file to other cases (a wider sweep by hand); 0: the fixed set
SEED_SHIFT = 100003 * int(os.environ.get("MEGA_SWEEP_SEED_SHIFT", "0"))
pytestmark = pytest.mark.gpu
DTYPES = [torch.float32, torch.bfloat16, torch.float16]
LENGTHS = [1, 2, 31, 63, 64, 65, 100, 255, 256, 257, 511, 1000, 1023, 1024, 1025, 2047, 2048, 2052, 3000, 4096, 4100]


def _state_err(h, ho):
    """rel_err with a floor: behind a long masked tail the state has decayed below what fp32 holds at all (states of
    an active row are of order one; 1e-6 of that is the floor)."""
    a, b = np.asarray(h, np.float64), np.asarray(ho, np.float64)
    den = np.maximum(np.abs(b), float(np.sqrt(np.mean(b * b))) + 1e-6)
    return float(np.max(np.abs(a - b) / den))


def _out_err(y, yo, eps=1.0):
    """rel_err whose floor does not collapse on an output that is mostly small (a padded row whose only content is
    the carried state decaying away; the late rows of a long causal attention, averages over a thousand values, next
    to early rows of order one): max |y - yo| / max(|yo|, eps rms(yo), max |yo| / 8).  A sum of bf16-rounded terms as
    large as the largest outputs is off by 2^-9 of those terms wherever it lands."""
    a, b = np.asarray(y, np.float64), np.asarray(yo, np.float64)
    if not b.size:
        return 0.0
    floor = max(eps * float(np.sqrt(np.mean(b * b))), float(np.abs(b).max()) / 8.0, 1e-300)
    return float(np.max(np.abs(a - b) / np.maximum(np.abs(b), floor)))


def _worst(y, yo):
    """Where rel_err takes its maximum, for the messages of failing cases."""
    a, b = np.asarray(y, np.float64), np.asarray(yo, np.float64)
    rms = float(np.sqrt(np.mean(b * b)))
    ratio = np.abs(a - b) / np.maximum(np.abs(b), rms + 1e-300)
    idx = np.unravel_index(int(np.argmax(ratio)), ratio.shape)
    return f"worst at {tuple(int(i) for i in idx)}: got {a[idx]:.6g} ref {b[idx]:.6g} rms {rms:.4g} max |ref| {np.abs(b).max():.4g}"


def _coeffs(rng, K, N, cplx):
    if cplx:
        return O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    return O.ema_coeffs_real(*mega_init_real(rng, K, N))


@pytest.mark.parametrize("seed", range(16))
def test_moving_average_sweep(seed):
    rng = np.random.default_rng(1000 + seed + SEED_SHIFT)
    for case in range(12):
        dtype = DTYPES[int(rng.integers(0, 3))]
        L = int(rng.choice(LENGTHS))
        D = int(rng.choice([1, 3, 15, 16, 17, 32, 48, 130]))
        B = int(rng.choice([1, 2, 3, 5]))
        if B * D * L > 3_000_000:
            B, D = 1, min(D, 32)
        N = int(rng.choice([1, 2, 5, 8, 15, 16, 32])) if L <= 2052 else int(rng.choice([2, 16]))
        cplx = bool(rng.integers(0, 2))
        bidir = bool(rng.integers(0, 2))
        time_major = bool(rng.integers(0, 2))
        masked = bool(rng.integers(0, 2))
        shift = bool(rng.integers(0, 2))
        trunc = int(rng.choice([0, 0, 7, 40, 300])) if bidir else 0
        with_state = (not bidir) and bool(rng.integers(0, 2)) and B * D * N * L < 4_000_000
        out_layout = "input" if rng.integers(0, 3) == 0 else "rows"
        tag = (f"seed {seed} case {case}: {dtype} B={B} D={D} L={L} N={N} cplx={cplx} bidir={bidir} shift={shift} "
               f"trunc={trunc} time_major={time_major} masked={masked} state={with_state} out={out_layout}")
        print(tag, flush=True)
        p, q, g = _coeffs(rng, 2 * D if bidir else D, N, cplx)
        om = rng.normal(size=D)
        if time_major:
            xt, xt64 = rounded(rng.normal(size=(B, L, D)), dtype)
            x, x64 = xt.transpose(1, 2), xt64.transpose(0, 2, 1)
        else:
            x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
        mask = None
        if masked:
            mask = rng.random((B, L)) < 0.1
            mask[0, L - L // 5:] = True
        h0 = None
        if with_state:
            h0 = rng.normal(size=(B, D, N)) + (1j * rng.normal(size=(B, D, N)) if cplx else 0)
            h0 = h0.astype(np.complex64) if cplx else h0.astype(np.float32)
        y, h = M.ops.ema_forward(x, dev(p), dev(q), dev(g), dev(om),
                                 padding_mask=None if mask is None else dev(mask, torch.bool),
                                 h=None if h0 is None else dev(h0), want_state=with_state, bidirectional=bidir,
                                 truncation=trunc if trunc else None, shift=shift, out_layout=out_layout)
        torch.cuda.synchronize()
        yo, ho = O.ema_forward(x64, p, q, g, om, mask, h=h0, bidirectional=bidir, truncation=trunc if trunc else None,
                               shift=shift, incremental=with_state)
        assert y.shape == (B, D, L), tag
        assert rel_err(host(y), yo) < TOL[dtype], (tag, _worst(host(y), yo))
        if with_state:
            tol = 1e-4 if dtype is torch.float32 else 2e-3
            assert _state_err(np.real(host(h)), np.real(ho)) < tol, tag
            if cplx:
                assert _state_err(np.imag(host(h)), np.imag(ho)) < tol, tag


@pytest.mark.parametrize("seed", range(16))
def test_timestep_norm_sweep(seed):
    rng = np.random.default_rng(2000 + seed + SEED_SHIFT)
    for case in range(10):
        dtype = DTYPES[int(rng.integers(0, 3))]
        L = int(rng.choice([1, 2, 7, 8, 15, 16, 17, 33, 64, 100, 257, 1000, 1024, 2049]))
        feature = rng.integers(0, 4) == 0
        if feature:
            H = int(rng.choice([1, 4, 12, 64, 200]))
            G = None
        else:
            G = int(rng.choice([1, 2, 3, 4, 16]))
            H = G * int(rng.choice([1, 2, 8, 24, 64, 128]))
        B = int(rng.choice([1, 2, 5]))
        masked = bool(rng.integers(0, 2))
        prior = bool(rng.integers(0, 2))
        if H // (H if G is None else G) == 1 and L < 8:
            L = 17              # one value per statistic and hardly any steps: the variance is 0, rstd = eps^-1/2 amplifies rounding
        tag = f"seed {seed} case {case}: {dtype} B={B} L={L} H={H} G={G} masked={masked} prior={prior}"
        print(tag, flush=True)
        Gn = H if G is None else G
        x, x64 = rounded(rng.normal(size=(B, L, H)) * 2.0 + 0.5, dtype)
        gam = rng.normal(size=H) * 0.2 + 1.0
        bet = rng.normal(size=H) * 0.2
        mask = None
        if masked:
            mask = rng.random((B, L)) < 0.15
            mask[B - 1, L // 2:] = True
        pc = rng.integers(1, 50, size=B) if prior else np.zeros(B, np.int64)
        pm = rng.normal(size=(B, Gn)) if prior else np.zeros((B, Gn))
        pv = rng.random((B, Gn)) + 0.5 if prior else np.ones((B, Gn))
        pm, pv = pm.astype(np.float32).astype(np.float64), pv.astype(np.float32).astype(np.float64)
        args = (x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gam), dev(bet), None if mask is None else dev(mask, torch.bool))
        if feature:
            out = M.ops.timestep_norm_fwd(*args, 1e-5)
        else:
            out = M.ops.group_timestep_norm_fwd(*args, G, 1e-5)
        torch.cuda.synchronize()
        y, cnt, mean, var = out[0], out[1], out[2], out[3]
        gam32, bet32 = gam.astype(np.float32).astype(np.float64), bet.astype(np.float32).astype(np.float64)
        yo, co, mo, vo = O.timestep_norm(x64, pc, pm, pv, gam32, bet32, mask, G)
        assert cnt.tolist() == co.tolist(), tag
        # fp32: groups of one or two channels have variances that are differences of nearly equal numbers, and the
        # reciprocal square root is the hardware's (1 ulp): 2e-4 instead of the 1e-4 of the other fp32 checks
        assert rel_err(host(y), yo) < max(TOL[dtype], 2e-4), tag
        assert rel_err(host(mean), mo) < 1e-4 and rel_err(host(var), vo) < 1e-4, tag
    assert M.ops.timestep_norm_status() == 0


@pytest.mark.parametrize("seed", range(10))
def test_norm_then_moving_average_sweep(seed):
    rng = np.random.default_rng(3000 + seed + SEED_SHIFT)
    for case in range(6):
        G = int(rng.choice([1, 2, 4]))
        dg = int(rng.choice([64, 64, 128, 32, 16]))           # 64 and 128 per group: the one-kernel block
        D = G * dg
        L = int(rng.choice([64, 300, 1024, 2048, 2050, 3072]))
        B = int(rng.choice([1, 2, 3]))
        N = int(rng.choice([2, 7, 16]))
        cplx = bool(rng.integers(0, 2))
        masked = rng.integers(0, 3) == 0
        with_state = bool(rng.integers(0, 2))
        out_layout = "input" if rng.integers(0, 2) else "rows"
        tag = (f"seed {seed} case {case}: B={B} L={L} D={D} G={G} N={N} cplx={cplx} masked={masked} "
               f"state={with_state} out={out_layout}")
        print(tag, flush=True)
        p, q, g = _coeffs(rng, D, N, cplx)
        om = rng.normal(size=D)
        gam = (rng.normal(size=D) * 0.1 + 1.0).astype(np.float32).astype(np.float64)
        bet = (rng.normal(size=D) * 0.1).astype(np.float32).astype(np.float64)
        x, x64 = rounded(rng.normal(size=(B, L, D)) * 1.5 + 0.3, torch.bfloat16)
        mask = None
        if masked:
            mask = np.zeros((B, L), bool); mask[0, L - L // 4:] = True
            if rng.integers(0, 2):
                mask[-1, :int(rng.integers(1, min(L, 1500)))] = True       # a row that starts padded (whole blocks too)
                mask[B // 2] |= rng.random(L) < 0.05
        h0 = None
        if with_state:
            h0 = (rng.normal(size=(B, D, N)) + (1j * rng.normal(size=(B, D, N)) if cplx else 0))
            h0 = h0.astype(np.complex64) if cplx else h0.astype(np.float32)
        pc = rng.integers(0, 30, size=B)
        pm = rng.normal(size=(B, G)).astype(np.float32).astype(np.float64)
        pv = (rng.random((B, G)) + 0.5).astype(np.float32).astype(np.float64)
        layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
        xn, y, cnt, mean, var, h = layer.norm_forward(
            x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gam), dev(bet), G, 1e-5,
            padding_mask=None if mask is None else dev(mask, torch.bool), h=None if h0 is None else dev(h0),
            want_state=with_state, out_layout=out_layout)
        torch.cuda.synchronize()
        xno, co, mo, vo = O.timestep_norm(x64, pc, pm, pv, gam, bet, mask, G)
        assert cnt.tolist() == co.tolist(), tag
        assert rel_err(host(xn), xno) < 2e-2, tag
        assert rel_err(host(mean), mo) < 1e-4 and rel_err(host(var), vo) < 1e-4, tag
        yo, ho = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, mask, h=h0, incremental=with_state)
        assert _out_err(host(y), yo) < 2e-2, tag
        if with_state:
            assert _state_err(np.real(host(h)), np.real(ho)) < 2e-3, tag
    assert M.ops.timestep_norm_status() == 0


@pytest.mark.parametrize("seed", range(8))
def test_norm_then_moving_average_sweep_fp32_fp16(seed):
    """The same call in fp32 / fp16: rows of 64 to 16 384 tokens go through the norm and the moving average on rows in
    time, shorter rows, more than 16 states and carried states into ragged rows through the library's own pair."""
    rng = np.random.default_rng(3500 + seed + SEED_SHIFT)
    for case in range(6):
        dtype = torch.float32 if rng.integers(0, 2) else torch.float16
        tol = 2e-4 if dtype is torch.float32 else 4e-3
        G = int(rng.choice([1, 2, 4]))
        D = G * int(rng.choice([64, 24, 128, 8]))
        L = int(rng.choice([40, 64, 300, 1024, 2048, 2050, 3072]))
        B = int(rng.choice([1, 2, 3]))
        N = int(rng.choice([2, 7, 16, 20]))
        cplx = bool(rng.integers(0, 2))
        masked = rng.integers(0, 3) == 0
        with_state = bool(rng.integers(0, 2))
        out_layout = "input" if rng.integers(0, 2) else "rows"
        tag = (f"seed {seed} case {case}: {dtype} B={B} L={L} D={D} G={G} N={N} cplx={cplx} masked={masked} "
               f"state={with_state} out={out_layout}")
        print(tag, flush=True)
        p, q, g = _coeffs(rng, D, N, cplx)
        om = rng.normal(size=D)
        gam = (rng.normal(size=D) * 0.1 + 1.0).astype(np.float32).astype(np.float64)
        bet = (rng.normal(size=D) * 0.1).astype(np.float32).astype(np.float64)
        x, x64 = rounded(rng.normal(size=(B, L, D)) * 1.5 + 0.3, dtype)
        mask = None
        if masked:
            mask = np.zeros((B, L), bool); mask[0, L - L // 4:] = True
            if rng.integers(0, 2):
                mask[-1, :int(rng.integers(1, min(L, 1500)))] = True
                mask[B // 2] |= rng.random(L) < 0.05
        h0 = None
        if with_state:
            h0 = (rng.normal(size=(B, D, N)) + (1j * rng.normal(size=(B, D, N)) if cplx else 0))
            h0 = h0.astype(np.complex64) if cplx else h0.astype(np.float32)
        pc = rng.integers(0, 30, size=B)
        pm = rng.normal(size=(B, G)).astype(np.float32).astype(np.float64)
        pv = (rng.random((B, G)) + 0.5).astype(np.float32).astype(np.float64)
        layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om))
        xn, y, cnt, mean, var, h = layer.norm_forward(
            x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gam), dev(bet), G, 1e-5,
            padding_mask=None if mask is None else dev(mask, torch.bool), h=None if h0 is None else dev(h0),
            want_state=with_state, out_layout=out_layout)
        torch.cuda.synchronize()
        assert y.shape == (B, D, L), tag
        xno, co, mo, vo = O.timestep_norm(x64, pc, pm, pv, gam, bet, mask, G)
        assert cnt.tolist() == co.tolist(), tag
        assert rel_err(host(xn), xno) < tol, tag
        assert rel_err(host(mean), mo) < 1e-4 and rel_err(host(var), vo) < 1e-4, tag
        yo, ho = O.ema_forward(host(xn).transpose(0, 2, 1), p, q, g, om, mask, h=h0, incremental=with_state)
        assert _out_err(host(y), yo) < tol, tag
        if with_state:
            assert _state_err(np.real(host(h)), np.real(ho)) < 2e-3, tag
    assert M.ops.timestep_norm_status() == 0


@pytest.mark.parametrize("seed", range(10))
def test_attention_sweep(seed):
    """EfficientAttention's forward with and without the weights: head sizes on both sides of what the one-kernel
    path takes (H1 64 / 128, H2 a multiple of 8 from 64 on, L from 64 on), lengths that end inside a tile."""
    rng = np.random.default_rng(4000 + seed + SEED_SHIFT)
    for case in range(6):
        dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
        L = int(rng.choice([1, 5, 63, 64, 65, 200, 256, 257, 700, 1024, 1300]))
        Nh = int(rng.choice([1, 2, 3]))
        H1 = int(rng.choice([8, 32, 64, 96, 128]))
        H2 = int(rng.choice([8, 24, 64, 72, 256, 264, 512]))
        B = int(rng.choice([1, 2]))
        causal = bool(rng.integers(0, 2))
        tag = f"seed {seed} case {case}: {dtype} B={B} L={L} Nh={Nh} H1={H1} H2={H2} causal={causal}"
        print(tag, flush=True)
        q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.7, dtype)
        k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.7, dtype)
        v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
        scale = float(rng.choice([0.5, 1.0, 3.0])) / np.sqrt(H1)
        yo, wo = O.attention(q64, k64, v64, scale, causal)
        y, w = M.ops.attention_fwd(q, k, v, scale, 0.0, causal)
        torch.cuda.synchronize()
        assert w is None, tag
        assert _out_err(host(y), yo, eps=2.0) < TOL[dtype], tag
        y2, w2 = M.ops.attention_fwd(q, k, v, scale, 0.0, causal, need_weights=True)
        torch.cuda.synchronize()
        assert _out_err(host(y2), yo, eps=2.0) < TOL[dtype], tag
        assert np.abs(host(w2) - wo).max() < (1e-5 if dtype is torch.float32 else 4e-3), tag


@pytest.mark.parametrize("seed", range(8))
def test_attention_backward_sweep(seed):
    """ops.attention_bwd from the forward's weights against the oracle's fp64 gradients: head sizes on both sides of
    what mega_attention_bwd takes (multiples of 8; the others go through the library products), lengths around the
    128- and 256-row tiles of its products and lengths that are not a multiple of 8, with and without the mask."""
    rng = np.random.default_rng(4500 + seed + SEED_SHIFT)
    for case in range(5):
        dtype = [torch.bfloat16, torch.float16, torch.float32][int(rng.integers(0, 3))]
        L = int(rng.choice([1, 5, 63, 64, 65, 127, 129, 200, 255, 257, 300, 515, 770]))
        Nh = int(rng.choice([1, 2, 3]))
        H1 = int(rng.choice([8, 12, 32, 64, 128]))
        H2 = int(rng.choice([8, 20, 24, 64, 72, 256, 264]))
        B = int(rng.choice([1, 2]))
        causal = bool(rng.integers(0, 2))
        tag = f"seed {seed} case {case}: {dtype} B={B} L={L} Nh={Nh} H1={H1} H2={H2} causal={causal}"
        print(tag, flush=True)
        q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.7, dtype)
        k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.7, dtype)
        v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
        dy, dy64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
        scale = float(rng.choice([0.5, 1.0, 2.0])) / np.sqrt(H1)
        _, w = M.ops.attention_fwd(q, k, v, scale, 0.0, causal, need_weights=True)
        got = M.ops.attention_bwd(dy, q, k, v, w, scale, causal)
        torch.cuda.synchronize()
        want = O.attention_bwd(dy64, q64, k64, v64, scale, causal)
        tol = {torch.float32: 2e-4, torch.bfloat16: 2e-2, torch.float16: 4e-3}[dtype]
        for name, g, ref in zip("qkv", got, want):
            e = host(g) - ref
            rms = np.sqrt((ref ** 2).mean())
            assert np.isfinite(host(g)).all(), tag + " " + name
            assert np.sqrt((e ** 2).mean()) < tol * max(rms, 1e-3), tag + " " + name
            assert np.abs(e).max() < 4 * tol * max(rms, np.abs(ref).max(), 1e-3), tag + " " + name


@pytest.mark.parametrize("seed", range(8))
def test_sequence_norm_sweep(seed):
    rng = np.random.default_rng(5000 + seed + SEED_SHIFT)
    for case in range(8):
        dtype = DTYPES[int(rng.integers(0, 3))]
        L = int(rng.choice([1, 2, 17, 64, 100, 513, 2048]))
        feature = rng.integers(0, 3) == 0
        G = None if feature else int(rng.choice([1, 2, 4, 16]))
        H = int(rng.choice([1, 8, 40, 200])) if feature else G * int(rng.choice([1, 4, 8, 64]))
        B = int(rng.choice([1, 3]))
        last = bool(rng.integers(0, 2))
        masked = bool(rng.integers(0, 2))
        if L * (H // (H if G is None else G)) < 8:
            L = 17              # a statistic over one or two values has variance ~ 0: rstd = eps^-1/2 amplifies rounding
        tag = f"seed {seed} case {case}: {dtype} B={B} L={L} H={H} G={G} length_last={last} masked={masked}"
        print(tag, flush=True)
        x, x64 = rounded(rng.normal(size=(B, H, L) if last else (B, L, H)) * 2.0 + 0.5, dtype)
        gam = (rng.normal(size=H) * 0.2 + 1.0).astype(np.float32).astype(np.float64)
        bet = (rng.normal(size=H) * 0.2).astype(np.float32).astype(np.float64)
        mask = None
        if masked and L > 1:
            mask = rng.random((B, L)) < 0.2
            mask[:, 0] = False                              # at least one valid token per row
        tm = None if mask is None else dev(mask, torch.bool)
        if feature:
            y, cnt, mean, rstd = M.ops.sequence_norm_fwd(x, dev(gam), dev(bet), tm, 1e-5, last)
        else:
            y, cnt, mean, rstd = M.ops.group_sequence_norm_fwd(x, dev(gam), dev(bet), tm, G, 1e-5, last)
        torch.cuda.synchronize()
        yo, co, mo, ro = O.sequence_norm(x64, gam, bet, mask, G, 1e-5, last)
        assert cnt.tolist() == co.tolist(), tag
        assert rel_err(host(y), yo) < TOL[dtype], tag
        assert rel_err(host(mean), mo) < 1e-4 and rel_err(host(rstd), ro) < 1e-3, tag


@pytest.mark.parametrize("seed", range(6))
def test_explicit_kernel_convolution_sweep(seed):
    """fftconv / bidirectional_fftconv with an explicit kernel: kernel lengths on both sides of the 512 lags from
    which the transform path takes over, row lengths up to its 16384-point limit and beyond."""
    rng = np.random.default_rng(6000 + seed + SEED_SHIFT)
    for case in range(5):
        dtype = DTYPES[int(rng.integers(0, 3))]
        L = int(rng.choice([1, 33, 511, 512, 513, 1000, 2048, 3000, 8192, 9000]))
        Lk = min(L, int(rng.choice([1, 7, 64, 511, 512, 600, 2048, 8192])))
        D = int(rng.choice([1, 3, 8]))
        B = int(rng.choice([1, 2, 3]))
        bidir = bool(rng.integers(0, 2))
        shift = bool(rng.integers(0, 2))
        tag = f"seed {seed} case {case}: {dtype} B={B} D={D} L={L} Lk={Lk} bidir={bidir} shift={shift}"
        print(tag, flush=True)
        x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
        k = (rng.normal(size=(2 * D if bidir else D, Lk)) * np.exp(-np.arange(Lk) / 200.0) * 0.3).astype(np.float32)
        if bidir:
            y = M.ops.bidirectional_fftconv(x, dev(k), shift)
            ref = O.bidirectional_conv(x64, k.astype(np.float64), shift)
        else:
            y = M.ops.fftconv(x, dev(k))
            ref = O.causal_conv(x64, np.pad(k.astype(np.float64), ((0, 0), (0, L - Lk))))
        torch.cuda.synchronize()
        assert rel_err(host(y), ref) < TOL[dtype], tag


@pytest.mark.parametrize("seed", range(8))
def test_moving_average_backward_sweep(seed):
    """ema_backward (input gradient + parameter-gradient sums) for one- and two-sided layers in both layouts."""
    rng = np.random.default_rng(7000 + seed + SEED_SHIFT)
    for case in range(6):
        dtype = [torch.float32, torch.bfloat16][int(rng.integers(0, 2))]
        L = int(rng.choice([1, 31, 64, 100, 256, 300, 511, 1024, 1100, 1544, 2048]))
        D = int(rng.choice([1, 5, 16, 24, 40]))
        B = int(rng.choice([1, 2, 3]))
        N = int(rng.choice([1, 2, 7, 16, 24, 32]))
        cplx = bool(rng.integers(0, 2))
        bidir = bool(rng.integers(0, 2))
        shift = bool(rng.integers(0, 2))
        layout = str(rng.choice(["bdl", "bld", "mixed"]))
        masked = bool(rng.integers(0, 2))
        tag = (f"seed {seed} case {case}: {dtype} B={B} D={D} N={N} L={L} cplx={cplx} bidir={bidir} shift={shift} "
               f"layout={layout} masked={masked}")
        print(tag, flush=True)
        p, q, g = _coeffs(rng, 2 * D if bidir else D, N, cplx)
        p = p.astype(np.float32).astype(np.float64)
        if cplx:
            q, g = q.astype(np.complex64).astype(np.complex128), g.astype(np.complex64).astype(np.complex128)
        else:
            q, g = q.astype(np.float32).astype(np.float64), g.astype(np.float32).astype(np.float64)
        om = rng.normal(size=D).astype(np.float32).astype(np.float64)
        x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
        dy, dy64 = rounded(rng.normal(size=(B, D, L)), dtype)
        if layout in ("bld", "mixed"):
            x = x.transpose(1, 2).contiguous().transpose(1, 2)
        if layout == "bld":
            dy = dy.transpose(1, 2).contiguous().transpose(1, 2)
        mask = (rng.random((B, L)) < 0.2) if masked else None
        tm = None if mask is None else torch.from_numpy(mask).to(DEV)
        layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om), bidir, None, shift)
        got = M.ops.ema_backward(dy, x, dev(p), dev(q), dev(g), dev(om), tm, layer=layer)
        torch.cuda.synchronize()
        ref = O.ema_backward(dy64, x64, p, q, g, om, mask, bidir, shift)
        assert rel_err(host(got[0]), ref[0]) < TOL[dtype], tag
        for a, b, name in zip(got[1:], ref[1:], ("dp", "dq", "dgamma", "domega")):
            a = host(a)
            if np.iscomplexobj(b) and cplx:
                assert rel_err(a.real, b.real) < 5e-4 and rel_err(a.imag, b.imag) < 5e-4, (tag, name)
            else:
                assert rel_err(np.real(a), np.real(b)) < 5e-4, (tag, name)


@pytest.mark.parametrize("seed", range(8))
def test_timestep_norm_backward_sweep(seed):
    rng = np.random.default_rng(8000 + seed + SEED_SHIFT)
    for case in range(6):
        dtype = DTYPES[int(rng.integers(0, 3))]
        L = int(rng.choice([1, 2, 15, 16, 17, 37, 96, 130, 257, 1000]))
        feature = rng.integers(0, 4) == 0
        G = None if feature else int(rng.choice([1, 2, 4, 5, 16]))
        H = int(rng.choice([1, 6, 24, 100])) if feature else G * int(rng.choice([1, 6, 8, 24, 64]))
        B = int(rng.choice([1, 2, 3]))
        masked = bool(rng.integers(0, 2))
        prior = bool(rng.integers(0, 2))
        tag = f"seed {seed} case {case}: {dtype} B={B} L={L} H={H} G={G} masked={masked} prior={prior}"
        print(tag, flush=True)
        GG = H if G is None else G
        x, x64 = rounded(rng.normal(size=(B, L, H)) * 1.3 + 0.2, dtype)
        dy, dy64 = rounded(rng.normal(size=(B, L, H)), dtype)
        mask = (rng.random((B, L)) < 0.25) if masked else None
        if mask is not None:
            mask[:, 0] = False
        pc = rng.integers(1, 5, B).astype(np.int64) if prior else np.zeros(B, np.int64)
        pm = (rng.normal(size=(B, GG)) * 0.2 * prior).astype(np.float32).astype(np.float64)
        pv = (rng.random((B, GG)) + 0.5 if prior else np.ones((B, GG))).astype(np.float32).astype(np.float64)
        gamma = (rng.normal(size=H) * 0.3 + 1).astype(np.float32).astype(np.float64)
        beta = rng.normal(size=H).astype(np.float32).astype(np.float64)
        dm = rng.normal(size=(B, GG)).astype(np.float32).astype(np.float64)
        dv = rng.normal(size=(B, GG)).astype(np.float32).astype(np.float64)
        tm = None if mask is None else torch.from_numpy(mask).to(DEV)
        if G is None:
            y, cnt, mu, var, cm, cr = M.ops.timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma),
                                                              dev(beta), tm, 1e-5)
            got = M.ops.timestep_norm_bwd(dy, dev(dm), dev(dv), x, dev(pm), cnt, cm, cr, dev(gamma), tm)
        else:
            y, cnt, mu, var, gm, cm, cr = M.ops.group_timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv),
                                                                        dev(gamma), dev(beta), tm, G, 1e-5)
            got = M.ops.group_timestep_norm_bwd(dy, dev(dm), dev(dv), x, dev(pm), cnt, gm, cm, cr, dev(gamma), tm, G)
        torch.cuda.synchronize()
        ocnt, ogm, ocm, ocr = O.timestep_norm_saved(x64, pc, pm, pv, mask, G, 1e-5)
        assert np.array_equal(host(cnt), ocnt), tag
        ref = O.timestep_norm_bwd(dy64, dm, dv, x64, pm, ocnt, ogm if G else None, ocm, ocr, gamma, mask, G)
        # fp32: the saved statistics come from the forward kernel (hardware reciprocal square root, 1 ulp) and the walk
        # runs over up to a thousand tokens from a first token whose variance is zero: a few 1e-4 is what fp32 leaves
        assert rel_err(host(got[0]), ref[0]) < max(TOL[dtype], 3e-4), tag
        for a, b in zip(got[1:], ref[1:]):
            assert rel_err(host(a), b) < 3e-4, tag
    assert M.ops.timestep_norm_status() == 0


@pytest.mark.parametrize("seed", range(10))
def test_gated_attention_layer_sweep(seed):
    """The whole MovingAverageGatedAttention forward in fp32 (a tight bound shows any wrong glue): widths that are
    not multiples of the vector sizes of the gate kernels, heads, chunk sizes above, at and below the length,
    both activations of the moving average, one- and two-sided layers with padding."""
    rng = np.random.default_rng(9000 + seed + SEED_SHIFT)
    for case in range(4):
        heads = int(rng.choice([1, 2, 4]))
        S = heads * int(rng.choice([2, 6, 8, 16]))
        E = heads * int(rng.choice([4, 10, 16, 24, 64]))
        G = int(rng.choice([1, 2, 4]))
        D = G * int(rng.choice([3, 8, 10, 16, 64]))
        N = int(rng.choice([1, 4, 16]))
        C = int(rng.choice([16, 64, 128]))
        nchunks = int(rng.choice([1, 1, 2, 5]))
        L = C * nchunks if nchunks > 1 else int(rng.choice([C, C // 2 + 3, 7]))
        B = int(rng.choice([1, 2, 3]))
        act = str(rng.choice(['silu', 'rmsnorm']))
        moving = str(rng.choice(['cema', 'ema']))
        bidir = bool(rng.integers(0, 2))
        masked = bidir and bool(rng.integers(0, 2))
        tag = (f"seed {seed} case {case}: B={B} L={L} D={D} S={S} E={E} N={N} G={G} C={C} heads={heads} act={act} "
               f"moving={moving} bidir={bidir} masked={masked}")
        print(tag, flush=True)
        torch.manual_seed(9000 + 10 * seed + case + SEED_SHIFT)
        layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_layer=moving, moving_act=act,
                                              norm_num_groups=G, num_heads=heads, bidirectional=bidir).to(DEV).eval()
        with torch.no_grad():
            for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
                prm.normal_(0, 0.15)
            layer.gamma.normal_(0, 0.1); layer.beta.normal_(0, 0.1)
            layer.norm.weight.normal_(0, 0.1); layer.norm.bias.normal_(0, 0.1)
            if isinstance(layer.move_act, M.RMSNorm):
                layer.move_act.weight.normal_(0, 0.2)
        p, q, g = layer.move.coeffs()
        P = dict(norm_weight=host(layer.norm.weight), norm_bias=host(layer.norm.bias), p=host(p.squeeze(-1)),
                 q=host(q.squeeze(-1)), ema_gamma=host(g), omega=host(layer.move.omega).reshape(-1),
                 v_w=host(layer.v_proj.weight), v_b=host(layer.v_proj.bias), mx_w=host(layer.mx_proj.weight),
                 mx_b=host(layer.mx_proj.bias), h_w=host(layer.h_proj.weight), gamma=host(layer.gamma),
                 beta=host(layer.beta))
        if isinstance(layer.move_act, M.RMSNorm):
            P['rms_weight'] = host(layer.move_act.weight)
        x = torch.randn(B, L, D, device=DEV)
        mask = None
        if masked:
            mask = np.zeros((B, L), bool); mask[0, L - max(L // 4, 1):] = True
        with torch.no_grad():
            y, _ = layer(x, None if mask is None else dev(mask, torch.bool))
        torch.cuda.synchronize()
        yo = O.gated_attention_layer(host(x), P, chunk=C, num_heads=heads, moving_act=act, num_groups=G,
                                     bidirectional=bidir, padding_mask=mask)
        keep = np.ones((B, L), bool) if mask is None else ~mask
        assert rel_err(host(y)[keep], yo[keep]) < 2e-4, tag
        # the training path (autograd functions and backward kernels) sees the same shapes: same output, and
        # gradients that are finite and not all zero
        layer.train()
        xg = x.clone().requires_grad_(True)
        yt, _ = layer(xg, None if mask is None else dev(mask, torch.bool))
        assert rel_err(host(yt)[keep], host(y)[keep]) < 2e-4, tag
        wgt = torch.randn_like(yt)
        if mask is not None:
            wgt = wgt * dev(~mask).unsqueeze(-1)
        (yt * wgt).sum().backward()
        torch.cuda.synchronize()
        grads = [xg.grad] + [prm.grad for prm in layer.parameters() if prm.requires_grad]
        assert all(gr is not None and torch.isfinite(gr).all() for gr in grads), tag
        assert xg.grad.abs().max().item() > 0, tag
        # the 16-bit kernels (other vector widths and alignment rules) on the same shape: close to the fp32 result
        # in the root mean square, and a training step that runs
        import copy
        for dt16 in (torch.bfloat16, torch.float16):
            l16 = copy.deepcopy(layer).to(dt16).eval()
            with torch.no_grad():
                y16, _ = l16(x.to(dt16), None if mask is None else dev(mask, torch.bool))
            e = (host(y16) - host(y))[keep]
            assert np.isfinite(e).all() and np.sqrt(np.mean(e ** 2)) < 5e-2 * np.sqrt(np.mean(host(y)[keep] ** 2)), (tag, dt16)
            l16.train()
            x16 = x.to(dt16).requires_grad_(True)
            yt16, _ = l16(x16, None if mask is None else dev(mask, torch.bool))
            (yt16.float() * wgt).sum().backward()
            torch.cuda.synchronize()
            e = (host(x16.grad) - host(xg.grad))
            # (a z of two or four features makes the q / k normalisation ill-conditioned: the 16-bit run differentiates
            # at a slightly different point and the bound means nothing there; finite gradients are still asked for)
            bound16 = 0.1 if S >= 8 else 10.0
            ok16 = np.isfinite(e).all() and np.sqrt(np.mean(e ** 2)) < bound16 * np.sqrt(np.mean(host(xg.grad) ** 2)) + 1e-6
            if not ok16:        # which parameters' gradients are off, for the message
                rep = {n: float(np.sqrt(np.mean((host(a.grad) - host(b.grad)) ** 2)) / (np.sqrt(np.mean(host(b.grad) ** 2)) + 1e-12))
                       for (n, a), (_, b) in zip(l16.named_parameters(), layer.named_parameters()) if a.grad is not None}
                rep["x"] = float(np.sqrt(np.mean(e ** 2)) / (np.sqrt(np.mean(host(xg.grad) ** 2)) + 1e-12))
                print("16-bit gradients against fp32, relative rms error:", {k: round(v, 3) for k, v in rep.items()}, flush=True)
            assert ok16, (tag, dt16)
        if L <= 128:
            # a few entries of the input and projection gradients against central differences of the oracle
            okw = dict(chunk=C, num_heads=heads, moving_act=act, num_groups=G, bidirectional=bidir, padding_mask=mask)
            w64, x64 = host(wgt), host(x)
            loss = lambda Pd, xx: (O.gated_attention_layer(xx, Pd, **okw) * w64).sum()
            eps = 1e-5
            gx = host(xg.grad)
            for _ in range(2):
                idx = tuple(int(rng.integers(0, n)) for n in x64.shape)
                xp, xm = x64.copy(), x64.copy()
                xp[idx] += eps; xm[idx] -= eps
                fd = (loss(P, xp) - loss(P, xm)) / (2 * eps)
                assert abs(fd - gx[idx]) < 3e-3 * (np.abs(gx).max() + 1e-6), (tag, "x", idx, fd, gx[idx])
            for name, prm in (("mx_w", layer.mx_proj.weight), ("gamma", layer.gamma), ("norm_weight", layer.norm.weight)):
                gp = host(prm.grad)
                idx = tuple(int(rng.integers(0, n)) for n in P[name].shape)
                Pp = dict(P); Pp[name] = P[name].copy(); Pp[name][idx] += eps
                Pm = dict(P); Pm[name] = P[name].copy(); Pm[name][idx] -= eps
                fd = (loss(Pp, x64) - loss(Pm, x64)) / (2 * eps)
                assert abs(fd - gp[idx]) < 3e-3 * (np.abs(gp).max() + 1e-6), (tag, name, idx, fd, gp[idx])


@pytest.mark.parametrize("seed", range(8))
def test_decode_sweep(seed):
    """Streaming decode of the norm -> moving-average pair: tokens arrive one at a time and in batches of random
    sizes (the multi-token kernel where the coefficient shape allows it), against the oracle on the whole sequence."""
    rng = np.random.default_rng(10000 + seed + SEED_SHIFT)
    for case in range(4):
        dtype = [torch.float32, torch.bfloat16, torch.float16][int(rng.integers(0, 3))]
        G = int(rng.choice([1, 2, 3, 8]))
        D = G * int(rng.choice([1, 4, 24, 64]))
        N = int(rng.choice([1, 2, 4, 6, 8, 16, 32]))
        B = int(rng.choice([1, 2, 5]))
        cplx = bool(rng.integers(0, 2))
        T = int(rng.choice([1, 9, 70, 150]))
        tag = f"seed {seed} case {case}: {dtype} B={B} D={D} G={G} N={N} cplx={cplx} T={T}"
        print(tag, flush=True)
        p, q, g = _coeffs(rng, D, N, cplx)
        om = rng.normal(size=D)
        nw = (rng.normal(size=D) * 0.1).astype(np.float32).astype(np.float64)
        nb = (rng.normal(size=D) * 0.1).astype(np.float32).astype(np.float64)
        x, x64 = rounded(rng.normal(size=(B, T, D)) + 0.2, dtype)
        step = M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
        xs, ys, a = [], [], 0
        while a < T:
            K = min(T - a, int(rng.choice([1, 1, 2, 5, 64, 100])))
            if K == 1 and rng.integers(0, 2):
                xn, y = step(x[:, a])
                xn, y = xn.unsqueeze(1), y.unsqueeze(1)
            else:
                xn, y = step.steps(x[:, a:a + K])
            xs.append(xn); ys.append(y)
            a += K
        xn_s, y_s = torch.cat(xs, 1), torch.cat(ys, 1)
        torch.cuda.synchronize()
        tol = {torch.float32: 1e-4, torch.bfloat16: 2e-2, torch.float16: 4e-3}[dtype]
        xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, None, G)
        assert step.count.tolist() == [T] * B, tag
        assert rel_err(host(xn_s), xno) < tol, tag
        assert rel_err(host(step.mean), mu) < 1e-4 and rel_err(host(step.var), v) < 1e-4, tag
        yo, ho = O.ema_forward(host(xn_s).transpose(0, 2, 1), p, q, g, om, incremental=True)
        assert rel_err(host(y_s), yo.transpose(0, 2, 1)) < tol, tag
        assert _state_err(np.real(host(step.state)), np.real(ho)) < 1e-4, tag


@pytest.mark.parametrize("seed", range(8))
def test_streaming_equals_one_shot_sweep(seed):
    """A causal gated-attention layer fed slices of random lengths with carried state (norm statistics, moving-
    average state, the partial chunk's keys and values) gives what one call on the whole sequence gives; a batch
    of bf16 follows the fp32 result."""
    rng = np.random.default_rng(11000 + seed + SEED_SHIFT)
    for case in range(3):
        heads = int(rng.choice([1, 2]))
        S = heads * int(rng.choice([4, 8, 16]))
        E = heads * int(rng.choice([8, 24, 64]))
        G = int(rng.choice([1, 2, 4]))
        D = G * int(rng.choice([8, 16, 64]))
        N = int(rng.choice([2, 16]))
        C = int(rng.choice([16, 64, 128]))
        L = C * int(rng.choice([1, 2, 4])) + int(rng.choice([0, 0, 5]))
        B = int(rng.choice([1, 2]))
        act = str(rng.choice(['silu', 'rmsnorm']))
        tag = f"seed {seed} case {case}: B={B} L={L} D={D} S={S} E={E} N={N} G={G} C={C} heads={heads} act={act}"
        print(tag, flush=True)
        torch.manual_seed(11000 + 10 * seed + case + SEED_SHIFT)
        layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_act=act, norm_num_groups=G,
                                              num_heads=heads).to(DEV).eval()
        with torch.no_grad():
            for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
                prm.normal_(0, 0.15)
        x = torch.randn(B, L, D, device=DEV)
        # slices the reference's cache logic takes (moving_average_gated_attention.py:332-387): whole chunks from
        # a chunk boundary, or a piece that stays inside the current chunk
        cuts = [0]
        while cuts[-1] < L:
            a = cuts[-1]
            room = C - a % C
            if a % C == 0:
                step = int(rng.choice([1, 3, C // 2, C, 2 * C]))
                step = step if (step <= C or a + step <= L - L % C) else C
            else:
                step = int(rng.choice([1, 2, room]))
            cuts.append(min(L, a + min(step, room if step < C else step)))
        with torch.no_grad():
            if L % C == 0 or L < C:
                full, _ = layer(x)
            else:                                   # a one-shot call wants whole chunks: the whole part, then the rest
                st = {}
                full = torch.cat([layer(x[:, :L - L % C], None, st)[0], layer(x[:, L - L % C:], None, st)[0]], 1)
            state = {}
            parts = [layer(x[:, a:b], None, state)[0] for a, b in zip(cuts[:-1], cuts[1:])]
        torch.cuda.synchronize()
        assert rel_err(host(torch.cat(parts, 1)), host(full)) < 2e-4, (tag, cuts)
    assert M.ops.timestep_norm_status() == 0


@pytest.mark.parametrize("seed", range(8))
def test_kernel_generation_and_state_operators_sweep(seed):
    """ema_parameters (kernel and carried-state bias) and ema_hidden (state after the last token), forward and
    backward, at operator level (fairseq/csrc/ops/ema_parameters.cc:80-286, ema_hidden.cc:66-194): state counts
    from 1 to 32, lengths from 1 to past a tile, with and without a carried state."""
    rng = np.random.default_rng(12000 + seed + SEED_SHIFT)
    for case in range(5):
        D = int(rng.choice([1, 3, 16, 40]))
        N = int(rng.choice([1, 2, 7, 16, 32]))
        L = int(rng.choice([1, 2, 31, 64, 100, 513]))
        B = int(rng.choice([1, 2, 3]))
        with_h = bool(rng.integers(0, 2))
        tag = f"seed {seed} case {case}: B={B} D={D} N={N} L={L} h={with_h}"
        print(tag, flush=True)
        p, q, g = _coeffs(rng, D, N, True)
        p = p.astype(np.float32).astype(np.float64)
        q, g = q.astype(np.complex64).astype(np.complex128), g.astype(np.complex64).astype(np.complex128)
        h = None
        if with_h:
            h = (rng.normal(size=(B, D, N)) + 1j * rng.normal(size=(B, D, N))).astype(np.complex64).astype(np.complex128)
        x, x64 = rounded(rng.normal(size=(B, D, L)), torch.float32)
        tq = dev(q)
        th = None if h is None else dev(h)
        w, bias, _ = M.ops.ema_parameters_fwd(dev(p), tq.log(), dev(g), th, L)
        assert rel_err(host(w), O.ema_kernel(p, q, g, L)) < 1e-4, tag
        if with_h:
            assert rel_err(host(bias), O.ema_bias(q, g, h, L)) < 1e-4, tag
        hy, _ = M.ops.ema_hidden_fwd(x, dev(p), tq.log(), th)
        ho = O.ema_hidden(x64, p, q, h)
        assert rel_err(np.real(host(hy)), np.real(ho)) < 1e-4 and rel_err(np.imag(host(hy)), np.imag(ho)) < 1e-4, tag
        # backward of both
        dk = rng.normal(size=(D, L)).astype(np.float32).astype(np.float64)
        db = rng.normal(size=(B, D, L)).astype(np.float32).astype(np.float64) if with_h else None
        dp, dq, dg, dh = M.ops.ema_parameters_bwd(dev(dk), None if db is None else dev(db), dev(p), tq.log(), dev(g), th)
        rp, rq, rg = O.ema_kernel_bwd(dk, p, q, g)
        if with_h:
            bq, bg, bh = O.ema_bias_bwd(db, q, g, h)
            rq, rg = rq + bq, rg + bg
            assert _state_err(np.real(host(dh)), np.real(bh)) < 5e-4 and _state_err(np.imag(host(dh)), np.imag(bh)) < 5e-4, tag
        assert rel_err(host(dp), rp) < 5e-4, tag
        for a, r_, name in ((dq, rq, "dq"), (dg, rg, "dgamma")):
            a = host(a)
            assert rel_err(a.real, r_.real) < 5e-4 and rel_err(a.imag, r_.imag) < 5e-4, (tag, name)
        dy = (rng.normal(size=(B, D, N)) + 1j * rng.normal(size=(B, D, N))).astype(np.complex64).astype(np.complex128)
        dx, dp2, dq2, dh2 = M.ops.ema_hidden_bwd(dev(dy), x, dev(p), tq.log(), th)
        torch.cuda.synchronize()
        ox, op_, oq, oh = O.ema_hidden_bwd(dy, x64, p, q, h)
        assert rel_err(host(dx), ox) < 5e-4 and rel_err(host(dp2), op_) < 5e-4, tag
        a = host(dq2)
        assert rel_err(a.real, oq.real) < 5e-4 and rel_err(a.imag, oq.imag) < 5e-4, tag
        if with_h:
            a = host(dh2)
            assert _state_err(a.real, oh.real) < 5e-4 and _state_err(a.imag, oh.imag) < 5e-4, tag
