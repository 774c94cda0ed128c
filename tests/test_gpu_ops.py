"""The remaining operator entry points on the GPU against the oracle."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, rel_err
from gpu_util import DEV, TOL, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu


def test_ema_parameters_and_hidden_ops():
    rng = np.random.default_rng(21)
    K, N, L, B = 40, 16, 300, 3
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    h = rng.normal(size=(B, K, N)) + 1j * rng.normal(size=(B, K, N))
    tq = dev(q)
    w, b, _ = M.ops.ema_parameters_fwd(dev(p), tq.log(), dev(g), dev(h), L)
    assert rel_err(host(w), O.ema_kernel(p, q, g, L)) < 1e-4
    assert rel_err(host(b), O.ema_bias(q, g, h, L)) < 1e-4
    w0, b0, _ = M.ops.ema_parameters_fwd(dev(p), tq.log(), dev(g), None, 1)
    assert b0 is None and rel_err(host(w0), O.ema_kernel(p, q, g, 1)) < 1e-5
    x, x64 = rounded(rng.normal(size=(B, K, L)), torch.bfloat16)
    hh, _ = M.ops.ema_hidden_fwd(x, dev(p), tq.log(), dev(h))
    ref = O.ema_hidden(x64, p, q, h)
    assert rel_err(np.real(host(hh)), ref.real) < 1e-4 and rel_err(np.imag(host(hh)), ref.imag) < 1e-4


def test_long_kernel_phase_accuracy():
    """|q| close to 1 and 16k lags: the phase l*theta must not drift in fp32."""
    K, N, L = 4, 16, 16384
    rng = np.random.default_rng(22)
    mag = 1 - 10 ** rng.uniform(-5, -3, size=(K, N))
    q = mag * np.exp(1j * rng.uniform(0, np.pi, size=(K, N)))
    p = rng.random((K, N)); g = rng.normal(size=(K, N)) + 0j
    lq = dev(q).log()
    w, _, _ = M.ops.ema_parameters_fwd(dev(p), lq, dev(g), None, L)
    logq = host(lq)                                # exactly the complex64 values the op is handed
    ref = np.real((p[..., None] * g[..., None] * np.exp(np.arange(L) * logq[..., None])).sum(1))
    assert rel_err(host(w), ref) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Lk", [700, 1, 33])
def test_long_conv(dtype, Lk):
    rng = np.random.default_rng(23)
    B, D, L = 2, 6, 700
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    k = (rng.normal(size=(2 * D, Lk)) * 0.2).astype(np.float32)
    y = M.ops.fftconv(x, dev(k[:D]))
    assert rel_err(host(y), O.causal_conv(x64, np.pad(k[:D].astype(np.float64), ((0, 0), (0, L - Lk))))) < TOL[dtype]
    for shift in (True, False):
        y = M.ops.bidirectional_fftconv(x, dev(k), shift)
        assert rel_err(host(y), O.bidirectional_conv(x64, k.astype(np.float64), shift)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,D,L,Lk", [(3, 5, 4096, 4096), (1, 4, 5000, 3000), (2, 3, 8192, 8192), (5, 2, 1500, 512),
                                      (2, 600, 2048, 2048)])
def test_long_conv_transform_path(dtype, B, D, L, Lk):
    """Kernels of 512 lags and more go through the Fourier transform in LDS (M = pow2ceil(L + Lk) <= 16384 points):
    odd batch sizes (rows travel in pairs), M from 2048 to 16384, many channels; against numpy's convolution."""
    print(f"case {dtype} B={B} D={D} L={L} Lk={Lk}", flush=True)
    rng = np.random.default_rng(27)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    k = (rng.normal(size=(2 * D, Lk)) * np.exp(-np.arange(Lk) / 300.0) * 0.3).astype(np.float32)
    sel = slice(0, min(D, 8))                      # the oracle's convolution is O(L Lk) per row
    y = M.ops.fftconv(x, dev(k[:D]))
    ref = O.causal_conv(x64[:, sel], np.pad(k[:D][sel].astype(np.float64), ((0, 0), (0, L - Lk))))
    assert rel_err(host(y)[:, sel], ref) < TOL[dtype]
    for shift in (True, False):
        y = M.ops.bidirectional_fftconv(x, dev(k), shift)
        kk = np.concatenate([k[:D][sel], k[D:][sel]], 0).astype(np.float64)
        assert rel_err(host(y)[:, sel], O.bidirectional_conv(x64[:, sel], kk, shift)) < TOL[dtype]
    if D > 8:                                      # the remaining channels against the first ones' code path: linearity
        y2 = M.ops.fftconv(2 * x, dev(k[:D]))
        assert rel_err(host(y2), 2 * host(M.ops.fftconv(x, dev(k[:D])))) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(3, 5, 40, 40), (2, 17, 300), (2, 64, 2048), (1, 6, 3)])
@pytest.mark.parametrize("causal", [False, True])
def test_attention_softmax(dtype, shape, causal):
    rng = np.random.default_rng(24)
    a = rng.normal(size=shape) * 3
    a[..., 0, :] = -np.inf
    x, x64 = rounded(a, dtype)
    y = M.AttentionSoftmax(use_causal_mask=causal).eval()(x)
    yo = O.attention_softmax(x64, causal)
    assert np.abs(host(y) - yo).max() < (1e-5 if dtype == torch.float32 else 4e-3)
    assert torch.all(y[..., 0, :] == 0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,Nh,H1,H2", [(2, 50, 1, 16, 24), (1, 130, 4, 32, 64), (2, 7, 2, 5, 3)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention(dtype, B, L, Nh, H1, H2, causal):
    rng = np.random.default_rng(25)
    q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    y, w = M.ops.attention_fwd(q, k, v, 0.8, 0.0, causal, need_weights=True)
    yo, wo = O.attention(q64, k64, v64, 0.8, causal)
    assert rel_err(host(y), yo) < TOL[dtype]
    assert np.abs(host(w) - wo).max() < (1e-5 if dtype == torch.float32 else 4e-3)
    if Nh == 1:
        ym = M.EfficientAttention(scale=0.8, use_causal_mask=causal).eval()(q[:, :, 0], k[:, :, 0], v[:, :, 0])
        assert torch.equal(ym, y[:, :, 0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,Nh,H1,H2", [(2, 300, 2, 64, 256), (1, 1000, 1, 128, 512), (1, 129, 3, 32, 256),
                                          (1, 64, 1, 96, 256), (1, 2048, 2, 128, 320), (3, 520, 1, 64, 72),
                                          (2, 700, 2, 128, 1024), (1, 300, 1, 64, 520), (1, 1100, 3, 128, 768),
                                          (1, 2048, 1, 64, 1024)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_no_weights(dtype, B, L, Nh, H1, H2, causal):
    """No weights requested (the inference call of the layer), at sizes where the matrix-core GEMMs
    run many tiles; also against the call that returns the weights."""
    print(f"case {dtype} B={B} L={L} Nh={Nh} H1={H1} H2={H2} causal={causal}", flush=True)
    rng = np.random.default_rng(26)
    q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.7, dtype)
    k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.7, dtype)
    v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    scale = 1.0 / np.sqrt(H1) * 2.0
    y, w = M.ops.attention_fwd(q, k, v, scale, 0.0, causal)
    assert w is None
    torch.cuda.synchronize()
    yo, _ = O.attention(q64, k64, v64, scale, causal)
    # the probabilities enter the second product rounded to 16 bits (as the reference's do: its softmax
    # output has the activation dtype): over 10^5..10^6 outputs the largest deviation sits ~5 sigma out,
    # so the denominator floor of the error measure is 2 rms here (eps = 2) instead of 1 rms
    assert rel_err(host(y), yo, eps=2.0) < TOL[dtype]
    y2, _ = M.ops.attention_fwd(q, k, v, scale, 0.0, causal, need_weights=True)
    assert rel_err(host(y), host(y2), eps=2.0) < 2 * TOL[dtype]      # two 16-bit results


@pytest.mark.parametrize("causal", [True, False])
@pytest.mark.parametrize("gain", [6.0, 20.0])
def test_attention_wide_score_range(gain, causal):
    """Scores that spread over tens to hundreds of units and whose row maximum keeps rising along the keys (a
    drift in k): the running maximum of the one-kernel path moves by more than its rescaling threshold many times
    per row, late keys dominate early ones by far more than 2^24."""
    rng = np.random.default_rng(27)
    B, L, Nh, H1, H2 = 1, 1536, 2, 128, 256
    drift = np.linspace(0.0, 1.0, L)[None, :, None, None]
    q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5 + 0.3, torch.bfloat16)
    k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5 + 0.3 * drift, torch.bfloat16)
    v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), torch.bfloat16)
    scale = gain / np.sqrt(H1)
    y, _ = M.ops.attention_fwd(q, k, v, scale, 0.0, causal)
    torch.cuda.synchronize()
    yo, _ = O.attention(q64, k64, v64, scale, causal)
    assert np.isfinite(host(y)).all()
    assert rel_err(host(y), yo, eps=2.0) < TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_silu(dtype, n):
    """The activation alone, out of place, in place, and on a view that starts off the 16-byte boundary."""
    rng = np.random.default_rng(28)
    a, a64 = rounded(rng.normal(size=n + 3) * 3, dtype)
    ref = a64 / (1.0 + np.exp(-a64))
    tol = 1e-6 if dtype is torch.float32 else TOL[dtype]
    y = M.ops.silu(a)
    assert y.data_ptr() != a.data_ptr() and rel_err(host(y), ref) < tol
    view = a[1:n + 1]
    assert rel_err(host(M.ops.silu(view)), ref[1:n + 1]) < tol
    b = a.clone()
    assert M.ops.silu(b, inplace=True).data_ptr() == b.data_ptr() and rel_err(host(b), ref) < tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [1, 7, 4096, 100003])
def test_swiglu(dtype, n):
    rng = np.random.default_rng(26)
    a, a64 = rounded(rng.normal(size=n) * 3, dtype)
    b, b64 = rounded(rng.normal(size=n), dtype)
    assert rel_err(host(M.ops.swiglu(a, b)), O.swiglu(a64, b64)) < TOL[dtype]


# ----------------------------------------------------------------------------------------------
# per-token glue of the gated-attention layer; operands are slices of a wider row (the layout the
# layer hands over) and odd sizes take the element-wise fallback
# ----------------------------------------------------------------------------------------------
def _wide(rng, shape, width, off, dtype):
    """A [..., W] slice starting at column `off` of a [..., width] tensor, and its values."""
    t, t64 = rounded(rng.normal(size=shape[:-1] + (width,)) * 1.5, dtype)
    return t[..., off:off + shape[-1]], t64[..., off:off + shape[-1]]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,width,off", [((2, 33, 256), 256, 0), ((3, 17, 1024), 1304, 24), ((5, 77), 91, 3)])
def test_rms_norm(dtype, shape, width, off):
    rng = np.random.default_rng(41)
    x, x64 = _wide(rng, shape, width, off, dtype)
    w = rng.normal(size=shape[-1]) + 1
    assert rel_err(host(M.ops.rms_norm_fwd(x, dev(w), 1e-5)), O.rms_norm(x64, w, 1e-5)) < TOL[dtype]
    assert rel_err(host(M.ops.rms_norm_fwd(x, None, 1e-3)), O.rms_norm(x64, None, 1e-3)) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,S,heads,chunk,width,off", [(2, 64, 128, 1, 64, 128, 0), (1, 96, 64, 4, 32, 200, 72),
                                                         (3, 40, 36, 2, 40, 50, 6), (1, 4096, 512, 4, 2048, 512, 0)])
def test_gate_qk(dtype, B, L, S, heads, chunk, width, off):
    rng = np.random.default_rng(42)
    z, z64 = _wide(rng, (B, L, S), width, off, dtype)
    g = rng.normal(size=(2, S)) * 0.3 + 1
    b = rng.normal(size=(2, S)) * 0.3
    Hd = S // heads
    freqs = (1.0 / (10000.0 ** (np.arange(0, Hd, 2) / Hd))).astype(np.float32)
    q, k = M.ops.gate_qk_fwd(z, dev(g), dev(b), dev(freqs), heads, chunk)
    zn = z64 / np.maximum(np.sqrt((z64 * z64).sum(-1, keepdims=True)), 1e-5)
    for got, i in ((q, 0), (k, 1)):
        a = (zn * g[i] + b[i]).reshape(B * (L // chunk), chunk, heads, Hd)
        ref = O.rotary(a.transpose(0, 2, 1, 3)).transpose(0, 2, 1, 3).reshape(B, L, S)
        # positions reach 2047 rad in fp32: the angle itself carries ~1e-4 absolute error there
        assert rel_err(host(got), ref) < max(TOL[dtype], 5e-4)
    # a zero row stays finite (the norm is clamped at eps)
    zz = torch.zeros(1, 2, S, dtype=dtype, device=DEV)
    q0, k0 = M.ops.gate_qk_fwd(zz, dev(g), dev(b), dev(freqs), heads, 2)
    assert torch.isfinite(q0).all() and torch.isfinite(k0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("shape,width,off", [((2, 50, 512), 1100, 80), ((4, 9, 35), 35, 0), ((1, 5000, 64), 72, 8)])
def test_gate_mul_and_out(dtype, shape, width, off):
    rng = np.random.default_rng(43)
    a, a64 = rounded(rng.normal(size=shape), dtype)
    r, r64 = _wide(rng, shape, width, off, dtype)
    assert rel_err(host(M.ops.gate_mul_fwd(a, r)), a64 * O._silu(r64)) < TOL[dtype]
    u, u64 = _wide(rng, shape, width, 0, dtype)
    hx, hx64 = _wide(rng, shape, width, off, dtype)
    hp, hp64 = rounded(rng.normal(size=shape), dtype)
    res, res64 = rounded(rng.normal(size=shape), dtype)
    ref = res64 + O._sigmoid(u64) * (O._silu(hx64 + hp64) - res64)
    assert rel_err(host(M.ops.gate_out_fwd(res, u, hx, hp)), ref) < TOL[dtype]


def test_glue_rejects_bad_arguments():
    z = torch.zeros(2, 4, 30, device=DEV)
    g = torch.ones(2, 30, device=DEV)
    with pytest.raises(RuntimeError):
        M.ops.gate_qk_fwd(z, g, g, torch.ones(5, device=DEV), 4, 4)       # 30 does not split into 4 heads
    with pytest.raises(RuntimeError):
        M.ops.gate_mul_fwd(torch.zeros(2, 8, device=DEV), torch.zeros(2, 9, device=DEV))
    with pytest.raises(RuntimeError):
        M.ops.rms_norm_fwd(torch.zeros(2, 8), None, 1e-5)                  # CPU tensor: no CPU path


# ----------------------------------------------------------------------------------------------
# SequenceNorm
# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,H,G,last,masked", [
    (2, 100, 64, 8, False, True),       # [B, L, H], vectors of 8 channels inside a group
    (1, 4096, 1024, 16, False, False),  # the headline geometry, 128 tiles to combine
    (2, 70, 48, 2, False, True),        # 24 channels per group
    (3, 33, 30, 5, False, True),        # 6 channels per group: element-wise path
    (2, 45, 24, None, False, True),     # per feature
    (2, 256, 64, 8, True, True),        # [B, H, L], 16-byte rows
    (2, 77, 40, 4, True, True),         # [B, H, L], odd row length
    (1, 16384, 32, None, True, False),  # long rows, per feature
])
def test_sequence_norm(dtype, B, L, H, G, last, masked):
    rng = np.random.default_rng(81)
    x, x64 = rounded(rng.normal(size=(B, H, L) if last else (B, L, H)) * 1.5 + 0.7, dtype)
    gamma = (rng.normal(size=H) * 0.3 + 1).astype(np.float32)
    beta = rng.normal(size=H).astype(np.float32)
    mask = (rng.random((B, L)) < 0.3) if masked else None
    if mask is not None:
        mask[0, :] = False
    tm = None if mask is None else torch.from_numpy(mask).to(DEV)
    if G is None:
        y, n, mu, r = M.ops.sequence_norm_fwd(x, dev(gamma), dev(beta), tm, 1e-5, last)
    else:
        y, n, mu, r = M.ops.group_sequence_norm_fwd(x, dev(gamma), dev(beta), tm, G, 1e-5, last)
    yo, no, muo, ro = O.sequence_norm(x64, gamma, beta, mask, G, 1e-5, last)
    assert np.array_equal(host(n), no)
    assert rel_err(host(mu), muo) < 1e-4 and rel_err(host(r), ro) < 1e-4
    assert rel_err(host(y), yo) < TOL[dtype]


def test_sequence_norm_module_and_edge_cases():
    rng = np.random.default_rng(82)
    B, H, L = 2, 32, 60
    mod = M.SequenceNorm(H, 4).to(DEV).eval()
    with torch.no_grad():
        mod.weight.normal_(0, 0.2); mod.bias.normal_(0, 0.2)
    x64 = rng.normal(size=(B, H, L))
    mask = np.zeros((B, L), bool)
    mask[1, :] = True                                     # a fully padded row: zeros out, finite statistics
    mask[0, 50:] = True
    with torch.no_grad():
        y = mod(dev(x64), torch.from_numpy(mask).to(DEV))
    yo = O.sequence_norm(x64.astype(np.float32).astype(np.float64), host(mod.weight) + 1, host(mod.bias), mask, 4, 1e-5, True)[0]
    assert rel_err(host(y), yo) < 1e-4 and torch.isfinite(y).all() and float(y[1].abs().max()) == 0.0
    with pytest.raises(RuntimeError):
        M.ops.group_sequence_norm_fwd(dev(x64), dev(np.ones(H)), dev(np.zeros(H)), None, 5, 1e-5, True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape,causal", [((3, 5, 40, 40), True), ((2, 17, 300), False), ((2, 64, 2048), True)])
def test_attention_softmax_dropkey(dtype, shape, causal):
    """DropKey (softmax.cuh:157-185): the keys whose draw falls below `dropout` get weight zero, the
    others the softmax over the survivors; the mask is the one the seed names."""
    rng = np.random.default_rng(27)
    x, x64 = rounded(rng.normal(size=shape) * 2, dtype)
    p, seed = 0.3, 0x1234_5678_9ABC_DEF1
    y = M.ops.attention_softmax_fwd(x, p, causal, seed=seed)
    drop = O.dropkey_draws(seed, shape) < p
    yo = O.attention_softmax(x64, causal, drop)
    assert np.abs(host(y) - yo).max() < (1e-5 if dtype == torch.float32 else 4e-3)
    assert np.all(host(y)[drop] == 0)
    assert torch.equal(y, M.ops.attention_softmax_fwd(x, p, causal, seed=seed))
    y2 = M.ops.attention_softmax_fwd(x, p, causal, seed=seed + 1)
    assert not torch.equal(y, y2)
    # the mask has the asked-for rate and does not repeat from row to row
    assert abs(drop.mean() - p) < 5 * np.sqrt(p * (1 - p) / drop.size) + 1e-3
    d2 = drop.reshape(-1, shape[-1])
    assert abs((d2[:-1] & d2[1:]).mean() - p * p) < 0.01
    # eval mode and dropout = 0 ignore it
    mod = M.AttentionSoftmax(dropout=p, use_causal_mask=causal)
    assert torch.equal(mod.eval()(x), M.ops.attention_softmax_fwd(x, 0.0, causal))
    torch.manual_seed(5)
    a = mod.train()(x)
    torch.manual_seed(5)
    assert torch.equal(a, mod(x)) and not torch.equal(a, mod(x))


def test_attention_softmax_dropkey_extremes():
    x = torch.randn(2, 8, 8, device=DEV)
    assert torch.all(M.ops.attention_softmax_fwd(x, 1.0, False, seed=3) == 0)      # every key dropped: zero rows
    with pytest.raises(RuntimeError):
        M.ops.attention_softmax_fwd(x, 1.5, False)
    with pytest.raises(RuntimeError):
        M.ops.attention_fwd(x[..., None], x[..., None], x[..., None], 1.0, -0.1, True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,Nh,H1,H2", [(2, 50, 1, 16, 24), (1, 130, 4, 32, 64), (2, 300, 2, 64, 256)])
@pytest.mark.parametrize("causal", [True, False])
def test_attention_dropkey(dtype, B, L, Nh, H1, H2, causal):
    """The fused op (row kernel for fp32, matrix-core path for bf16) drops the same keys as the softmax
    op does on the [B,Nh,L,L] scores."""
    rng = np.random.default_rng(28)
    q, q64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    k, k64 = rounded(rng.normal(size=(B, L, Nh, H1)) * 0.5, dtype)
    v, v64 = rounded(rng.normal(size=(B, L, Nh, H2)), dtype)
    p, seed = 0.2, 987654321
    drop = O.dropkey_draws(seed, (B, Nh, L, L)) < p
    y, w = M.ops.attention_fwd(q, k, v, 0.8, p, causal, need_weights=True, seed=seed)
    yo, wo = O.attention(q64, k64, v64, 0.8, causal, drop)
    assert rel_err(host(y), yo, eps=2.0) < TOL[dtype]
    assert np.abs(host(w) - wo).max() < (1e-5 if dtype == torch.float32 else 4e-3)
    assert np.all(host(w)[drop] == 0)
    y1, _ = M.ops.attention_fwd(q, k, v, 0.8, p, causal, seed=seed)
    assert rel_err(host(y1), host(y), eps=2.0) < 2 * TOL[dtype]
    # no dropout afterwards: the workspace keeps nothing of the mask
    y0, _ = M.ops.attention_fwd(q, k, v, 0.8, 0.0, causal)
    assert rel_err(host(y0), O.attention(q64, k64, v64, 0.8, causal)[0], eps=2.0) < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("L", [700, 1024, 33])
def test_spectral_convolution_operators(dtype, L):
    """rfft / fftconv_fwd / fftconv_bwd under the reference's names and call forms
    (fused_ops/fftconv.py:14-41): spectra are unnormalised transforms of length 2 * pow2ceil(L)."""
    rng = np.random.default_rng(29)
    B, D = 2, 6
    n = 2 * O.pow2ceil(L)
    x, x64 = rounded(rng.normal(size=(B, D, L)), dtype)
    k = (rng.normal(size=(D, L)) * 0.2).astype(np.float32)
    dy, dy64 = rounded(rng.normal(size=(B, D, L)), dtype)
    k_f = M.ops.rfft(dev(k), False)
    assert k_f.shape == (D, n // 2 + 1) and k_f.dtype == torch.complex64
    ref = np.fft.rfft(k.astype(np.float64), n=n)
    assert rel_err(host(k_f).real, ref.real) < 1e-5 and rel_err(host(k_f).imag, ref.imag) < 1e-5
    refl = np.fft.rfft(x64[..., ::-1], n=n)
    got = host(M.ops.rfft(x, True))
    assert rel_err(got.real, refl.real) < 1e-5 and rel_err(got.imag, refl.imag) < 1e-5
    y, x_f = M.ops.fftconv_fwd(x, k_f)
    assert y.dtype == dtype and x_f.shape == (B, D, n // 2 + 1)
    assert rel_err(host(y), O.causal_conv(x64, k.astype(np.float64))) < TOL[dtype]
    assert rel_err(host(x_f).real, np.fft.rfft(x64, n=n).real) < 1e-5
    x_grad, k_grad = M.ops.fftconv_bwd(dy, x_f, k_f, torch.float32)
    assert x_grad.dtype == dtype and k_grad.shape == (D, L) and k_grad.dtype == torch.float32
    # x_grad[t] = sum_l k[l] dy[t+l]: the causal convolution of the reversed gradient, reversed
    ref_xg = O.causal_conv(dy64[..., ::-1], k.astype(np.float64))[..., ::-1]
    assert rel_err(host(x_grad), ref_xg) < TOL[dtype]
    # k_grad[l] = sum_{b,t} dy[t] x[t-l]
    ref_kg = np.stack([sum(np.correlate(dy64[b, d], x64[b, d], "full")[L - 1:] for b in range(B)) for d in range(D)])
    assert rel_err(host(k_grad), ref_kg) < 2e-4
    xt, kt = M.ops.fftconv_bwd(dy, x, dev(k))
    assert rel_err(host(xt), host(x_grad)) < TOL[dtype] and rel_err(host(kt), host(k_grad)) < 1e-4
    with pytest.raises(RuntimeError):
        M.ops.fftconv_fwd(x, k_f[:, :-1])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,R,C", [(2, 64, 64), (3, 100, 37), (1, 1, 300), (2, 257, 1), (1, 4096, 1024), (0, 5, 5)])
def test_transpose_2d(dtype, B, R, C):
    """The tiled transposition the host uses between time-major memory and rows in time: elements are moved as they
    are, whole and partial tiles of 64 x 64."""
    x = torch.randn(B, R, C, device=DEV).to(dtype)
    y = M.ops.transpose_2d(x)
    assert y.shape == (B, C, R) and y.is_contiguous()
    assert torch.equal(y, x.transpose(1, 2).contiguous())
    assert torch.equal(M.ops.transpose_2d(x, reverse_rows=True), x.flip(1).transpose(1, 2).contiguous())
    assert torch.equal(M.ops.transpose_2d(x, reverse_cols=True), x.flip(2).transpose(1, 2).contiguous())


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("bidirectional", [False, True])
@pytest.mark.parametrize("B,D,L,masked", [(2, 96, 1500, True), (1, 40, 4096, False), (3, 16, 64, False)])
def test_time_major_rows_route(dtype, bidirectional, B, D, L, masked):
    """fp32 / fp16 activations that lie time-major in memory run on the rows kernels between two transpositions: the
    same result as from rows in time, in both output layouts, and the oracle's."""
    print(f"case {dtype} bidirectional={bidirectional} B={B} D={D} L={L} masked={masked}", flush=True)
    rng = np.random.default_rng(71)
    N = 16
    K = 2 * D if bidirectional else D
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    om = rng.normal(size=D)
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(om), bidirectional=bidirectional)
    xt, x64 = rounded(rng.normal(size=(B, L, D)), dtype)          # [B, L, D] memory
    mask = None
    if masked:
        mask = np.zeros((B, L), bool)
        for b in range(B):
            mask[b, L - 17 * (b + 1):] = True
    tm = None if mask is None else dev(mask, torch.bool)
    y_rows, _ = layer(xt.transpose(1, 2), tm)
    y_in, _ = layer(xt.transpose(1, 2), tm, out_layout="input")
    y_ref, _ = layer(xt.transpose(1, 2).contiguous(), tm)
    torch.cuda.synchronize()
    assert y_rows.is_contiguous() and y_in.stride() == (L * D, 1, D)
    assert torch.equal(y_rows, y_ref) and torch.equal(y_in, y_ref)
    yo, _ = O.ema_forward(x64.transpose(0, 2, 1), p, q, g, om, padding_mask=mask, bidirectional=bidirectional)
    assert rel_err(host(y_rows), yo) < TOL[dtype]
    # the input gradient through the same route (time reversed inside the transpositions) against the rows form
    gt = torch.randn(B, L, D, device=DEV).to(dtype)
    dx = layer.adjoint(gt.transpose(1, 2), tm)
    dx_ref = layer.adjoint(gt.transpose(1, 2).contiguous(), tm)
    assert dx.stride() == (L * D, 1, D)
    assert rel_err(host(dx), host(dx_ref)) < 1e-5
