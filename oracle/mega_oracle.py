"""CPU oracle for the Mega/Mega2 sequence-mixing path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may
import this module.  It is never on the product path: the product is the HIP
library under fairseq-apollo_amd/csrc and fails loudly without it.

Every function restates, in numpy (fp64 unless told otherwise), what the
reference computes; the reference location it follows is cited per function
(paths relative to the reference tree).  The reference ships no tests, golden
vectors or fixtures for this path, so each function is pinned by
tests/test_oracle_*.py against closed forms, brute force and library routines
(and against oracle/_ref, the reference's own CPU translation units compiled in
place, where that build exists).  Pin status per function:

  ema_coeffs_real / ema_coeffs_complex   closed forms + invariants
  ema_kernel / ema_bias / ema_hidden     brute-force powers, geometric series, oracle/_ref
  causal_conv / bidirectional_conv       direct O(L^2) sums, numpy.convolve, impulse/shift
  ema_forward / ema_one_step             chunk-split invariance, step-vs-parallel equality
  timestep_norm (group / per feature)    numpy.mean/var on prefixes, oracle/_ref
  attention_softmax / attention          explicit masked softmax, rows sum to 1
  rotary / simple_relative_bias          the reference modules' own outputs
                                         (tests/golden/position_vectors.npz, written from
                                         fairseq/modules/relative_positional_bias.py)
  swiglu / rms_norm                      silu identities and known values, rms of constant
                                         vectors, scale invariance, torch's F.silu / F.rms_norm
  swiglu_ffn / silu_ffn                  per-row loops, identity and one-hot weights
  gated_attention_layer                  MovingAverageGatedAttention.forward restated with the
                                         library calls the reference makes (torch.split,
                                         F.normalize, F.softmax, ...) over the pinned primitives,
                                         all branches (rms / relu2 / laplace / simple bias /
                                         two-sided / padding), and closed-form special cases
                                         (gamma = -1: running means of v; W_h = 0; z under the
                                         normalize clamp; one-hot mx_proj rows)
                                         (tests/test_oracle_layer.py)
  normalized_ffn                         torch's F.layer_norm / F.linear / F.silu with the stored
                                         weight plus one, identity for a zero second projection
  mega_lm_decoder                        no layers: textbook prefix statistics + library
                                         projections; two layers: hand composition of the pinned
                                         pieces, order asymmetry, causality in the tokens, the
                                         chunk padding cut back, zero logits at padding tokens
The SwiGLU feed-forward block and the multi-head split of the gated attention are north-star
specification, not reference code (the reference FFN is the SiLU block, its layer single-head):
their formulas are pinned as above, their parity with the reference is unpinned by construction.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np

# --------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def _silu(x):
    return x * _sigmoid(x)


def pow2ceil(L: int) -> int:
    """fused_ops/fftconv.py:47 -- N = L if L is a power of two else 1 << bit_length."""
    return L if (L & (L - 1)) == 0 else (1 << int(L).bit_length())


# --------------------------------------------------------------------------
# A1/A2: coefficients
# --------------------------------------------------------------------------


def ema_coeffs_real(alpha, delta, beta, gamma, dtype=np.float64):
    """Real EMA coefficients, modules/exponential_moving_average.py:71-80.

    alpha, delta, beta: [K, N, 1] (or [K, N]); gamma: [K, N].
    Returns p[K,N], q[K,N], gamma'[K,N] with q = 1 - s(alpha) s(delta),
    p = s(alpha) beta, gamma' = gamma sqrt(1/N).
    """
    alpha = np.asarray(alpha, dtype).reshape(gamma.shape[0], -1)
    delta = np.asarray(delta, dtype).reshape(gamma.shape[0], -1)
    beta = np.asarray(beta, dtype).reshape(gamma.shape[0], -1)
    gamma = np.asarray(gamma, dtype)
    N = gamma.shape[1]
    a = _sigmoid(alpha)
    d = _sigmoid(delta)
    q = 1.0 - a * d
    p = a * beta
    return p, q, gamma * math.sqrt(1.0 / N)


def ema_coeffs_complex(alpha, delta, theta, gamma, dtype=np.float64):
    """Complex EMA coefficients, modules/complex_exponential_moving_average.py:79-96.

    alpha, delta: [K, N, 1]; theta: [K, 1, 1]; gamma: [K, N, 2] (re, im).
    theta_{d,n} = (n+1) s(theta_d) 2pi/N; p = s(alpha);
    q = (1 - s(alpha) s(delta)) e^{i theta}; gamma' = (g0 + i g1) sqrt(1/N).
    """
    gamma = np.asarray(gamma, dtype)
    K, N = gamma.shape[0], gamma.shape[1]
    alpha = np.asarray(alpha, dtype).reshape(K, N)
    delta = np.asarray(delta, dtype).reshape(K, N)
    theta = np.asarray(theta, dtype).reshape(K, 1)
    ctype = np.complex128 if dtype == np.float64 else np.complex64
    phi = _sigmoid(theta) * (2.0 * math.pi / N)
    wav = np.arange(1, N + 1, dtype=dtype).reshape(1, N)
    ang = wav * phi
    a = _sigmoid(alpha)
    d = _sigmoid(delta)
    mag = 1.0 - a * d
    q = (mag * np.cos(ang) + 1j * mag * np.sin(ang)).astype(ctype)
    g = (gamma[..., 0] + 1j * gamma[..., 1]).astype(ctype) * math.sqrt(1.0 / N)
    return a, q, g


# --------------------------------------------------------------------------
# A3: kernel / bias; A7: hidden state
# --------------------------------------------------------------------------


def ema_kernel(p, q, gamma, L: int):
    """w[d,l] = Re sum_n p gamma exp(l log q), csrc/ops/ema_parameters.cc:37-52
    (same as complex_exponential_moving_average.py:104-109 and
    exponential_moving_average.py:82-90 for real q)."""
    q = np.asarray(q)
    logq = np.log(q.astype(np.complex128 if np.iscomplexobj(q) else q.dtype))
    l = np.arange(L).reshape(1, 1, L)
    vander = np.exp(l * logq[..., None])            # K x N x L
    c = np.asarray(p)[..., None] * np.asarray(gamma)[..., None]
    return np.real((c * vander).sum(axis=1))


def ema_bias(q, gamma, h, L: int):
    """b[b,d,l] = Re sum_n exp((l+1) log q) gamma h, csrc/ops/ema_parameters.cc:54-77
    (equals base_moving_average.py:73-80).  h: [B, K, N]."""
    q = np.asarray(q)
    logq = np.log(q.astype(np.complex128 if np.iscomplexobj(q) else q.dtype))
    l = np.arange(1, L + 1).reshape(1, 1, L)
    vander = np.exp(l * logq[..., None]) * np.asarray(gamma)[..., None]   # K x N x L
    return np.real(np.einsum('bdn,dnl->bdl', np.asarray(h), vander))


def ema_hidden(x, p, q, h=None):
    """h'[b,d,n] = p sum_j q^{L-1-j} x[b,d,j] + q^L h, csrc/ops/ema_hidden.cc:31-63.
    x: [B, D, L] real.  Returns [B, D, N] (complex if q is)."""
    x = np.asarray(x, np.float64)
    q = np.asarray(q)
    L = x.shape[-1]
    logq = np.log(q.astype(np.complex128 if np.iscomplexobj(q) else q.dtype))
    e = np.arange(L - 1, -1, -1).reshape(1, 1, L)
    vander = np.exp(e * logq[..., None])            # D x N x L
    out = np.einsum('bdl,dnl->bdn', x, vander) * np.asarray(p)[None]
    if h is not None:
        out = out + np.exp(L * logq)[None] * np.asarray(h)
    return out


# --------------------------------------------------------------------------
# A4/A5: long convolution
# --------------------------------------------------------------------------


def causal_conv(x, k):
    """y[...,t] = sum_{j<=t, j<Lk} k[d,j] x[...,t-j] through the zero-padded real FFT of
    length 2*pow2ceil(L), exactly the order of operations of
    fused_ops/fftconv.py:45-61 (_fftconv_fwd).  x: [B, D, L]; k: [D, Lk], Lk <= L."""
    x = np.asarray(x, np.float64)
    k = np.asarray(k, np.float64)
    L = x.shape[-1]
    n2 = 2 * pow2ceil(L)
    x_f = np.fft.rfft(x, n=n2)
    k_f = np.fft.rfft(k, n=n2) / n2                 # norm="forward" on the kernel
    y = np.fft.irfft(x_f * k_f, n=n2) * n2          # norm="forward" on the inverse
    return y[..., :L]


def causal_conv_direct(x, k):
    """The same convolution as an explicit double loop (small inputs only)."""
    x = np.asarray(x, np.float64)
    k = np.asarray(k, np.float64)
    B, D, L = x.shape
    Lk = k.shape[-1]
    y = np.zeros_like(x)
    for t in range(L):
        for j in range(min(t + 1, Lk)):
            y[:, :, t] += k[None, :, j] * x[:, :, t - j]
    return y


def bidirectional_conv(x, k, shift: bool = True):
    """fused_ops/fftconv.py:85-100 (bidirectional_fftconv): k = [k1; k2] of shape
    [2D, Lk]; circular real FFT of length L + Lk."""
    x = np.asarray(x, np.float64)
    k = np.asarray(k, np.float64)
    B, D, L = x.shape
    Lk = k.shape[1]
    F = L + Lk
    k1, k2 = k[:D], k[D:]
    kk = np.zeros((D, F))
    kk[:, :Lk] += k1
    if shift:
        kk[:, L:] += k2[:, ::-1]
    else:
        kk[:, 0] += k2[:, 0]
        kk[:, L + 1:] += k2[:, 1:][:, ::-1]
    k_f = np.fft.rfft(kk, n=F) / F
    x_f = np.fft.rfft(x, n=F)
    return (np.fft.irfft(x_f * k_f, n=F) * F)[..., :L]


def bidirectional_conv_direct(x, k, shift: bool = True):
    """The two explicit lag sums: forward lags j >= 0 with k1; backward lags m >= 1 with
    k2[m-1] (shift) or k2[m] plus the lag-0 tap k2[0] (no shift)."""
    x = np.asarray(x, np.float64)
    k = np.asarray(k, np.float64)
    B, D, L = x.shape
    Lk = k.shape[1]
    k1, k2 = k[:D], k[D:]
    y = np.zeros_like(x)
    for t in range(L):
        for j in range(min(t + 1, Lk)):
            y[:, :, t] += k1[None, :, j] * x[:, :, t - j]
        if shift:
            for m in range(1, Lk + 1):
                if t + m < L:
                    y[:, :, t] += k2[None, :, m - 1] * x[:, :, t + m]
        else:
            y[:, :, t] += k2[None, :, 0] * x[:, :, t]
            for m in range(1, Lk):
                if t + m < L:
                    y[:, :, t] += k2[None, :, m] * x[:, :, t + m]
    return y


# --------------------------------------------------------------------------
# A6: the moving-average layer
# --------------------------------------------------------------------------


def ema_forward(x, p, q, gamma, omega, padding_mask=None, h=None,
                bidirectional: bool = False, truncation: Optional[int] = None,
                shift: bool = True, incremental: bool = False):
    """BaseMovingLayer.forward, modules/base_moving_average.py:120-172.

    x: [B, D, L]; p, q, gamma: [K, N] with K = 2D when bidirectional; omega: [D];
    padding_mask: [B, L] (True = pad); h: [B, D, N] carried state or None.
    Returns (y[B,D,L], h' or None).  The carried-state bias is always added (the GPU
    behaviour of the reference; its CPU branch drops it, see
    complex_exponential_moving_average.py:98-109).
    """
    x = np.asarray(x, np.float64)
    B, D, L = x.shape
    residual = x * np.asarray(omega, np.float64).reshape(1, D, 1)
    xm = x
    if padding_mask is not None:
        xm = x * (1.0 - np.asarray(padding_mask, np.float64)[:, None, :])
    Lk = L if truncation is None or truncation < 1 else min(truncation, L)
    k = ema_kernel(p, q, gamma, Lk)
    h_new = None
    if bidirectional:
        assert h is None and not incremental
        out = bidirectional_conv(xm, k, shift)
    else:
        out = causal_conv(xm, k)
        if incremental or h is not None:
            if h is not None:
                out = out + ema_bias(q, gamma, h, L)
            h_new = ema_hidden(xm, p, q, h)
    return out + residual, h_new


def ema_kernel_bwd(dk, p, q, gamma):
    """RowwiseEMAWeightCPUBwd, csrc/ops/ema_parameters.cc:80-97: from the kernel gradient
    dk [D, L] to (dp [D,N] real, dq [D,N], dgamma [D,N]) with
    sum1 = sum_l dk[l] l q^(l-1), sum2 = sum_l dk[l] q^l; dp = Re(sum2 gamma),
    dq = conj(sum1 p gamma), dgamma = conj(sum2 p)."""
    dk = np.asarray(dk, np.float64)
    p = np.asarray(p, np.float64)
    q = np.asarray(q, np.complex128)
    gamma = np.asarray(gamma, np.complex128)
    L = dk.shape[-1]
    l = np.arange(L)
    qw2 = q[..., None] ** l                                             # q^l
    qw1 = np.where(l > 0, q[..., None] ** np.maximum(l - 1, 0), 0.0)    # q^(l-1), 0 at l = 0
    sum1 = (dk[:, None, :] * qw1 * l).sum(-1)
    sum2 = (dk[:, None, :] * qw2).sum(-1)
    return (sum2 * gamma).real, np.conj(sum1 * p * gamma), np.conj(sum2 * p)


def ema_hidden_bwd(dy, x, p, q, h=None):
    """EMAHiddenCPUBwdImpl, csrc/ops/ema_hidden.cc:66-159, for h' = q^L h + sum_j p q^(L-1-j) x[j]
    (dy: gradient of h', complex [B, D, N]):
    dx[j] = Re sum_n conj(dy) p q^(L-1-j); dp = Re sum_{b,j} conj(dy) x[j] q^(L-1-j);
    dq = conj(sum_{b,j} conj(dy) x[j] p (L-1-j) q^(L-2-j) + sum_b conj(dy) h L q^(L-1)); dh = conj(conj(dy) q^L).
    Returns (dx, dp, dq, dh or None)."""
    x = np.asarray(x, np.float64)
    p = np.asarray(p, np.float64)
    q = np.asarray(q, np.complex128)
    dyc = np.conj(np.asarray(dy, np.complex128))
    B, D, L = x.shape
    e = L - 1 - np.arange(L)                                         # exponent of q at token j
    qw = q[..., None] ** e                                           # [D, N, L]
    qd = np.where(e > 0, e * q[..., None] ** np.maximum(e - 1, 0), 0.0)
    dx = np.real(np.einsum('bdn,dn,dnl->bdl', dyc, p, qw))
    dp = np.real(np.einsum('bdn,bdl,dnl->dn', dyc, x, qw))
    s2 = np.einsum('bdn,bdl,dn,dnl->dn', dyc, x, p, qd)
    dh = None
    if h is not None:
        h = np.asarray(h, np.complex128)
        s2 = s2 + (dyc * h).sum(0) * L * q ** (L - 1)
        dh = np.conj(dyc * q ** L)
    return dx, dp, np.conj(s2), dh


def ema_bias_bwd(db, q, gamma, h):
    """RowwiseEMABiasCPUBwd, csrc/ops/ema_parameters.cc:99-116: the bias is
    b[b,d,l] = Re sum_n q^(l+1) gamma h; with sum1 = sum_l db[l] (l+1) q^l and sum2 = sum_l db[l] q^(l+1)
    per batch row: dq = sum_rows conj(sum1 gamma h), dgamma = sum_rows conj(sum2 h), dh = conj(sum2 gamma).
    db: [B, D, L]; h: [B, D, N].  Returns (dq [D,N], dgamma [D,N], dh [B,D,N])."""
    db = np.asarray(db, np.float64)
    q = np.asarray(q, np.complex128)
    gamma = np.asarray(gamma, np.complex128)
    h = np.asarray(h, np.complex128)
    L = db.shape[-1]
    l = np.arange(L)
    qw1 = q[..., None] ** l                     # q^l
    qw2 = qw1 * q[..., None]                    # q^(l+1)
    sum1 = (db[:, :, None, :] * qw1[None] * (l + 1)).sum(-1)
    sum2 = (db[:, :, None, :] * qw2[None]).sum(-1)
    return np.conj(sum1 * gamma * h).sum(0), np.conj(sum2 * h).sum(0), np.conj(sum2 * gamma)


def ema_backward(dy, x, p, q, gamma, omega, padding_mask=None, bidirectional: bool = False, shift: bool = True):
    """Backward of ema_forward (no carried state): the reference's chain fftconv backward
    (modules/fused_ops/fftconv.py:66-88, 85-100: dx = correlation of dy with k, dk = sum over the
    batch of the correlation of dy with x) -> ema_kernel_bwd, with the correlations written out
    directly.  Two-sided layers: y[t] = sum_{j>=0} k1[j] x[t-j] + sum_{m>=1} k2[m-1] x[t+m] (shift) or
    sum_{m>=0} k2[m] x[t+m] (no shift), k1 / k2 from the first / second D coefficient rows.
    Returns (dx, dp, dq, dgamma, domega)."""
    dy = np.asarray(dy, np.float64)
    x = np.asarray(x, np.float64)
    B, D, L = x.shape
    keep = np.ones((B, 1, L)) if padding_mask is None else 1.0 - np.asarray(padding_mask, np.float64)[:, None, :]
    xm = x * keep
    k = ema_kernel(p, q, gamma, L)
    dxc = np.zeros_like(x)
    dk = np.zeros((k.shape[0], L))
    for l in range(L):
        # forward lags: y[t] += k1[l] x[t - l]
        dxc[:, :, :L - l] += dy[:, :, l:] * k[None, :D, l:l + 1]
        dk[:D, l] = (dy[:, :, l:] * xm[:, :, :L - l]).sum(axis=(0, 2))
        if bidirectional:
            m = l + 1 if shift else l                       # backward lags: y[t] += k2[l] x[t + m]
            if m < L:
                dxc[:, :, m:] += dy[:, :, :L - m] * k[None, D:, l:l + 1]
                dk[D:, l] = (dy[:, :, :L - m] * xm[:, :, m:]).sum(axis=(0, 2))
    om = np.asarray(omega, np.float64).reshape(1, D, 1)
    dp, dq, dg = ema_kernel_bwd(dk, p, q, gamma)
    return dxc * keep + om * dy, dp, dq, dg, (dy * x).sum(axis=(0, 2))


def ema_one_step(x_t, p, q, gamma, omega, h=None):
    """BaseMovingLayer.one_step, modules/base_moving_average.py:105-118, plus the
    residual the caller adds.  x_t: [B, D]; h: [B, D, N]."""
    x_t = np.asarray(x_t, np.float64)
    hh = np.asarray(p)[None] * x_t[..., None]
    if h is not None:
        hh = hh + np.asarray(q)[None] * np.asarray(h)
    out = np.real(np.einsum('bdn,dn->bd', hh, np.asarray(gamma)))
    return out + x_t * np.asarray(omega, np.float64).reshape(1, -1), hh


# --------------------------------------------------------------------------
# A8: TimestepNorm
# --------------------------------------------------------------------------


def _welford_update(m0, m1, m2, x):
    """csrc/utils.h:55-64."""
    m0 = m0 + 1
    coef = 1.0 / m0
    d1 = x - m1
    m1 = m1 + coef * d1
    d2 = d1 * (x - m1) - m2
    m2 = m2 + coef * d2
    return m0, m1, m2


def _welford_combine(a0, a1, a2, b0, b1, b2):
    """csrc/utils.h:66-76."""
    m0 = a0 + b0
    c1 = 0.0 if m0 == 0 else a0 / m0
    c2 = 0.0 if m0 == 0 else b0 / m0
    delta = b1 - a1
    m1 = c1 * a1 + c2 * b1
    m2 = c1 * a2 + c2 * b2 + (c1 * delta) * (c2 * delta)
    return m0, m1, m2


def timestep_norm(x, prev_count, prev_mean, prev_var, gamma, beta,
                  padding_mask=None, num_groups: Optional[int] = None, eps: float = 1e-5,
                  dtype=np.float64):
    """Group variant: csrc/ops/timestep_norm.cc:218-316; per-feature variant
    (num_groups None): csrc/ops/timestep_norm.cc:23-103.  Literal serial loop.

    x: [B, L, H]; prev_count: [B] int; prev_mean, prev_var: [B, G]; gamma (= weight + 1),
    beta: [H].  Returns (y, count[B] int64, mean[B,G], var[B,G]).
    """
    x = np.asarray(x, dtype)
    B, L, H = x.shape
    gamma = np.asarray(gamma, dtype)
    beta = np.asarray(beta, dtype)
    G = H if num_groups is None else num_groups
    Dg = H // G
    y = np.zeros_like(x)
    count = np.array(prev_count, dtype=np.int64).copy()
    mean = np.array(prev_mean, dtype=dtype).reshape(B, G).copy()
    var = np.array(prev_var, dtype=dtype).reshape(B, G).copy()
    if num_groups is not None:
        xg = x.reshape(B, L, G, Dg)
        gmean = xg.mean(axis=-1)
        gvar = xg.var(axis=-1)                      # biased, as RowwiseMoments (utils.h:79-118)
    for b in range(B):
        m0 = int(count[b])
        u = mean[b].copy()
        v = var[b].copy()
        for t in range(L):
            masked = padding_mask is not None and bool(padding_mask[b][t])
            if num_groups is None:
                _, m1, m2 = _welford_update(m0, u, v, x[b, t])
                rstd = 1.0 / np.sqrt(m2 + dtype(eps))
                if not masked:
                    y[b, t] = (x[b, t] - m1) * rstd * gamma + beta
                    u, v = m1, m2
            else:
                _, m1, m2 = _welford_combine(m0, u, v, 1, gmean[b, t], gvar[b, t])
                rstd = 1.0 / np.sqrt(m2 + dtype(eps))
                if not masked:
                    y[b, t] = ((xg[b, t] - m1[:, None]) * rstd[:, None]).reshape(H) * gamma + beta
                    u, v = m1, m2
            if not masked:
                m0 += 1
        count[b] = m0
        mean[b] = u
        var[b] = v
    return y, count, mean, var


def timestep_norm_closed_form(x, padding_mask=None, num_groups: Optional[int] = None,
                              eps: float = 1e-5, gamma=None, beta=None):
    """Textbook statement for zero prior count: after step t the state is the mean and the
    biased variance of every unmasked element x[b, <=t, group].  Independent of the
    recurrences above (cumulative sums in fp64)."""
    x = np.asarray(x, np.float64)
    B, L, H = x.shape
    G = H if num_groups is None else num_groups
    Dg = H // G
    xg = x.reshape(B, L, G, Dg)
    keep = np.ones((B, L)) if padding_mask is None else 1.0 - np.asarray(padding_mask, np.float64)
    s1 = np.cumsum(xg.sum(-1) * keep[..., None], axis=1)
    s2 = np.cumsum((xg ** 2).sum(-1) * keep[..., None], axis=1)
    n = np.cumsum(keep, axis=1)[..., None] * Dg
    with np.errstate(divide='ignore', invalid='ignore'):
        mu = np.where(n > 0, s1 / n, 0.0)
        var = np.where(n > 0, s2 / n - mu ** 2, 0.0)
    y = (xg - mu[..., None]) / np.sqrt(var[..., None] + eps)
    y = y.reshape(B, L, H)
    if gamma is not None:
        y = y * np.asarray(gamma, np.float64)
    if beta is not None:
        y = y + np.asarray(beta, np.float64)
    y = y * keep[..., None]
    return y, mu, var


def sequence_norm(x, gamma, beta, padding_mask=None, num_groups: Optional[int] = None, eps: float = 1e-5,
                  length_last: bool = False):
    """csrc/ops/sequence_norm.cc:531-656 (groups) and :258-372 (per feature): statistics of one
    (row, group) over all unmasked tokens and the group's channels (biased variance),
    y = (x - mean) rstd gamma + beta, masked tokens 0.  x: [B, L, H], or [B, H, L] with length_last.
    Returns (y, count[B], mean[B,G], rstd[B,G])."""
    x = np.asarray(x, np.float64)
    xl = x.transpose(0, 2, 1) if length_last else x
    B, L, H = xl.shape
    G = H if num_groups is None else num_groups
    D = H // G
    keep = np.ones((B, L), bool) if padding_mask is None else ~np.asarray(padding_mask, bool)
    y = np.zeros_like(xl)
    count = keep.sum(1).astype(np.int64)
    mean = np.zeros((B, G))
    rstd = np.zeros((B, G))
    gw = np.asarray(gamma, np.float64)
    bw = np.asarray(beta, np.float64)
    for b in range(B):
        xg = xl[b][keep[b]].reshape(-1, G, D)
        for g in range(G):
            v = xg[:, g, :]
            mean[b, g] = v.mean() if v.size else 0.0
            rstd[b, g] = 1.0 / np.sqrt((v.var() if v.size else 0.0) + eps)
        yb = (xl[b].reshape(L, G, D) - mean[b][None, :, None]) * rstd[b][None, :, None]
        y[b] = yb.reshape(L, H) * gw + bw
        y[b][~keep[b]] = 0.0
    return (y.transpose(0, 2, 1) if length_last else y), count, mean, rstd


def sequence_norm_bwd(dy, x, gamma, padding_mask=None, num_groups: Optional[int] = None, eps: float = 1e-5,
                      length_last: bool = False):
    """csrc/ops/sequence_norm.cc:657-754 (and the time-last twin :756-842): per (row, channel)
    ds = sum dy x, db = sum dy over unmasked tokens; per group dsw = sum ds gamma, dbw = sum db gamma;
    dv = r^3 (u dbw - dsw) / 2, du = -r dbw; dx = r gamma dy + (2 (x - u) dv + du) / (count D);
    dgamma = sum_rows r (ds - u db), dbeta = sum_rows db.  Returns (dx, dgamma, dbeta)."""
    dy = np.asarray(dy, np.float64)
    x = np.asarray(x, np.float64)
    if length_last:
        dy, x = dy.transpose(0, 2, 1), x.transpose(0, 2, 1)
    B, L, H = x.shape
    G = H if num_groups is None else num_groups
    D = H // G
    _, count, mean, rstd = sequence_norm(x, gamma, np.zeros(H), padding_mask, num_groups, eps, False)
    keep = np.ones((B, L)) if padding_mask is None else 1.0 - np.asarray(padding_mask, np.float64)
    w = np.asarray(gamma, np.float64)
    dym = dy * keep[..., None]
    ds = (dym * x).sum(1)                                  # [B, H]
    db = dym.sum(1)
    dsw = (ds * w).reshape(B, G, D).sum(-1)
    dbw = (db * w).reshape(B, G, D).sum(-1)
    dv = 0.5 * rstd ** 3 * (mean * dbw - dsw)
    du = -rstd * dbw
    n = np.maximum(count[:, None] * D, 1)
    ue, re_ = np.repeat(mean, D, 1), np.repeat(rstd, D, 1)
    dx = re_[:, None, :] * w * dy + (2 * (x - ue[:, None, :]) * np.repeat(dv / n, D, 1)[:, None, :]
                                     + np.repeat(du / n, D, 1)[:, None, :])
    dx = dx * keep[..., None]
    dg = (re_ * (ds - ue * db)).sum(0)
    return (dx.transpose(0, 2, 1) if length_last else dx), dg, db.sum(0)


def timestep_norm_saved(x, prev_count, prev_mean, prev_var, padding_mask=None, num_groups: Optional[int] = None,
                        eps: float = 1e-5):
    """What the forward keeps for the backward pass (csrc/ops/timestep_norm.cc:283-300):
    (count[B], group_mean, cummean, cumrstd), the last three [B, L, G].  At a masked token
    cummean / cumrstd hold the carried (unchanged) state, which is what "the cumulative mean before
    the next token" must be for the backward recurrences to be the derivative of the forward."""
    x = np.asarray(x, np.float64)
    B, L, H = x.shape
    G = H if num_groups is None else num_groups
    xg = x.reshape(B, L, G, H // G)
    gmean, gvar = xg.mean(-1), xg.var(-1)
    cm = np.zeros((B, L, G))
    cr = np.zeros((B, L, G))
    count = np.array(prev_count, np.int64).copy()
    for b in range(B):
        m0 = int(count[b])
        u = np.array(prev_mean, np.float64).reshape(B, G)[b].copy()
        v = np.array(prev_var, np.float64).reshape(B, G)[b].copy()
        for t in range(L):
            if padding_mask is not None and bool(padding_mask[b][t]):
                cm[b, t], cr[b, t] = u, 1.0 / np.sqrt(v + eps)
                continue
            _, u, v = _welford_combine(m0, u, v, 1, gmean[b, t], gvar[b, t])
            m0 += 1
            cm[b, t], cr[b, t] = u, 1.0 / np.sqrt(v + eps)
        count[b] = m0
    return count, gmean, cm, cr


def timestep_norm_bwd(dy, dmean, dvar, x, prev_mean, count, group_mean, cummean, cumrstd, gamma,
                      padding_mask=None, num_groups: Optional[int] = None):
    """Group variant: csrc/ops/timestep_norm.cc:318-450, the literal reverse-time loop; the
    per-feature variant (:104-217) is the same recurrence with one channel per group and
    group_mean = x.  Returns (dx, dprev_mean, dprev_var, dgamma, dbeta)."""
    dy = np.asarray(dy, np.float64)
    x = np.asarray(x, np.float64)
    B, L, H = x.shape
    G = H if num_groups is None else num_groups
    D = H // G
    w = np.asarray(gamma, np.float64).reshape(G, D)
    dyg, xg = dy.reshape(B, L, G, D), x.reshape(B, L, G, D)
    gm = xg.mean(-1) if group_mean is None else np.asarray(group_mean, np.float64)
    dx = np.zeros((B, L, G, D))
    dw = np.zeros((G, D))
    dbeta = np.zeros((G, D))
    ug = np.zeros((B, G)) if dmean is None else np.array(dmean, np.float64).reshape(B, G).copy()
    vg = np.zeros((B, G)) if dvar is None else np.array(dvar, np.float64).reshape(B, G).copy()
    pm = np.asarray(prev_mean, np.float64).reshape(B, G)
    for b in range(B):
        m0 = int(count[b])
        for j in range(L - 1, -1, -1):
            if padding_mask is not None and bool(padding_mask[b][j]):
                continue
            c1, c2 = (m0 - 1) / m0, 1.0 / m0
            m0 -= 1
            prev_u = pm[b] if j == 0 else cummean[b, j - 1]
            u, r, ux = cummean[b, j], cumrstd[b, j], gm[b, j]
            ds = (dyg[b, j] * (xg[b, j] - u[:, None]) * w).sum(-1)
            db = (dyg[b, j] * w).sum(-1)
            du = ug[b] - r * db
            dv = vg[b] - 0.5 * r ** 3 * ds
            dux = c2 * du + 2 * c1 * c2 * dv * (ux - prev_u)
            dvx = c2 * dv
            dx[b, j] = dyg[b, j] * r[:, None] * w + (dux[:, None] + 2 * dvx[:, None] * (xg[b, j] - ux[:, None])) / D
            dw += dyg[b, j] * (xg[b, j] - u[:, None]) * r[:, None]
            dbeta += dyg[b, j]
            ug[b] = c1 * du - 2 * c1 * c2 * dv * (ux - prev_u)
            vg[b] = c1 * dv
    return dx.reshape(B, L, H), ug, vg, dw.reshape(H), dbeta.reshape(H)


# --------------------------------------------------------------------------
# A9/A10: attention softmax and the fused attention op
# --------------------------------------------------------------------------


def dropkey_draws(seed: int, shape):
    """The uniform draws in [0, 1) the HIP kernels use for DropKey: draw e (the element's place in
    the flattened score tensor) is the splitmix64 finaliser of seed + (e + 1) * golden ratio, top
    24 bits.  The reference draws from Philox (csrc/softmax.cuh:157-185); which generator names the
    mask is not part of the op's contract, only `draw < dropout -> -inf` is.  Restated here so a
    test can hand the same mask to the fp64 softmax below."""
    n = int(np.prod(shape))
    with np.errstate(over='ignore'):
        z = np.uint64(seed & (2 ** 64 - 1)) + (np.arange(n, dtype=np.uint64) + np.uint64(1)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        z = z ^ (z >> np.uint64(31))
    return ((z >> np.uint64(40)).astype(np.float64) / 16777216.0).reshape(shape)


def attention_softmax(x, causal: bool = False, drop=None):
    """csrc/softmax.cuh:90-185: softmax over the last axis of x[..., R, C]; causal keeps
    columns [0, C - R + r] of row r; `drop` (boolean, x's shape) marks the keys DropKey replaces
    by -inf first; a row whose maximum is -inf (or whose sum is 0) becomes zeros."""
    x = np.asarray(x, np.float64)
    R, C = x.shape[-2], x.shape[-1]
    if drop is not None:
        x = np.where(np.asarray(drop, bool), -np.inf, x)
    if causal:
        r = np.arange(R)[:, None]
        c = np.arange(C)[None, :]
        x = np.where(c <= C - R + r, x, -np.inf)
    m = x.max(axis=-1, keepdims=True)
    dead = ~np.isfinite(m)
    e = np.exp(x - np.where(dead, 0.0, m))
    e = np.where(dead, 0.0, e)
    s = e.sum(axis=-1, keepdims=True)
    return np.where(s > 0, e / np.where(s > 0, s, 1.0), 0.0)


def attention(q, k, v, scale: float = 1.0, causal: bool = True, drop=None):
    """csrc/ops/attention_kernel.cu:40-131: q, k: [B, L, Nh, H1]; v: [B, L, Nh, H2];
    w[b,n] = softmax_causal(scale q k^T) with the keys marked in drop[B, Nh, L, L] removed;
    y[b,:,n,:] = w v.  Returns (y, w)."""
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    s = np.einsum('blnh,bmnh->bnlm', q, k) * scale
    w = attention_softmax(s, causal, drop)
    y = np.einsum('bnlm,bmnh->blnh', w, v)
    return y, w


def attention_softmax_bwd(dy, y):
    """csrc/softmax.cuh AttentionSoftmaxBwdKernel: dx = y (dy - sum(y dy, -1)); masked columns hold
    y = 0 and get dx = 0."""
    dy = np.asarray(dy, np.float64)
    y = np.asarray(y, np.float64)
    return y * (dy - (y * dy).sum(-1, keepdims=True))


def attention_bwd(dy, q, k, v, scale: float = 1.0, causal: bool = True, drop=None):
    """csrc/ops/attention_kernel.cu:133-255: dv = w^T dy, dw = dy v^T, ds = softmax_bwd(dw, w),
    dk = scale ds^T q, dq = scale ds k per (batch, head).  Returns (dq, dk, dv)."""
    dy = np.asarray(dy, np.float64)
    q = np.asarray(q, np.float64)
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    _, w = attention(q, k, v, scale, causal, drop)
    dv = np.einsum('bnlm,blnh->bmnh', w, dy)
    dw = np.einsum('blnh,bmnh->bnlm', dy, v)
    ds = attention_softmax_bwd(dw, w)
    dk = scale * np.einsum('bnlm,blnh->bmnh', ds, q)
    dq = scale * np.einsum('bnlm,bmnh->blnh', ds, k)
    return dq, dk, dv


# --------------------------------------------------------------------------
# A11/A12: layer glue (spec-level restatement)
# --------------------------------------------------------------------------


def swiglu(a, b):
    """silu(a) * b -- the gate of the north-star SwiGLU FFN; not present in the
    reference (its FFN is normalized_feedforward_network.py:77-93): specification only."""
    a = np.asarray(a, np.float64)
    return _silu(a) * np.asarray(b, np.float64)


def swiglu_ffn(x, w1, w3, w2):
    """W2 (silu(W1 x) * W3 x); weights are [out, in]."""
    x = np.asarray(x, np.float64)
    return swiglu(x @ np.asarray(w1, np.float64).T, x @ np.asarray(w3, np.float64).T) @ np.asarray(w2, np.float64).T


def silu_ffn(x, w1, b1, w2, b2):
    """normalized_feedforward_network.py:77-93 without the norm: x + fc2(silu(fc1(x)))."""
    x = np.asarray(x, np.float64)
    return x + _silu(x @ np.asarray(w1, np.float64).T + b1) @ np.asarray(w2, np.float64).T + b2


def rotary(x, base: float = 10000.0, start: int = 0):
    """modules/relative_positional_bias.py:46-94 (RotaryEmbedding):
    x: [..., L, S]; features (2i, 2i+1) form one complex number that is multiplied by
    exp(i t base^{-2i/S}) for position t = start, start + 1, ... (`start`: the reference's `qidx`, the place of
    a single query behind cached keys, :89-92).  Pinned by the reference module's own outputs
    (tests/golden/position_vectors.npz)."""
    x = np.asarray(x, np.float64)
    L, S = x.shape[-2], x.shape[-1]
    freq = 1.0 / (base ** (np.arange(0, S, 2) / S))
    ang = (start + np.arange(L))[:, None] * freq[None, :]
    z = (x[..., 0::2] + 1j * x[..., 1::2]) * np.exp(1j * ang)
    out = np.empty_like(x)
    out[..., 0::2] = z.real
    out[..., 1::2] = z.imag
    return out


def simple_relative_bias(param, C: int):
    """modules/relative_positional_bias.py:13-42 (SimpleRelativePositionalBias.forward): the [C, C] matrix added to
    q k^T, entry (i, j) = param[max_positions - 1 + j - i] for the 2 max_positions - 1 learned offsets.  Pinned by
    the reference module's own outputs (tests/golden/position_vectors.npz)."""
    sb = np.asarray(param, np.float64)
    mp = (sb.shape[0] + 1) // 2
    if C > mp:
        raise ValueError(f"sequence length {C} beyond max length {mp}")
    pos = np.arange(C)
    return sb[(mp - 1) + pos[None, :] - pos[:, None]]


def rms_norm(x, weight=None, eps: float = 1e-5):
    """RMSNorm over the last axis (modules/norm_layer/layer_norm.py:41-59: apex FusedRMSNorm):
    x / sqrt(mean(x^2) + eps) * weight."""
    x = np.asarray(x, np.float64)
    y = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps)
    return y if weight is None else y * np.asarray(weight, np.float64)


def gated_attention_layer(x, P, chunk: int, num_heads: int = 1, moving_act: str = 'silu', eps: float = 1e-5,
                          num_groups: Optional[int] = None, bidirectional: bool = False, padding_mask=None,
                          simple_bias=None, attention_activation: str = 'softmax'):
    """MovingAverageGatedAttention.forward, unidirectional, softmax attention through the fused
    (rotary, causal, scale 1) op: modules/moving_average_gated_attention.py:263-417, step by
    step.  x: [B, L, D]; P: dict of numpy parameters
      norm_weight, norm_bias [D]; ema p, q, gamma [D, N], omega [D];
      v_w [E, D], v_b [E]; mx_w [D+S+E+D, D], mx_b; h_w [D, E]; gamma, beta [2, S];
      optional rms_weight [D] (the stored parameter: the multiplier is rms_weight + 1).
    num_heads > 1 splits q, k (S) and v (E) into heads laid out [B, L, Nh, H] (the layout of the
    fused op, csrc/ops/attention_kernel.cu:46-50); the reference layer itself is single-head."""
    x = np.asarray(x, np.float64)
    B, L, D = x.shape
    S = P['gamma'].shape[1]
    E = P['v_w'].shape[0]
    if bidirectional:
        # moving_average_gated_attention.py:84-87, 297-302: SequenceNorm, two-sided moving average
        xn = sequence_norm(x, np.asarray(P['norm_weight'], np.float64) + 1.0, P['norm_bias'], padding_mask, num_groups,
                           eps)[0]
    else:
        xn, _, _, _ = timestep_norm(x, np.zeros(B, np.int64), np.zeros((B, num_groups or D)),
                                    np.ones((B, num_groups or D)), np.asarray(P['norm_weight'], np.float64) + 1.0,
                                    P['norm_bias'], padding_mask, num_groups, eps)
    v = _silu(xn @ np.asarray(P['v_w'], np.float64).T + P['v_b'])
    mx, _ = ema_forward(xn.transpose(0, 2, 1), P['p'], P['q'], P['ema_gamma'], P['omega'], padding_mask,
                        bidirectional=bidirectional)
    mx = mx.transpose(0, 2, 1)
    # the RMSNorm weight is stored as its offset from one (norm_layer/layer_norm.py:47-56: zero-initialised, the
    # forward passes `self.weight + 1.0`); P['rms_weight'] is the stored parameter
    rms_w = None if P.get('rms_weight') is None else np.asarray(P['rms_weight'], np.float64) + 1.0
    mx = _silu(mx) if moving_act == 'silu' else rms_norm(mx, rms_w, eps)
    base = mx @ np.asarray(P['mx_w'], np.float64).T + P['mx_b']
    u, z, r, hx = np.split(base, [D, D + S, D + S + E], axis=-1)
    u = _sigmoid(u)
    z = z / np.maximum(np.sqrt((z * z).sum(-1, keepdims=True)), 1e-5)
    g = np.asarray(P['gamma'], np.float64) + 1.0
    bt = np.asarray(P['beta'], np.float64)
    q = z * g[0] + bt[0]
    k = z * g[1] + bt[1]
    r = _silu(r)
    nc = L // chunk if 1 < chunk < L else 1
    C = L // nc
    H1, H2 = S // num_heads, E // num_heads
    qc = q.reshape(B * nc, C, num_heads, H1)
    kc = k.reshape(B * nc, C, num_heads, H1)
    vc = v.reshape(B * nc, C, num_heads, H2)
    if simple_bias is None:
        # rotary on every head's features, positions restart in every chunk
        qr = rotary(qc.transpose(0, 2, 1, 3)).transpose(0, 2, 1, 3)
        kr = rotary(kc.transpose(0, 2, 1, 3)).transpose(0, 2, 1, 3)
    else:
        qr, kr = qc, kc
    if attention_activation != 'softmax':
        # element-wise attention (:153-208): scores over sqrt(keys seen), bias, relu^2 or the logistic
        # approximation of the Laplace function (fairseq/utils.py:444-457), then the masks as factors
        sc = np.einsum('blnh,bmnh->bnlm', qr, kr)
        pad = None if padding_mask is None else np.asarray(padding_mask, bool).reshape(B * nc, C)
        if not bidirectional:
            sc = sc / np.sqrt(np.arange(1, C + 1))[:, None]
        elif pad is not None:
            sc = sc / np.sqrt(np.maximum(C - pad.sum(-1), 1.0))[:, None, None, None]
        else:
            sc = sc / np.sqrt(C)
        if simple_bias is not None:
            sc = sc + simple_relative_bias(simple_bias, C)
        w = np.maximum(sc, 0.0) ** 2 if attention_activation == 'relu2' else _sigmoid((sc - 0.707107) * (1.702 / 0.282095))
        if pad is not None:
            w = w * (~pad)[:, None, None, :]
        if not bidirectional:
            w = w * np.tril(np.ones((C, C)))
        a = np.einsum('bnlm,bmnh->blnh', w, vc)
    elif bidirectional or simple_bias is not None:
        # softmax outside the fused op (:210-256): learned bias per relative offset j - i
        # (relative_positional_bias.py:25-42; simple_bias has 2 * max_positions - 1 entries), padded keys
        # excluded unless the whole chunk is padding, causal for one-sided layers
        sc = np.einsum('blnh,bmnh->bnlm', qr, kr)
        if simple_bias is not None:
            sc = sc + simple_relative_bias(simple_bias, C)
        if bidirectional and padding_mask is not None:
            pad = np.asarray(padding_mask, bool).reshape(B * nc, C)
            pad = pad & ~pad.all(-1, keepdims=True)
            sc = np.where(pad[:, None, None, :], -np.inf, sc)
        a = np.einsum('bnlm,bmnh->blnh', attention_softmax(sc, not bidirectional), vc)
    else:
        a, _ = attention(qr, kr, vc, 1.0, True)
    a = a.reshape(B, L, E)
    h = _silu(hx + (a * r) @ np.asarray(P['h_w'], np.float64).T)
    return x + u * (h - x)


# --------------------------------------------------------------------------
# f3/f4: the feed-forward block with its norm, and the decoder-only language model
# --------------------------------------------------------------------------


def normalized_ffn(x, P, norm_type: str = 'layernorm', eps: float = 1e-5):
    """NormalizedFeedForwardNetwork.forward (modules/normalized_feedforward_network.py:77-93):
    residual + [layerscale *] fc2(silu(fc1(norm(x)))).  P: norm_weight (stored as the offset from one,
    norm_layer/layer_norm.py:24-33, 47-56, 105-111) and norm_bias (layernorm only) or None, fc1_w [F, D], fc1_b [F],
    fc2_w [D, F], optional layerscale [D]."""
    x = np.asarray(x, np.float64)
    w = None if P.get('norm_weight') is None else np.asarray(P['norm_weight'], np.float64) + 1.0
    if norm_type == 'rmsnorm':
        xn = rms_norm(x, w, eps)
    else:
        mu = x.mean(-1, keepdims=True)
        xn = (x - mu) / np.sqrt(x.var(-1, keepdims=True) + eps)
        if w is not None:
            xn = xn * w + np.asarray(P['norm_bias'], np.float64)
    h = _silu(xn @ np.asarray(P['fc1_w'], np.float64).T + np.asarray(P['fc1_b'], np.float64))
    h = h @ np.asarray(P['fc2_w'], np.float64).T
    if P.get('layerscale') is not None:
        h = h * np.asarray(P['layerscale'], np.float64)
    return h + x


def mega_lm_decoder(tokens, P, chunk: int, padding_idx: int, num_groups: int, embed_scale: Optional[float],
                    moving_act: str = 'rmsnorm', norm_type: str = 'rmsnorm', eps: float = 1e-5,
                    simple_bias: bool = False, attention_activation: str = 'softmax'):
    """MegaDecoderNoCrossAttn.forward (models/mega_lm.py:267-386): tokens [B, T] (int) -> logits [B, T, V].
    The sequence is padded with padding_idx up to a whole number of chunks (:326-330), embedded and scaled (:333-335),
    run through the layers (mega_layer then nffn, modules/mega_layer.py:196-200) with the padding mask, normalised by
    the final TimestepNorm (:356), passed through pre_logits (fc + silu when present, :226-232), zeroed at padded
    positions (:360-363), cut back to T (:366-367) and projected (:379-385).
    P: embed [V, D]; layers: list of dicts {attn: gated_attention_layer's P (+ 'simple_bias' when simple_bias),
    ffn: normalized_ffn's P or None}; final_weight, final_bias [D]; optional pre_w [F, D], pre_b [F]; out_w [V, F]."""
    tokens = np.asarray(tokens)
    B, T = tokens.shape
    pad_to = T
    if T > chunk > 0 and T % chunk != 0:
        pad_to = -(-T // chunk) * chunk
        tokens = np.concatenate([tokens, np.full((B, pad_to - T), padding_idx, tokens.dtype)], 1)
    x = np.asarray(P['embed'], np.float64)[tokens]
    if embed_scale is not None:
        x = x * embed_scale
    mask = tokens == padding_idx
    if not mask.any():
        mask = None
    for lp in P['layers']:
        x = gated_attention_layer(x, lp['attn'], chunk if chunk > 0 else pad_to, 1, 'rms' if moving_act == 'rmsnorm' else 'silu',
                                  eps, num_groups, False, mask, lp['attn'].get('simple_bias') if simple_bias else None,
                                  attention_activation)
        if lp.get('ffn') is not None:
            x = normalized_ffn(x, lp['ffn'], norm_type, eps)
    G = num_groups
    x = timestep_norm(x, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)),
                      np.asarray(P['final_weight'], np.float64) + 1.0, P['final_bias'], mask, G, eps)[0]
    if P.get('pre_w') is not None:
        x = _silu(x @ np.asarray(P['pre_w'], np.float64).T + np.asarray(P['pre_b'], np.float64))
    if mask is not None:
        x = x * (~mask)[..., None]
    x = x[:, :T]
    return x @ np.asarray(P['out_w'], np.float64).T
