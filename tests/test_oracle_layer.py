"""Pins the layer-level functions of the oracle: swiglu, swiglu_ffn, silu_ffn, rms_norm, rotary,
simple_relative_bias and gated_attention_layer.

Three kinds of checks, chosen so that a plausible mistake (a dropped `+ 1`, a wrong split order, a transposed weight,
a wrong clamp, a wrong frequency convention) fails at least one of them:
  * values the mathematics fixes (silu identities, rms of a constant vector, identity / one-hot weights);
  * the reference's own outputs for its positional modules (tests/golden/position_vectors.npz, written by
    tests/golden/make_position_golden.py from fairseq/modules/relative_positional_bias.py);
  * for the gated-attention layer, a restatement of MovingAverageGatedAttention.forward
    (fairseq/modules/moving_average_gated_attention.py:153-412) with the library routines the reference itself
    calls (torch.split, F.normalize, F.silu, torch.sigmoid, torch.bmm, F.softmax, F.rms_norm) and explicit loops over
    chunks, on top of the oracle's already pinned primitives (timestep_norm, sequence_norm, ema_forward), plus special
    cases with closed-form answers.
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import mega_init_complex
from oracle import mega_oracle as O

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "position_vectors.npz"))


# ---------------------------------------------------------------- element-wise gates
def test_silu_identities_and_swiglu():
    x = np.linspace(-6, 6, 41)
    one = np.ones_like(x)
    silu = O.swiglu(x, one)                                  # silu(a) * 1
    assert np.allclose(silu - O.swiglu(-x, one), x, atol=1e-15)            # silu(x) - silu(-x) = x
    assert abs(O.swiglu(1.0, 1.0) - 0.7310585786300049) < 1e-15           # 1 / (1 + e^-1)
    assert O.swiglu(0.0, 3.0) == 0.0
    h = 1e-6
    assert abs((O.swiglu(h, 1.0) - O.swiglu(-h, 1.0)) / (2 * h) - 0.5) < 1e-9        # silu'(0) = 1/2
    assert abs(O.swiglu(-1.2784645427610738, 1.0) + 0.2784645427610738) < 1e-12     # the minimum of silu
    # linear in the second argument, not in the first
    rng = np.random.default_rng(0)
    a, b, c = rng.normal(size=(3, 5, 7))
    assert np.allclose(O.swiglu(a, 2.5 * b - c), 2.5 * O.swiglu(a, b) - O.swiglu(a, c), atol=1e-14)
    assert np.allclose(O.swiglu(a, b), F.silu(torch.from_numpy(a)).numpy() * b, atol=1e-15)
    # which argument goes through silu
    assert not np.allclose(O.swiglu(a, b), O.swiglu(b, a))


def test_rms_norm_closed_forms_and_library():
    eps = 1e-5
    for c in (3.0, -0.5, 1e-3):
        y = O.rms_norm(np.full((2, 8), c), None, eps)
        assert np.allclose(y, c / np.sqrt(c * c + eps), atol=1e-15)
    w = np.arange(1.0, 9.0)
    assert np.allclose(O.rms_norm(np.full((1, 8), 2.0), w, eps), 2.0 / np.sqrt(4.0 + eps) * w)
    rng = np.random.default_rng(1)
    x = rng.normal(size=(3, 4, 16)) * 5
    # scale invariance up to eps; the mean of squares, not of the values, not the variance
    assert np.allclose(O.rms_norm(1e4 * x, w.repeat(2), eps), O.rms_norm(x, w.repeat(2), 1e-13), atol=1e-9)
    shifted = x + 10.0
    assert np.allclose((O.rms_norm(shifted, None, 0.0) ** 2).mean(-1), 1.0)
    assert np.all(O.rms_norm(np.zeros((2, 4)), None, eps) == 0)
    ref = F.rms_norm(torch.from_numpy(x), (16,), torch.from_numpy(w.repeat(2)), eps).numpy()
    assert np.allclose(O.rms_norm(x, w.repeat(2), eps), ref, atol=1e-14)


def test_feed_forward_blocks_against_row_loops_and_one_hot_weights():
    rng = np.random.default_rng(2)
    T, D, Hd = 5, 4, 6
    x = rng.normal(size=(T, D))
    w1, w3 = rng.normal(size=(2, Hd, D))
    w2 = rng.normal(size=(D, Hd))
    b1, b2 = rng.normal(size=Hd), rng.normal(size=D)

    def silu(v):
        return v / (1.0 + np.exp(-v))

    got = O.swiglu_ffn(x, w1, w3, w2)
    got_s = O.silu_ffn(x, w1, b1, w2, b2)
    for t in range(T):
        hid = np.array([silu(sum(w1[h, d] * x[t, d] for d in range(D))) * sum(w3[h, d] * x[t, d] for d in range(D))
                        for h in range(Hd)])
        assert np.allclose(got[t], [sum(w2[d, h] * hid[h] for h in range(Hd)) for d in range(D)], atol=1e-13)
        hid = np.array([silu(sum(w1[h, d] * x[t, d] for d in range(D)) + b1[h]) for h in range(Hd)])
        assert np.allclose(got_s[t], [x[t, d] + sum(w2[d, h] * hid[h] for h in range(Hd)) + b2[d] for d in range(D)],
                           atol=1e-13)
    # identity weights: W2 (silu(x) * x); the residual of the SiLU block is x itself
    eye = np.eye(D)
    assert np.allclose(O.swiglu_ffn(x, eye, eye, eye), silu(x) * x)
    assert np.allclose(O.silu_ffn(x, eye, 0.0, eye, 0.0), x + silu(x))
    assert np.allclose(O.silu_ffn(x, eye, 0.0, np.zeros((D, D)), b2), x + b2)
    # one-hot weights fix the [out, in] convention: hidden unit 2 reads input 1 (gate) and input 3 (value),
    # output 0 reads hidden unit 2
    e1 = np.zeros((Hd, D)); e1[2, 1] = 1
    e3 = np.zeros((Hd, D)); e3[2, 3] = 1
    e2 = np.zeros((D, Hd)); e2[0, 2] = 1
    out = O.swiglu_ffn(x, e1, e3, e2)
    assert np.allclose(out[:, 0], silu(x[:, 1]) * x[:, 3]) and np.all(out[:, 1:] == 0)
    out = O.silu_ffn(x, e1, 0.0, e2, 0.0)
    assert np.allclose(out[:, 0], x[:, 0] + silu(x[:, 1])) and np.allclose(out[:, 1:], x[:, 1:])


# ---------------------------------------------------------------- positions: the reference modules' own outputs
@pytest.mark.parametrize("tag", ["rot_a", "rot_b", "rot_c", "rot_d"])
def test_rotary_matches_the_reference_module(tag):
    xq, xk = GOLD[f"{tag}.xq"], GOLD[f"{tag}.xk"]
    base, qidx = float(GOLD[f"{tag}.base"]), int(GOLD[f"{tag}.qidx"])
    # the reference rotates in fp32 (x.float(), complex64 phases): 1e-6 of the values
    assert np.allclose(O.rotary(xk, base), GOLD[f"{tag}.k"], atol=2e-6)
    assert np.allclose(O.rotary(xq, base, start=qidx), GOLD[f"{tag}.q"], atol=2e-6)
    S = xk.shape[-1]
    assert np.allclose(GOLD[f"{tag}.freqs"], base ** (-np.arange(0, S, 2) / S), rtol=1e-6)
    # a wrong pairing (halves instead of neighbours) or a wrong exponent would not pass
    half = np.concatenate([xk[..., : S // 2], xk[..., S // 2:]], -1)
    assert not np.allclose(O.rotary(half[..., np.r_[0:S:2, 1:S:2]], base), GOLD[f"{tag}.k"], atol=1e-3)


@pytest.mark.parametrize("tag", ["bias_a", "bias_b", "bias_c", "bias_d"])
def test_simple_relative_bias_matches_the_reference_module(tag):
    param, C = GOLD[f"{tag}.param"], int(GOLD[f"{tag}.C"])
    m = O.simple_relative_bias(param, C)
    assert m.shape == (C, C)
    assert np.array_equal(m, GOLD[f"{tag}.matrix"])
    mp = (len(param) + 1) // 2
    with pytest.raises(ValueError):
        O.simple_relative_bias(param, mp + 1)


# ---------------------------------------------------------------- the gated-attention layer
def _params(rng, D, S, E, N, bidirectional=False):
    K = 2 * D if bidirectional else D
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    return dict(norm_weight=rng.normal(size=D) * 0.1, norm_bias=rng.normal(size=D) * 0.1, p=p, q=q, ema_gamma=g,
                omega=rng.normal(size=D), v_w=rng.normal(size=(E, D)) * 0.3, v_b=rng.normal(size=E) * 0.1,
                mx_w=rng.normal(size=(2 * D + S + E, D)) * 0.3, mx_b=rng.normal(size=2 * D + S + E) * 0.1,
                h_w=rng.normal(size=(D, E)) * 0.3, gamma=rng.normal(size=(2, S)) * 0.3, beta=rng.normal(size=(2, S)) * 0.3,
                rms_weight=rng.normal(size=D) * 0.2)


def _restated_layer(x, P, chunk, num_groups, moving_act="silu", bidirectional=False, padding_mask=None,
                    simple_bias=None, attention_activation="softmax", eps=1e-5):
    """MovingAverageGatedAttention.forward (moving_average_gated_attention.py:295-412) with torch library calls and a
    loop over chunks; the norm and the moving average come from the oracle's pinned primitives."""
    t = torch.from_numpy
    B, L, D = x.shape
    S, E = P["gamma"].shape[1], P["v_w"].shape[0]
    G = num_groups or D
    if bidirectional:                                   # :297-302
        xn = O.sequence_norm(x, P["norm_weight"] + 1.0, P["norm_bias"], padding_mask, num_groups, eps)[0]
    else:                                               # :303-309
        xn = O.timestep_norm(x, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), P["norm_weight"] + 1.0,
                             P["norm_bias"], padding_mask, num_groups, eps)[0]
    v = F.silu(F.linear(t(xn), t(P["v_w"]), t(P["v_b"])))                    # :301 / :307
    mx = O.ema_forward(xn.transpose(0, 2, 1), P["p"], P["q"], P["ema_gamma"], P["omega"], padding_mask,
                       bidirectional=bidirectional)[0].transpose(0, 2, 1)   # :312-314
    mx = t(np.ascontiguousarray(mx))
    # :315; RMSNorm = FusedRMSNorm: `weight = self.weight + 1.0`, rms norm with it (norm_layer/layer_norm.py:54-56)
    mx = F.silu(mx) if moving_act == "silu" else F.rms_norm(mx, (D,), t(P["rms_weight"]) + 1.0, eps)
    base = F.linear(mx, t(P["mx_w"]), t(P["mx_b"]))                         # :318
    u, z, r, hx = torch.split(base, [D, S, E, D], dim=-1)                    # :319
    u = torch.sigmoid(u)                                                     # :321
    z = F.normalize(z, p=2, dim=-1, eps=1e-5)                                # :323
    z = z.unsqueeze(2) * (t(P["gamma"]) + 1.0) + t(P["beta"])                # :325
    q, k = torch.unbind(z, dim=2)                                            # :327
    r = F.silu(r)                                                            # :329
    nc = L // chunk if 1 < chunk < L else 1
    C = L // nc
    q, k, v = q.reshape(B * nc, C, S), k.reshape(B * nc, C, S), v.reshape(B * nc, C, E)      # :374-385
    pad = None if padding_mask is None else t(np.asarray(padding_mask, bool)).view(B * nc, C)
    attn = torch.zeros(B * nc, C, E, dtype=torch.float64)
    causal = torch.tril(torch.ones(C, C, dtype=torch.float64))
    for c in range(B * nc):
        qc, kc = q[c], k[c]
        bias = 0.0
        if simple_bias is not None:
            bias = t(O.simple_relative_bias(simple_bias, C))                 # pinned against the reference module
        else:
            qc, kc = t(O.rotary(qc.numpy())), t(O.rotary(kc.numpy()))        # pinned against the reference module
        qk = qc @ kc.T
        if attention_activation == "softmax":                                # softmax_attention, :210-246
            qk = qk + bias
            if not bidirectional:
                qk = qk.masked_fill(causal == 0, float("-inf"))              # the causal attn_mask / fused op
            if pad is not None and bidirectional:
                pm = pad[c] & ~pad[c].all()
                qk = qk.masked_fill(pm[None, :], float("-inf"))
            w = F.softmax(qk, dim=-1)
        else:                                                                # element_attention, :153-208
            if not bidirectional:
                len_scale = torch.rsqrt(causal.sum(-1, keepdim=True))        # :167-169
            elif pad is not None:
                len_scale = torch.rsqrt((C - pad[c].sum()).clamp(min=1.0).double())
            else:
                len_scale = 1.0 / np.sqrt(C)
            qk = qk * len_scale + bias
            w = torch.square(F.relu(qk)) if attention_activation == "relu2" else \
                torch.sigmoid((qk - 0.707107) * (1.702 / 0.282095))          # utils.py:444-457
            if pad is not None:
                w = w * (1.0 - pad[c].double())[None, :]
            if not bidirectional:
                w = w * causal
        attn[c] = w @ v[c]
    attn = attn.view(B, L, E) * r                                            # :406
    h = F.silu(hx + F.linear(attn, t(P["h_w"])))                             # :408
    return torch.addcmul(t(x), u, h - t(x)).numpy()                          # :411


@pytest.mark.parametrize("case", [
    dict(),                                                            # one-sided softmax through the fused op
    dict(moving_act="rms"),
    dict(attention_activation="relu2"),
    dict(attention_activation="laplace"),
    dict(simple=True),
    dict(simple=True, attention_activation="laplace"),
    dict(bidirectional=True, padded=True),
    dict(bidirectional=True, padded=True, attention_activation="relu2"),
    dict(bidirectional=True, simple=True),
    dict(padded=True),                                                 # one-sided with right padding
])
def test_layer_against_the_restated_forward(case):
    rng = np.random.default_rng(11)
    B, L, D, S, E, N, chunk, G = 2, 12, 8, 4, 6, 4, 4, 2
    bid = case.get("bidirectional", False)
    P = _params(rng, D, S, E, N, bid)
    x = rng.normal(size=(B, L, D))
    mask = None
    if case.get("padded"):
        mask = np.zeros((B, L), bool)
        mask[0, 9:] = True                               # the last chunk of row 0 is half padding, row 1 has none
        if bid:
            mask[1, 8:] = True                           # a chunk that is all padding (keeps all keys, :234-236)
    sb = rng.normal(size=2 * 5 - 1) * 0.5 if case.get("simple") else None
    kw = dict(moving_act=case.get("moving_act", "silu"), bidirectional=bid, padding_mask=mask, simple_bias=sb,
              attention_activation=case.get("attention_activation", "softmax"))
    got = O.gated_attention_layer(x, P, chunk, num_groups=G, **kw)
    want = _restated_layer(x, P, chunk, G, **kw)
    assert np.allclose(got, want, atol=1e-11), np.abs(got - want).max()


def test_layer_special_cases_with_closed_forms():
    rng = np.random.default_rng(12)
    B, L, D, S, E, N, chunk, G = 2, 8, 6, 4, 5, 3, 4, 2
    P = _params(rng, D, S, E, N)
    x = rng.normal(size=(B, L, D))

    def silu(v):
        return v / (1.0 + np.exp(-v))

    # the pieces every case below needs, from pinned primitives
    xn = O.timestep_norm(x, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), P["norm_weight"] + 1.0,
                         P["norm_bias"], None, G, 1e-5)[0]
    v = silu(xn @ P["v_w"].T + P["v_b"])
    mx = silu(O.ema_forward(xn.transpose(0, 2, 1), P["p"], P["q"], P["ema_gamma"], P["omega"])[0].transpose(0, 2, 1))
    base = mx @ P["mx_w"].T + P["mx_b"]
    u, r, hx = 1 / (1 + np.exp(-base[..., :D])), silu(base[..., D + S:D + S + E]), base[..., D + S + E:]

    # (1) gamma = -1, beta = 0  =>  q = k = 0  =>  equal weights over the keys seen so far in the chunk:
    #     attn[t] = mean(v[chunk start .. t]).  A missing `+ 1` on gamma leaves q = -z and fails this.
    P1 = dict(P, gamma=-np.ones((2, S)), beta=np.zeros((2, S)))
    a = np.stack([v[:, (t // chunk) * chunk:t + 1].mean(1) for t in range(L)], 1)
    want = x + u * (silu(hx + (a * r) @ P["h_w"].T) - x)
    assert np.allclose(O.gated_attention_layer(x, P1, chunk, num_groups=G), want, atol=1e-12)

    # (2) W_h = 0  =>  h = silu(hx): out = x + sigmoid(u) (silu(hx) - x), whatever the attention does.  Fixes the
    #     places of u (first D columns of mx_proj) and hx (last D columns).
    P2 = dict(P, h_w=np.zeros_like(P["h_w"]))
    assert np.allclose(O.gated_attention_layer(x, P2, chunk, num_groups=G), x + u * (silu(hx) - x), atol=1e-12)

    # (3) z below the clamp of F.normalize (eps = 1e-5): z / 1e-5, not z / |z|.  With q = z' (gamma0 = 0, beta0 = 0)
    #     and k = beta1 the scores are (z / 1e-5) . beta1 per query: the same for every key, so again equal weights;
    #     with a unit-norm z they would differ from key to key only through rotary, so use one chunk position pair
    #     whose closed form separates the two: compare against the restated forward and against a variant clamp.
    P3 = dict(P, mx_w=P["mx_w"].copy(), mx_b=P["mx_b"].copy())
    P3["mx_w"][D:D + S] = 0.0
    P3["mx_b"][D:D + S] = 1e-7 * np.arange(1, S + 1)
    got = O.gated_attention_layer(x, P3, chunk, num_groups=G)
    assert np.allclose(got, _restated_layer(x, P3, chunk, G), atol=1e-12)
    zc = P3["mx_b"][D:D + S] / 1e-5                                           # what the clamp makes of z
    zu = P3["mx_b"][D:D + S] / np.linalg.norm(P3["mx_b"][D:D + S])            # what a missing clamp would make
    g, bt = P["gamma"] + 1.0, P["beta"]

    def with_z(zv):
        q = np.broadcast_to(zv * g[0] + bt[0], (B, L, S))
        k = np.broadcast_to(zv * g[1] + bt[1], (B, L, S))
        out = np.empty((B, L, E))
        for b in range(B):
            for c0 in range(0, L, chunk):
                qr, kr = O.rotary(q[b, c0:c0 + chunk]), O.rotary(k[b, c0:c0 + chunk])
                w = O.attention_softmax((qr @ kr.T)[None], True)[0]
                out[b, c0:c0 + chunk] = w @ v[b, c0:c0 + chunk]
        return x + u * (silu(hx + (out * r) @ P["h_w"].T) - x)

    assert np.allclose(got, with_z(zc), atol=1e-12)
    assert not np.allclose(got, with_z(zu), atol=1e-6)

    # (4) u == 0 (a very negative gate bias): the identity layer
    P4 = dict(P, mx_w=P["mx_w"].copy(), mx_b=P["mx_b"].copy())
    P4["mx_w"][:D] = 0.0
    P4["mx_b"][:D] = -1e4
    assert np.allclose(O.gated_attention_layer(x, P4, chunk, num_groups=G), x, atol=1e-12)

    # (5) one-hot rows of mx_proj identify the four slices: only r's columns non-zero  =>  u = 1/2, z = 0 (q = beta0,
    #     k = beta1), hx = 0: out = x + (silu(W_h (a r)) - x) / 2 with r = silu(mx[..., 0]) in every column of the slice
    P5 = dict(P, mx_w=np.zeros_like(P["mx_w"]), mx_b=np.zeros_like(P["mx_b"]))
    P5["mx_w"][D + S:D + S + E, 0] = 1.0
    r5 = silu(mx[..., :1]).repeat(E, -1)
    q5 = np.broadcast_to(bt[0], (B, L, S)); k5 = np.broadcast_to(bt[1], (B, L, S))
    a5 = np.empty((B, L, E))
    for b in range(B):
        for c0 in range(0, L, chunk):
            w = O.attention_softmax((O.rotary(q5[b, c0:c0 + chunk]) @ O.rotary(k5[b, c0:c0 + chunk]).T)[None], True)[0]
            a5[b, c0:c0 + chunk] = w @ v[b, c0:c0 + chunk]
    want = x + 0.5 * (silu((a5 * r5) @ P["h_w"].T) - x)
    assert np.allclose(O.gated_attention_layer(x, P5, chunk, num_groups=G), want, atol=1e-12)


def test_layer_heads_split_features_not_tokens():
    """num_heads > 1 (north-star spec; the reference layer is single-head): head n owns features
    [n S/Nh, (n+1) S/Nh) of q, k and [n E/Nh, (n+1) E/Nh) of v, rotary per head; equal to single-head layers run on
    the feature slices."""
    rng = np.random.default_rng(13)
    B, L, D, S, E, N, chunk, G, Nh = 1, 8, 6, 4, 6, 3, 4, 2, 2
    P = _params(rng, D, S, E, N)
    x = rng.normal(size=(B, L, D))
    P0 = dict(P, h_w=np.eye(D, E))                      # h_proj copies the first D columns of attn * r
    got = O.gated_attention_layer(x, P0, chunk, num_heads=Nh, num_groups=G)

    def silu(v):
        return v / (1.0 + np.exp(-v))

    xn = O.timestep_norm(x, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), P["norm_weight"] + 1.0,
                         P["norm_bias"], None, G, 1e-5)[0]
    v = silu(xn @ P["v_w"].T + P["v_b"])
    mx = silu(O.ema_forward(xn.transpose(0, 2, 1), P["p"], P["q"], P["ema_gamma"], P["omega"])[0].transpose(0, 2, 1))
    base = mx @ P["mx_w"].T + P["mx_b"]
    u, z, r, hx = 1 / (1 + np.exp(-base[..., :D])), base[..., D:D + S], silu(base[..., D + S:D + S + E]), base[..., D + S + E:]
    z = z / np.maximum(np.linalg.norm(z, axis=-1, keepdims=True), 1e-5)
    q, k = z * (P["gamma"][0] + 1) + P["beta"][0], z * (P["gamma"][1] + 1) + P["beta"][1]
    a = np.empty((B, L, E))
    H1, H2 = S // Nh, E // Nh
    for n in range(Nh):
        for c0 in range(0, L, chunk):
            qr = O.rotary(q[0, c0:c0 + chunk, n * H1:(n + 1) * H1])
            kr = O.rotary(k[0, c0:c0 + chunk, n * H1:(n + 1) * H1])
            w = O.attention_softmax((qr @ kr.T)[None], True)[0]
            a[0, c0:c0 + chunk, n * H2:(n + 1) * H2] = w @ v[0, c0:c0 + chunk, n * H2:(n + 1) * H2]
    want = x + u * (silu(hx + (a * r)[..., :D]) - x)
    assert np.allclose(got, want, atol=1e-12)


# --------------------------------------------------------------------------
# the feed-forward block with its norm, and the whole decoder-only model
# --------------------------------------------------------------------------


@pytest.mark.parametrize("norm_type", ["layernorm", "rmsnorm"])
@pytest.mark.parametrize("affine,scale", [(True, True), (True, False), (False, False)])
def test_normalized_ffn_against_library_calls(norm_type, affine, scale):
    """normalized_feedforward_network.py:77-93 typed with torch's own layer_norm / linear / silu, the norm's multiplier
    being the stored weight plus one (norm_layer/layer_norm.py:24-33, 47-56, 105-111)."""
    rng = np.random.default_rng(11)
    D, Fh = 12, 20
    x = rng.standard_normal((2, 5, D))
    P = dict(norm_weight=rng.standard_normal(D) * 0.3 if affine else None,
             norm_bias=rng.standard_normal(D) * 0.3 if affine and norm_type == "layernorm" else None,
             fc1_w=rng.standard_normal((Fh, D)), fc1_b=rng.standard_normal(Fh), fc2_w=rng.standard_normal((D, Fh)),
             layerscale=rng.random(D) + 0.1 if scale else None)
    t = lambda a: None if a is None else torch.from_numpy(np.asarray(a, np.float64))
    xt = t(x)
    if norm_type == "layernorm":
        xn = F.layer_norm(xt, (D,), None if not affine else t(P["norm_weight"]) + 1.0, t(P["norm_bias"]), 1e-5)
    else:
        xn = xt * torch.rsqrt(xt.pow(2).mean(-1, keepdim=True) + 1e-5)
        if affine:
            xn = xn * (t(P["norm_weight"]) + 1.0)
    h = F.linear(F.silu(F.linear(xn, t(P["fc1_w"]), t(P["fc1_b"]))), t(P["fc2_w"]))
    want = (h * t(P["layerscale"]) if scale else h) + xt
    got = O.normalized_ffn(x, P, norm_type, 1e-5)
    assert np.abs(got - want.numpy()).max() < 1e-12
    # zero second projection: the block is the identity, whatever the norm does
    P0 = dict(P, fc2_w=np.zeros((D, Fh)))
    assert np.array_equal(O.normalized_ffn(x, P0, norm_type), x)


def _model_params(rng, V, D, S, E, N, Fh, n_layers, G, rep=None):
    layers = []
    for _ in range(n_layers):
        A = _params(rng, D, S, E, N)
        A["rms_weight"] = rng.standard_normal(D) * 0.2
        ffn = dict(norm_weight=rng.standard_normal(D) * 0.2, norm_bias=None, fc1_w=rng.standard_normal((Fh, D)) * 0.3,
                   fc1_b=rng.standard_normal(Fh) * 0.1, fc2_w=rng.standard_normal((D, Fh)) * 0.3, layerscale=None)
        layers.append(dict(attn=A, ffn=ffn))
    emb = rng.standard_normal((V, D))
    emb[1] = 0.0                                                     # the padding row of nn.Embedding
    P = dict(embed=emb, layers=layers, final_weight=rng.standard_normal(D) * 0.2, final_bias=rng.standard_normal(D) * 0.2,
             out_w=rng.standard_normal((V, rep or D)))
    if rep:
        P["pre_w"], P["pre_b"] = rng.standard_normal((rep, D)), rng.standard_normal(rep)
    return P


def test_model_without_layers_is_norm_and_projection():
    """No layers: logits = W_out silu(W_pre tsn(scale * E[tokens]) + b_pre), the norm in its textbook form (prefix
    means and variances), the rest through torch's library calls; a dropped scale, a missing `+ 1` on the norm's
    weight, a transposed projection or a forgotten pre_logits activation each change the result."""
    rng = np.random.default_rng(12)
    V, D, G, rep = 17, 8, 2, 6
    P = _model_params(rng, V, D, 4, 8, 2, 8, 0, G, rep)
    tok = rng.integers(2, V, (2, 9))
    got = O.mega_lm_decoder(tok, P, 4, 1, G, 3.0)                     # 9 tokens, chunk 4: padded to 12, cut back to 9
    pad = np.zeros((2, 12), bool)
    pad[:, 9:] = True
    x = np.concatenate([P["embed"][tok] * 3.0, np.zeros((2, 3, D))], 1)
    y = O.timestep_norm_closed_form(x, pad, G, 1e-5, P["final_weight"] + 1.0, P["final_bias"])[0][:, :9]
    t = lambda a: torch.from_numpy(np.asarray(a, np.float64))
    want = F.linear(F.silu(F.linear(t(y), t(P["pre_w"]), t(P["pre_b"]))), t(P["out_w"])).numpy()
    assert got.shape == (2, 9, V) and np.abs(got - want).max() < 1e-10
    # without the scale the norm sees other numbers (eps is not scale-free) and without pre_logits other features
    assert np.abs(O.mega_lm_decoder(tok, P, 4, 1, G, None) - want).max() > 1e-7
    P2 = {k: v for k, v in P.items() if k not in ("pre_w", "pre_b")}
    P2["out_w"] = rng.standard_normal((V, D))
    assert np.abs(O.mega_lm_decoder(tok, P2, 4, 1, G, 3.0) - y @ P2["out_w"].T).max() < 1e-10


def test_model_is_layers_then_ffn_in_order_and_pads_like_the_reference():
    """Two layers: (a) the order is attention layer, feed-forward, attention layer, feed-forward (mega_layer.py:196-200,
    mega_lm.py:348-354), checked by composing the pinned pieces by hand; (b) every position is causal in the tokens;
    (c) a length that is not a whole number of chunks gives the first rows of the longer sequence's logits, the padded
    end being cut off (mega_lm.py:326-330, 366-367); (d) padding tokens inside the input give zero logits there
    (mega_lm.py:360-363) and do not count in the norms."""
    rng = np.random.default_rng(13)
    V, D, S, E, N, Fh, G, C = 19, 8, 4, 8, 2, 12, 2, 4
    P = _model_params(rng, V, D, S, E, N, Fh, 2, G)
    tok = rng.integers(2, V, (2, 12))
    got = O.mega_lm_decoder(tok, P, C, 1, G, 2.0)
    x = P["embed"][tok] * 2.0
    for lp in P["layers"]:
        x = O.gated_attention_layer(x, lp["attn"], C, 1, "rms", 1e-5, G)
        x = O.normalized_ffn(x, lp["ffn"], "rmsnorm", 1e-5)
    y = O.timestep_norm_closed_form(x, None, G, 1e-5, P["final_weight"] + 1.0, P["final_bias"])[0]
    assert np.abs(got - y @ P["out_w"].T).max() < 1e-10
    # swapping the two layers' parameters changes the result: the order is not symmetric
    Q = dict(P, layers=P["layers"][::-1])
    assert np.abs(O.mega_lm_decoder(tok, Q, C, 1, G, 2.0) - got).max() > 1e-6
    # (b)
    tok2 = tok.copy()
    tok2[:, 7] = (tok2[:, 7] - 2 + 1) % (V - 2) + 2
    alt = O.mega_lm_decoder(tok2, P, C, 1, G, 2.0)
    assert np.abs(alt[:, :7] - got[:, :7]).max() < 1e-11 and np.abs(alt[:, 7:] - got[:, 7:]).max() > 1e-6
    # (c)
    short = O.mega_lm_decoder(tok[:, :10], P, C, 1, G, 2.0)
    assert short.shape == (2, 10, V) and np.abs(short - got[:, :10]).max() < 1e-11
    # a single chunk or less is not padded (seq_len > chunk fails, mega_lm.py:326): three tokens stay three
    assert np.abs(O.mega_lm_decoder(tok[:, :3], P, C, 1, G, 2.0) - got[:, :3]).max() < 1e-11
    # (d)
    tok3 = tok.copy()
    tok3[0, 8:] = 1
    padded = O.mega_lm_decoder(tok3, P, C, 1, G, 2.0)
    assert np.array_equal(padded[0, 8:], np.zeros((4, V)))
    assert np.abs(padded[0, :8] - got[0, :8]).max() < 1e-11 and np.abs(padded[1] - got[1]).max() < 1e-11
