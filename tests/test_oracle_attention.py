"""Pins the attention-softmax / attention / gate parts of the oracle."""
import numpy as np

from oracle import mega_oracle as O


def test_softmax_plain_and_right_aligned_causal():
    rng = np.random.default_rng(0)
    x = rng.normal(size=(2, 3, 4, 6))
    y = O.attention_softmax(x, False)
    e = np.exp(x - x.max(-1, keepdims=True))
    assert np.allclose(y, e / e.sum(-1, keepdims=True), atol=1e-14)
    yc = O.attention_softmax(x, True)
    for r in range(4):
        n = 6 - 4 + r + 1
        e = np.exp(x[..., r, :n] - x[..., r, :n].max(-1, keepdims=True))
        assert np.allclose(yc[..., r, :n], e / e.sum(-1, keepdims=True), atol=1e-14)
        assert np.all(yc[..., r, n:] == 0)
    assert np.allclose(yc.sum(-1), 1)


def test_softmax_fully_masked_rows_are_zero():
    x = np.full((1, 2, 3), -np.inf)
    x[0, 1, 0] = 0.5
    y = O.attention_softmax(x, False)
    assert np.all(y[0, 0] == 0) and np.allclose(y[0, 1], [1, 0, 0])
    # outer > inner with the causal mask: the first rows keep no column at all
    y = O.attention_softmax(np.zeros((1, 4, 2)), True)
    assert np.all(y[0, :2] == 0) and np.allclose(y[0, 2], [1, 0]) and np.allclose(y[0, 3], [.5, .5])


def test_attention_matches_loops_and_chunks_are_independent():
    rng = np.random.default_rng(1)
    B, L, Nh, H1, H2 = 2, 5, 2, 3, 4
    q = rng.normal(size=(B, L, Nh, H1)); k = rng.normal(size=(B, L, Nh, H1)); v = rng.normal(size=(B, L, Nh, H2))
    y, w = O.attention(q, k, v, 0.7, True)
    for b in range(B):
        for n in range(Nh):
            for l in range(L):
                s = np.array([0.7 * q[b, l, n] @ k[b, j, n] for j in range(l + 1)])
                p = np.exp(s - s.max()); p /= p.sum()
                assert np.allclose(y[b, l, n], sum(p[j] * v[b, j, n] for j in range(l + 1)), atol=1e-12)
                assert np.allclose(w[b, n, l, :l + 1], p, atol=1e-14) and np.all(w[b, n, l, l + 1:] == 0)
    q2 = q.copy(); q2[1] += 1.0
    y2, _ = O.attention(q2, k, v, 0.7, True)
    assert np.array_equal(y2[0], y[0])


def test_swiglu_and_rotary():
    a = np.array([-2.0, 0.0, 3.0]); b = np.array([1.5, 2.0, -1.0])
    assert np.allclose(O.swiglu(a, b), a / (1 + np.exp(-a)) * b)
    rng = np.random.default_rng(2)
    x = rng.normal(size=(2, 7, 8))
    r = O.rotary(x)
    assert np.allclose(r[:, 0], x[:, 0])                                   # position 0 is not rotated
    assert np.allclose((r ** 2).sum(-1), (x ** 2).sum(-1))                 # rotations keep the norm
    # q.k after rotary depends on the position difference only
    q = rng.normal(size=(1, 1, 8)).repeat(7, 1); k = rng.normal(size=(1, 1, 8)).repeat(7, 1)
    rq, rk = O.rotary(q), O.rotary(k)
    assert np.isclose(rq[0, 5] @ rk[0, 3], rq[0, 4] @ rk[0, 2])


def _layer_params(rng, D, S, E, N):
    from conftest import mega_init_complex
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    return dict(norm_weight=rng.normal(size=D) * 0.1, norm_bias=rng.normal(size=D) * 0.1, p=p, q=q, ema_gamma=g,
                omega=rng.normal(size=D), v_w=rng.normal(size=(E, D)) * 0.2, v_b=rng.normal(size=E) * 0.1,
                mx_w=rng.normal(size=(2 * D + S + E, D)) * 0.2, mx_b=rng.normal(size=2 * D + S + E) * 0.1,
                h_w=rng.normal(size=(D, E)) * 0.2, gamma=rng.normal(size=(2, S)) * 0.1, beta=rng.normal(size=(2, S)) * 0.1)


def test_layer_gate_closed_forms_and_chunk_causality():
    rng = np.random.default_rng(5)
    B, L, D, S, E, N = 2, 12, 8, 4, 6, 4
    P = _layer_params(rng, D, S, E, N)
    x = rng.normal(size=(B, L, D))
    y = O.gated_attention_layer(x, P, chunk=4, num_groups=2)
    # u == 0 (a very negative gate bias) makes the layer the identity
    P0 = dict(P); P0['mx_b'] = P['mx_b'].copy(); P0['mx_b'][:D] = -1e4; P0['mx_w'] = P['mx_w'].copy(); P0['mx_w'][:D] = 0
    assert np.allclose(O.gated_attention_layer(x, P0, chunk=4, num_groups=2), x, atol=1e-12)
    # causal: outputs before t do not see x[t:]
    x2 = x.copy(); x2[:, 7:] += rng.normal(size=(B, 5, D))
    y2 = O.gated_attention_layer(x2, P, chunk=4, num_groups=2)
    assert np.allclose(y2[:, :7], y[:, :7], atol=1e-10) and not np.allclose(y2[:, 7:], y[:, 7:])
    # head split with one head equals the single-head layer; rms variant follows its formula
    assert np.allclose(O.gated_attention_layer(x, P, chunk=4, num_heads=1, num_groups=2), y)
    z = rng.normal(size=(3, 5))
    assert np.allclose(O.rms_norm(z, None, 1e-5), z / np.sqrt((z ** 2).mean(-1, keepdims=True) + 1e-5))
    yh = O.gated_attention_layer(x, P, chunk=4, num_heads=2, num_groups=2)
    assert yh.shape == y.shape and not np.allclose(yh, y)


def test_dropkey_draws_and_masked_softmax(tmp_path):
    """The draws: against a C restatement of the hash (64-bit wrap-around and the 24-bit float
    conversion are where numpy could differ), uniform, independent from row to row.  The masked
    softmax: equal to the plain softmax over the surviving keys, zeros at dropped keys and in rows
    that lose every key (softmax.cuh:157-185)."""
    import subprocess
    src = tmp_path / "h.c"
    src.write_text(r'''
#include <stdio.h>
#include <stdint.h>
int main(void) {
  const uint64_t seeds[2] = {12345ull, 0xFEDCBA9876543210ull};
  for (int s = 0; s < 2; ++s)
    for (uint64_t i = 0; i < 64; ++i) {
      uint64_t z = seeds[s] + (i + 1) * 0x9E3779B97F4A7C15ull;
      z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
      z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
      z ^= z >> 31;
      printf("%.9g\n", (float)(z >> 40) * (1.0f / 16777216.0f));
    }
  return 0;
}''')
    exe = tmp_path / "h"
    subprocess.run(["gcc", "-O1", str(src), "-o", str(exe)], check=True)
    out = np.array([float(t) for t in subprocess.run([str(exe)], check=True, capture_output=True,
                                                     text=True).stdout.split()])
    got = np.concatenate([O.dropkey_draws(12345, (64,)), O.dropkey_draws(0xFEDCBA9876543210, (8, 8)).ravel()])
    assert np.array_equal(out.astype(np.float32), got.astype(np.float32))      # %.9g round-trips fp32
    d = O.dropkey_draws(99, (2000, 500))
    assert 0 <= d.min() and d.max() < 1 and abs(d.mean() - 0.5) < 2e-3 and abs(d.var() - 1 / 12) < 1e-3
    assert abs(np.corrcoef(d[:-1].ravel(), d[1:].ravel())[0, 1]) < 5e-3
    assert abs(np.corrcoef(d[:, :-1].ravel(), d[:, 1:].ravel())[0, 1]) < 5e-3
    rng = np.random.default_rng(5)
    x = rng.normal(size=(3, 6, 9))
    drop = O.dropkey_draws(7, x.shape) < 0.4
    drop[1, 2] = True                                   # a row that loses every key
    y = O.attention_softmax(x, False, drop)
    assert np.all(y[drop] == 0) and np.all(y[1, 2] == 0)
    for b, r in [(0, 0), (2, 5), (1, 3)]:
        keep = ~drop[b, r]
        e = np.exp(x[b, r, keep] - x[b, r, keep].max())
        assert np.allclose(y[b, r, keep], e / e.sum(), atol=1e-15)
