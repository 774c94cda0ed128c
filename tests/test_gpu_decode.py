"""Recurrent decode path: single-step EMA state update plus streaming TimestepNorm, checked against
the parallel path on the concatenated sequence (both HIP) and against the fp64 oracle."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex, rel_err
from gpu_util import DEV, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu


def _setup(B, D, N, G, seed):
    rng = np.random.default_rng(seed)
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    om = rng.normal(size=D)
    nw = rng.normal(size=D) * 0.1
    nb = rng.normal(size=D) * 0.1
    return rng, p, q, g, om, nw, nb


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 2e-2)])
def test_small_streams_against_oracle(dtype, tol):
    B, D, N, G, T = 3, 96, 16, 4, 200
    rng, p, q, g, om, nw, nb = _setup(B, D, N, G, 41)
    x, x64 = rounded(rng.normal(size=(B, T, D)), dtype)
    step = M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
    xs, ys = [], []
    for t in range(T):
        xn, y = step(x[:, t])
        xs.append(xn); ys.append(y)
    xn_s, y_s = torch.stack(xs, 1), torch.stack(ys, 1)
    torch.cuda.synchronize()
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, None, G)
    assert rel_err(host(xn_s), xno) < max(tol, 1e-4)
    yo, ho = O.ema_forward(host(xn_s).transpose(0, 2, 1), p, q, g, om, incremental=True)
    assert rel_err(host(y_s), yo.transpose(0, 2, 1)) < max(tol, 1e-4)
    assert step.count.tolist() == [T] * B
    assert rel_err(host(step.mean), mu) < 1e-4 and rel_err(host(step.var), v) < 1e-4
    assert rel_err(np.real(host(step.state)), np.real(ho)) < 1e-4
    # the same tokens through the parallel kernels
    norm = M.TimestepNorm(D, G).to(DEV).eval()
    with torch.no_grad():
        norm.weight.copy_(dev(nw)); norm.bias.copy_(dev(nb))
        xn_p = norm(x)
        y_p, h_p = M.ops.ema_forward(xn_p.transpose(1, 2), dev(p), dev(q), dev(g), dev(om), want_state=True)
    assert rel_err(host(xn_s), host(xn_p)) < tol
    assert rel_err(host(y_s), host(y_p.transpose(1, 2))) < tol


def test_config3_b64_d2048_2048_steps():
    """B = 64 streams, D = 2048, N = 16, complex q, 2048 consecutive steps, fp32: the recurrent
    path agrees with the parallel path on the concatenated sequence to 1e-5; four streams are also
    checked against the fp64 oracle."""
    B, D, N, G, T = 64, 2048, 16, 16, 2048
    rng, p, q, g, om, nw, nb = _setup(B, D, N, G, 1237)
    gen = torch.Generator().manual_seed(1237)
    x = torch.randn(B, T, D, generator=gen).to(DEV)
    step = M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
    xn_s = torch.empty_like(x)
    y_s = torch.empty_like(x)
    for t in range(T):
        xn_s[:, t], y_s[:, t] = step(x[:, t])
    norm = M.TimestepNorm(D, G).to(DEV).eval()
    with torch.no_grad():
        norm.weight.copy_(dev(nw)); norm.bias.copy_(dev(nb))
        state = {}
        xn_p = norm(x, None, state)
        y_p, h_p = M.ops.ema_forward(xn_p.transpose(1, 2), dev(p), dev(q), dev(g), dev(om), want_state=True)
    torch.cuda.synchronize()
    assert M.ops.timestep_norm_status() == 0
    def rel(a, b):       # max |a - b| / max(|b|, rms(b)), evaluated on the device
        rms = b.abs().pow(2).mean().sqrt()
        return ((a - b).abs() / torch.clamp(b.abs(), min=rms)).max().item()

    e1 = rel(xn_s, xn_p)
    e2 = rel(y_s, y_p.transpose(1, 2))
    e3 = rel(step.state, h_p)
    print(f"recurrent vs parallel: norm {e1:.2e}, ema {e2:.2e}, state {e3:.2e}", flush=True)
    assert e1 < 1e-5 and e2 < 1e-5 and e3 < 1e-5
    saved = norm._get_input_buffer(state)
    assert torch.equal(saved["prev_count"], step.count)
    # the carried statistics, relative to their rms: one step folded with the weight of the next
    # step's count (1 / (c + 2) instead of 1 / (c + 1)) would show here
    for a, b_ in ((step.mean, saved["prev_mean"]), (step.var, saved["prev_var"])):
        assert ((a - b_).abs().max() / b_.pow(2).mean().sqrt()).item() < 1e-5
    sel = [0, 17, 40, 63]
    x64 = x[sel].double().cpu().numpy()
    xno, c_o, mu_o, v_o = O.timestep_norm(x64, np.zeros(4, np.int64), np.zeros((4, G)), np.ones((4, G)), nw + 1, nb, None, G)
    assert rel_err(host(xn_s[sel]), xno) < 1e-4
    assert step.count[sel].tolist() == c_o.tolist() == [T] * 4
    assert rel_err(host(step.mean[sel]), mu_o) < 1e-5 and rel_err(host(step.var[sel]), v_o) < 1e-5
    yo, _ = O.ema_forward(xno.transpose(0, 2, 1), p, q, g, om)
    assert rel_err(host(y_s[sel]), yo.transpose(0, 2, 1)) < 1e-4


def test_config3_bf16_full_width():
    """configs[3] in its own arithmetic: 64 streams, D = 2048, N = 16, bf16 activations, 512 consecutive single-token
    steps and then the same tokens as launches of 64; a sample of streams against the fp64 oracle (the norm on the
    bf16 inputs, the moving average on the bf16 xn the step produced, as a layer behind it would see it), every stream
    against the parallel path in bf16."""
    B, D, N, G, T = 64, 2048, 16, 16, 512
    rng, p, q, g, om, nw, nb = _setup(B, D, N, G, 1241)
    gen = torch.Generator().manual_seed(1241)
    x = torch.randn(B, T, D, generator=gen).to(torch.bfloat16).to(DEV)
    step = M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
    xn_s = torch.empty_like(x)
    y_s = torch.empty_like(x)
    for t in range(T):
        xn_s[:, t], y_s[:, t] = step(x[:, t])
    torch.cuda.synchronize()
    sel = [0, 21, 42, 63]
    x64 = x[sel].double().cpu().numpy()
    xno, c_o, mu_o, v_o = O.timestep_norm(x64, np.zeros(4, np.int64), np.zeros((4, G)), np.ones((4, G)), nw + 1, nb, None, G)
    assert rel_err(host(xn_s[sel]), xno) < 2e-2
    assert step.count[sel].tolist() == c_o.tolist() == [T] * 4
    assert rel_err(host(step.mean[sel]), mu_o) < 1e-4 and rel_err(host(step.var[sel]), v_o) < 1e-4
    yo, ho = O.ema_forward(host(xn_s[sel]).transpose(0, 2, 1), p, q, g, om, incremental=True)
    assert rel_err(host(y_s[sel]), yo.transpose(0, 2, 1)) < 2e-2
    assert rel_err(np.real(host(step.state[sel])), np.real(ho)) < 2e-3
    # the parallel path on the whole batch
    norm = M.TimestepNorm(D, G).to(DEV).eval()
    with torch.no_grad():
        norm.weight.copy_(dev(nw)); norm.bias.copy_(dev(nb))
        xn_p = norm(x, None, {})
        # the moving average on the xn the steps produced: both paths then see the same bf16 inputs
        y_p, _ = M.ops.ema_forward(xn_s.transpose(1, 2), dev(p), dev(q), dev(g), dev(om))
    torch.cuda.synchronize()
    # two bf16 paths against each other (each is held to 2e-2 of the fp64 result above): 3e-2
    assert rel_err(host(xn_s), host(xn_p)) < 2e-2 and rel_err(host(y_s), host(y_p.transpose(1, 2))) < 3e-2
    # the same tokens, 64 per launch
    step2 = M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
    outs = [step2.steps(x[:, a:a + 64]) for a in range(0, T, 64)]
    torch.cuda.synchronize()
    assert M.ops.timestep_norm_status() == 0
    assert rel_err(host(torch.cat([o[0] for o in outs], 1)), host(xn_s)) < 2e-2
    assert rel_err(host(torch.cat([o[1] for o in outs], 1)), host(y_s)) < 2e-2


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("B,D,N,G,chunks", [(3, 96, 16, 4, (1, 7, 64, 65, 130)), (2, 256, 8, 2, (16, 16)),
                                            (5, 64, 4, 1, (3, 200))])
def test_multi_token_launch_equals_single_steps(dtype, tol, B, D, N, G, chunks):
    """K tokens per launch (mega_norm_ema_steps) against the same tokens one launch each, chunk after chunk with the
    state carried (chunks shorter, equal to and longer than the kernel's batch of 64 tokens), and against the fp64
    oracle on the whole sequence."""
    rng, p, q, g, om, nw, nb = _setup(B, D, N, G, 43)
    T = sum(chunks)
    x, x64 = rounded(rng.normal(size=(B, T, D)) + 0.2, dtype)
    mk = lambda: M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
    one, many = mk(), mk()
    xs, ys = [], []
    for t in range(T):
        xn, y = one(x[:, t])
        xs.append(xn); ys.append(y)
    xn_1, y_1 = torch.stack(xs, 1), torch.stack(ys, 1)
    xk, yk, a = [], [], 0
    for K in chunks:
        print(f"case B={B} D={D} N={N} G={G} chunk K={K} at {a}", flush=True)
        xn, y = many.steps(x[:, a:a + K])
        assert xn.shape == y.shape == (B, K, D)
        xk.append(xn); yk.append(y)
        a += K
    xn_k, y_k = torch.cat(xk, 1), torch.cat(yk, 1)
    torch.cuda.synchronize()
    assert many.count.tolist() == one.count.tolist() == [T] * B
    assert rel_err(host(many.mean), host(one.mean)) < 1e-5 and rel_err(host(many.var), host(one.var)) < 1e-5
    assert rel_err(host(xn_k), host(xn_1)) < (1e-5 if dtype is torch.float32 else 1e-2)
    assert rel_err(host(y_k), host(y_1)) < tol
    assert rel_err(np.real(host(many.state)), np.real(host(one.state))) < 1e-4
    assert rel_err(np.imag(host(many.state)), np.imag(host(one.state))) < 1e-4
    xno, c, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)), nw + 1, nb, None, G)
    assert rel_err(host(xn_k), xno) < max(tol, 1e-4)
    yo, ho = O.ema_forward(host(xn_k).transpose(0, 2, 1), p, q, g, om, incremental=True)
    assert rel_err(host(y_k), yo.transpose(0, 2, 1)) < max(tol, 1e-4)
    assert rel_err(np.real(host(many.state)), np.real(ho)) < 1e-4


def test_multi_token_launch_other_coefficient_shapes_take_single_steps():
    """ndim = 6 is outside the multi-token kernel: the C entry point says so, DecodeStep.steps runs K single steps."""
    B, D, N, G, K = 2, 64, 6, 2, 5
    rng, p, q, g, om, nw, nb = _setup(B, D, N, G, 44)
    x, _ = rounded(rng.normal(size=(B, K, D)), torch.float32)
    a = M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
    b = M.ops.DecodeStep(dev(nw), dev(nb), G, 1e-5, dev(p), dev(q), dev(g), dev(om), B)
    xn_a, y_a = a.steps(x)
    outs = [b(x[:, k]) for k in range(K)]
    torch.cuda.synchronize()
    assert torch.equal(y_a, torch.stack([o[1] for o in outs], 1)) and torch.equal(a.h, b.h)
    lib = M._lib.load()
    ptr = lambda t: t.data_ptr()
    rc = lib.mega_norm_ema_steps(ptr(x), ptr(xn_a), ptr(y_a), 0, K, ptr(a.count), ptr(a.mean), ptr(a.var),
                                 ptr(a._count_next), ptr(a.mean), ptr(a.var), ptr(a.nw), ptr(a.nb), 1e-5, ptr(a.p), ptr(a.q),
                                 ptr(a.gamma), 1, ptr(a.omega), ptr(a.h), ptr(a.h), B, D, G, N, None)
    assert rc == -2 and b"ndim" in lib.mega_last_error()
