"""Committed golden vectors (tests/golden/ref_cpu_vectors.npz: outputs of the reference's own CPU
operators, written by tests/golden/make_golden.py) against the numpy oracle, the C oracle and,
on a GPU box, the HIP library.  fp32 inputs; tolerance 2e-5 for the fp64/fp32 oracles
(the vectors are fp32 results), 1e-4 for the HIP fp32 path."""
import os

import numpy as np
import pytest

from conftest import rel_err
from oracle import mega_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_cpu_vectors.npz")


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def _case(gold, tag):
    return {k[len(tag) + 1:]: gold[k] for k in gold.files if k.startswith(tag + ".")}


GROUP_CASES = ["gtsn_a", "gtsn_b", "gtsn_c"]


@pytest.mark.parametrize("tag", GROUP_CASES)
def test_oracle_group_norm(gold, tag):
    c = _case(gold, tag)
    y, n, mu, v = O.timestep_norm(c["x"], c["prev_count"], c["prev_mean"], c["prev_var"], c["gamma"], c["beta"],
                                  c.get("mask"), int(c["groups"]), 1e-5)
    assert rel_err(y, c["y"]) < 2e-5 and np.array_equal(n, c["count"])
    assert rel_err(mu, c["mean"]) < 2e-5 and rel_err(v, c["var"]) < 2e-5


def test_oracle_feature_norm(gold):
    c = _case(gold, "tsn")
    y, n, mu, v = O.timestep_norm(c["x"], c["prev_count"], c["prev_mean"], c["prev_var"], c["gamma"], c["beta"],
                                  c["mask"], None, 1e-5)
    assert rel_err(y, c["y"]) < 2e-5 and np.array_equal(n, c["count"])
    assert rel_err(mu, c["mean"]) < 2e-5 and rel_err(v, c["var"]) < 2e-5


def test_oracle_ema(gold):
    c = _case(gold, "ema")
    L = int(c["length"])
    p, q, g, h = c["p"].astype(np.float64), c["q"].astype(np.complex128), c["gamma"].astype(np.complex128), c["h"]
    assert rel_err(O.ema_kernel(p, q, g, L), c["kernel"]) < 2e-5
    assert rel_err(O.ema_bias(q, g, h, L), c["bias"]) < 2e-5
    hy = O.ema_hidden(c["x"], p, q, h)
    assert rel_err(hy.real, c["hidden"].real) < 2e-5 and rel_err(hy.imag, c["hidden"].imag) < 2e-5
    hy0 = O.ema_hidden(c["x"], p, q, None)
    assert rel_err(hy0.real, c["hidden_zero_start"].real) < 2e-5
    assert rel_err(hy0.imag, c["hidden_zero_start"].imag) < 2e-5


@pytest.mark.parametrize("tag", GROUP_CASES)
def test_oracle_c_group_norm(gold, oracle_c, tag):
    import oracle_c_api as OC

    c = _case(gold, tag)
    y, n, mu, v = OC.timestep_norm(c["x"], c["prev_count"], c["prev_mean"], c["prev_var"], c["gamma"], c["beta"],
                                   c.get("mask"), int(c["groups"]), 1e-5, np.float32)
    assert rel_err(y, c["y"]) < 2e-5 and np.array_equal(n, c["count"])
    assert rel_err(mu, c["mean"]) < 2e-5 and rel_err(v, c["var"]) < 2e-5


def test_oracle_c_kernel(gold, oracle_c):
    import oracle_c_api as OC

    c = _case(gold, "ema")
    k = OC.ema_kernel(c["p"], c["q"], c["gamma"], int(c["length"]), np.float32)
    assert rel_err(k, c["kernel"]) < 2e-5


# ----------------------------------------------------------------------------------------------
# HIP library
# ----------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("tag", GROUP_CASES)
def test_hip_group_norm(gold, tag):
    import torch

    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, tag)
    mask = None if "mask" not in c else torch.from_numpy(c["mask"]).to("cuda:0")
    y, n, mu, v = M.ops.group_timestep_norm_fwd(dev(c["x"]), dev(c["prev_count"], torch.int64), dev(c["prev_mean"]),
                                                dev(c["prev_var"]), dev(c["gamma"]), dev(c["beta"]), mask,
                                                int(c["groups"]), 1e-5)[:4]
    assert rel_err(host(y), c["y"]) < 1e-4 and np.array_equal(host(n), c["count"])
    assert rel_err(host(mu), c["mean"]) < 1e-4 and rel_err(host(v), c["var"]) < 1e-4


@pytest.mark.gpu
def test_hip_feature_norm(gold):
    import torch

    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, "tsn")
    y, n, mu, v = M.ops.timestep_norm_fwd(dev(c["x"]), dev(c["prev_count"], torch.int64), dev(c["prev_mean"]),
                                          dev(c["prev_var"]), dev(c["gamma"]), dev(c["beta"]),
                                          torch.from_numpy(c["mask"]).to("cuda:0"), 1e-5)[:4]
    assert rel_err(host(y), c["y"]) < 1e-4 and np.array_equal(host(n), c["count"])
    assert rel_err(host(mu), c["mean"]) < 1e-4 and rel_err(host(v), c["var"]) < 1e-4


@pytest.mark.gpu
def test_hip_ema(gold):
    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, "ema")
    L = int(c["length"])
    w, b, _ = M.ops.ema_parameters_fwd(dev(c["p"]), dev(c["log_q"]), dev(c["gamma"]), dev(c["h"]), L)
    assert rel_err(host(w), c["kernel"]) < 1e-4 and rel_err(host(b), c["bias"]) < 1e-4
    hy, _ = M.ops.ema_hidden_fwd(dev(c["x"]), dev(c["p"]), dev(c["log_q"]), dev(c["h"]))
    assert rel_err(host(hy).real, c["hidden"].real) < 1e-4 and rel_err(host(hy).imag, c["hidden"].imag) < 1e-4
    hy0, _ = M.ops.ema_hidden_fwd(dev(c["x"]), dev(c["p"]), dev(c["log_q"]), None)
    assert rel_err(host(hy0).real, c["hidden_zero_start"].real) < 1e-4
    assert rel_err(host(hy0).imag, c["hidden_zero_start"].imag) < 1e-4
    # the whole moving-average layer output from the same coefficients: kernel * x + bias
    omega = np.zeros(c["p"].shape[0], np.float32)
    y = M.ops.ema_forward(dev(c["x"]), dev(c["p"]), dev(c["q"]), dev(c["gamma"]), dev(omega), h=dev(c["h"]))
    y = y[0] if isinstance(y, tuple) else y
    ref = O.causal_conv_direct(c["x"].astype(np.float64), c["kernel"].astype(np.float64)) + c["bias"]
    assert rel_err(host(y), ref) < 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["gtsn_bwd_a", "gtsn_bwd_b", "tsn_bwd"])
def test_hip_timestep_norm_bwd(gold, tag):
    import torch

    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, tag)
    G = int(c["groups"])
    mask = None if "mask" not in c else torch.from_numpy(c["mask"]).to("cuda:0")
    x, pm, gamma = dev(c["x"]), dev(c["prev_mean"]), dev(c["gamma"])
    fwd_args = (x, dev(c["prev_count"], torch.int64), pm, dev(c["prev_var"]), gamma, dev(c["beta"]), mask)
    if G:
        _, cnt, _, _, gm, cm, cr = M.ops.group_timestep_norm_fwd(*fwd_args, G, 1e-5)
        got = M.ops.group_timestep_norm_bwd(dev(c["y_grad"]), dev(c["mean_grad"]), dev(c["var_grad"]), x, pm, cnt, gm,
                                            cm, cr, gamma, mask, G)
    else:
        _, cnt, _, _, cm, cr = M.ops.timestep_norm_fwd(*fwd_args, 1e-5)
        got = M.ops.timestep_norm_bwd(dev(c["y_grad"]), dev(c["mean_grad"]), dev(c["var_grad"]), x, pm, cnt, cm, cr,
                                      gamma, mask)
    for a, name in zip(got, ("x_grad", "prev_mean_grad", "prev_var_grad", "gamma_grad", "beta_grad")):
        assert rel_err(host(a), c[name]) < 1e-4, name


@pytest.mark.gpu
def test_hip_ema_backward_against_kernel_gradient_vectors(gold):
    """With x a unit impulse at t = 0 the kernel gradient sum_t dy[t] x[t - l] is dy itself, so the
    fused backward must return what the reference's ema_parameters_bwd returned for dk = dy."""
    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, "ema_bwd")
    K, L = c["kernel_grad"].shape
    x = np.zeros((1, K, L), np.float32)
    x[:, :, 0] = 1.0
    _, dp, dq, dg, _ = M.ops.ema_backward(dev(c["kernel_grad"][None]), dev(x), dev(c["p"]), dev(c["q"]),
                                          dev(c["gamma"]), dev(np.zeros(K, np.float32)))
    assert rel_err(host(dp), c["p_grad"]) < 1e-4
    for a, b in ((host(dq), c["q_grad"]), (host(dg), c["gamma_grad"])):
        assert rel_err(a.real, b.real) < 1e-4 and rel_err(a.imag, b.imag) < 1e-4


SEQ_CASES = ["gsn_a", "gsn_b", "gsn_c", "sn_a", "sn_b"]


@pytest.mark.parametrize("tag", SEQ_CASES)
def test_oracle_sequence_norm(gold, tag):
    c = _case(gold, tag)
    G = int(c["groups"]) or None
    y, n, mu, r = O.sequence_norm(c["x"], c["gamma"], c["beta"], c.get("mask"), G, 1e-5, bool(c["length_last"]))
    assert rel_err(y, c["y"]) < 2e-5 and np.array_equal(n, c["count"])
    assert rel_err(mu, c["mean"]) < 2e-5 and rel_err(r, c["rstd"]) < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("tag", SEQ_CASES)
def test_hip_sequence_norm(gold, tag):
    import torch

    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, tag)
    G = int(c["groups"])
    mask = None if "mask" not in c else torch.from_numpy(c["mask"]).to("cuda:0")
    last = bool(c["length_last"])
    if G:
        y, n, mu, r = M.ops.group_sequence_norm_fwd(dev(c["x"]), dev(c["gamma"]), dev(c["beta"]), mask, G, 1e-5, last)
    else:
        y, n, mu, r = M.ops.sequence_norm_fwd(dev(c["x"]), dev(c["gamma"]), dev(c["beta"]), mask, 1e-5, last)
    assert rel_err(host(y), c["y"]) < 1e-4 and np.array_equal(host(n), c["count"])
    assert rel_err(host(mu), c["mean"]) < 1e-4 and rel_err(host(r), c["rstd"]) < 1e-4


@pytest.mark.gpu
def test_hip_ema_parameters_bwd(gold):
    """The operator under the reference's name: kernel gradient (and bias gradient with a carried
    state) to coefficient gradients."""
    import torch

    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, "ema_bwd")
    log_q = torch.from_numpy(c["q"]).log().to("cuda:0")
    dp, dq, dg, dh = M.ops.ema_parameters_bwd(dev(c["kernel_grad"]), None, dev(c["p"]), log_q, dev(c["gamma"]), None)
    assert dh is None and rel_err(host(dp), c["p_grad"]) < 1e-4
    for a, b in ((host(dq), c["q_grad"]), (host(dg), c["gamma_grad"])):
        assert rel_err(a.real, b.real) < 1e-4 and rel_err(a.imag, b.imag) < 1e-4
    dp, dq, dg, dh = M.ops.ema_parameters_bwd(dev(c["kernel_grad"]), dev(c["bias_grad"]), dev(c["p"]), log_q,
                                              dev(c["gamma"]), dev(c["h"]))
    assert rel_err(host(dp), c["p_grad_b"]) < 1e-4
    for a, b in ((host(dq), c["q_grad_b"]), (host(dg), c["gamma_grad_b"]), (host(dh), c["h_grad_b"])):
        assert rel_err(a.real, b.real) < 1e-4 and rel_err(a.imag, b.imag) < 1e-4


@pytest.mark.gpu
def test_hip_ema_hidden_bwd(gold):
    import torch

    import fairseq_apollo_amd as M
    from gpu_util import dev, host

    c = _case(gold, "hid_bwd")
    log_q = torch.from_numpy(c["q"]).log().to("cuda:0")
    dx, dp, dq, dh = M.ops.ema_hidden_bwd(dev(c["y_grad"]), dev(c["x"]), dev(c["p"]), log_q, dev(c["h"]))
    assert rel_err(host(dx), c["x_grad"]) < 1e-4 and rel_err(host(dp), c["p_grad"]) < 1e-4
    for a, b in ((host(dq), c["q_grad"]), (host(dh), c["h_grad"])):
        assert rel_err(a.real, b.real) < 1e-4 and rel_err(a.imag, b.imag) < 1e-4
    dx0, dp0, dq0, dh0 = M.ops.ema_hidden_bwd(dev(c["y_grad"]), dev(c["x"]), dev(c["p"]), log_q, None)
    assert dh0 is None and rel_err(host(dx0), c["x_grad"]) < 1e-4 and rel_err(host(dp0), c["p_grad"]) < 1e-4
