"""The oracle against the reference's own CPU translation units (ops/timestep_norm.cc,
ops/ema_parameters.cc, ops/ema_hidden.cc), compiled in place into oracle/_ref by
`make -C oracle ref`.  Skipped where that build does not exist."""
import numpy as np
import pytest
import torch

from conftest import mega_init_complex, rel_err
from oracle import mega_oracle as O


@pytest.mark.parametrize("G", [4, 2])
@pytest.mark.parametrize("masked", [False, True])
def test_group_timestep_norm(ref_cpu, G, masked):
    rng = np.random.default_rng(0)
    B, L, H = 3, 29, 40
    x = rng.normal(size=(B, L, H)).astype(np.float32)
    mask = (rng.random((B, L)) < 0.3) if masked else None
    pc = np.array([0, 4, 1], np.int64)
    pm = (rng.normal(size=(B, G)) * 0.2).astype(np.float32)
    pv = (rng.random((B, G)) + 0.5).astype(np.float32)
    gamma = (rng.normal(size=H) + 1).astype(np.float32); beta = rng.normal(size=H).astype(np.float32)
    out = ref_cpu.group_timestep_norm_fwd(torch.from_numpy(x), torch.from_numpy(pc), torch.from_numpy(pm),
                                          torch.from_numpy(pv), torch.from_numpy(gamma), torch.from_numpy(beta),
                                          None if mask is None else torch.from_numpy(mask), G, 1e-5)
    y, c, mu, v = O.timestep_norm(x, pc, pm, pv, gamma, beta, mask, G, 1e-5)
    assert rel_err(out[0].numpy(), y) < 2e-5
    assert np.array_equal(out[1].numpy(), c)
    assert rel_err(out[2].numpy(), mu) < 2e-5 and rel_err(out[3].numpy(), v) < 2e-5


def test_feature_timestep_norm(ref_cpu):
    rng = np.random.default_rng(1)
    B, L, H = 2, 33, 12
    x = rng.normal(size=(B, L, H)).astype(np.float32)
    mask = rng.random((B, L)) < 0.2
    pc = np.array([2, 3], np.int64)
    pm = np.zeros((B, H), np.float32); pv = np.ones((B, H), np.float32)
    gamma = (rng.normal(size=H) + 1).astype(np.float32); beta = rng.normal(size=H).astype(np.float32)
    out = ref_cpu.timestep_norm_fwd(torch.from_numpy(x), torch.from_numpy(pc), torch.from_numpy(pm),
                                    torch.from_numpy(pv), torch.from_numpy(gamma), torch.from_numpy(beta),
                                    torch.from_numpy(mask), 1e-5)
    y, c, mu, v = O.timestep_norm(x, pc, pm, pv, gamma, beta, mask, None, 1e-5)
    assert rel_err(out[0].numpy(), y) < 2e-5 and np.array_equal(out[1].numpy(), c)
    assert rel_err(out[2].numpy(), mu) < 2e-5 and rel_err(out[3].numpy(), v) < 2e-5


def test_ema_parameters_and_hidden(ref_cpu):
    rng = np.random.default_rng(2)
    K, N, L, B = 5, 16, 48, 3
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    h = rng.normal(size=(B, K, N)) + 1j * rng.normal(size=(B, K, N))
    tp = torch.from_numpy(p.astype(np.float32))
    tq = torch.from_numpy(q.astype(np.complex64))
    tg = torch.from_numpy(g.astype(np.complex64))
    th = torch.from_numpy(h.astype(np.complex64))
    w, b, _ = ref_cpu.ema_parameters_fwd(tp, tq.log(), tg, th, L)
    assert rel_err(w.numpy(), O.ema_kernel(p, q, g, L)) < 2e-5
    assert rel_err(b.numpy(), O.ema_bias(q, g, h, L)) < 2e-5
    w0, b0, _ = ref_cpu.ema_parameters_fwd(tp, tq.log(), tg, None, L)
    assert b0 is None and rel_err(w0.numpy(), O.ema_kernel(p, q, g, L)) < 2e-5
    x = rng.normal(size=(B, K, L)).astype(np.float32)
    y, _ = ref_cpu.ema_hidden_fwd(torch.from_numpy(x), tp, tq.log(), th)
    ref = O.ema_hidden(x, p, q, h)
    assert rel_err(y.numpy().real, ref.real) < 2e-5 and rel_err(y.numpy().imag, ref.imag) < 2e-5
    y0, _ = ref_cpu.ema_hidden_fwd(torch.from_numpy(x), tp, tq.log(), None)
    ref0 = O.ema_hidden(x, p, q, None)
    assert rel_err(y0.numpy().real, ref0.real) < 2e-5
