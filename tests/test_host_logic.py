"""Host-side mirror of the reference modules: parameter names / shapes (checkpoint
compatibility), coefficient formulas against the oracle, incremental-state bookkeeping."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from oracle import mega_oracle as O


def test_parameter_names_and_shapes():
    ema = M.MultiHeadEMA(8, ndim=4, bidirectional=True)
    sd = {k: tuple(v.shape) for k, v in ema.state_dict().items()}
    assert sd == {"alpha": (16, 4, 1), "delta": (16, 4, 1), "beta": (16, 4, 1), "gamma": (16, 4), "omega": (8,)}
    cema = M.MultiHeadComplexEMA(8, ndim=4)
    sd = {k: tuple(v.shape) for k, v in cema.state_dict().items()}
    assert sd == {"alpha": (8, 4, 1), "delta": (8, 4, 1), "theta": (8, 1, 1), "gamma": (8, 4, 2), "omega": (8, 1)}
    assert [n for n, _ in cema.parameters_no_weight_decay()] == ["alpha", "delta", "theta"]
    tn = M.TimestepNorm(32, 4)
    sd = {k: tuple(v.shape) for k, v in tn.state_dict().items()}
    assert sd == {"weight": (32,), "bias": (32,), "prior_count": (), "prior_mean": (4,), "prior_logv": (4,)}
    assert len(list(tn.parameters())) == 2
    tn2 = M.TimestepNorm(32, 4, prior_count=3)
    assert len(list(tn2.parameters())) == 4
    with pytest.raises(AssertionError):
        M.TimestepNorm(32)                      # per-feature variant needs prior_count > 1
    with pytest.raises(AssertionError):
        M.MultiHeadEMA(8, truncation=4)         # truncation only with bidirectional


def test_coefficients_match_oracle_and_init_statistics():
    torch.manual_seed(0)
    cema = M.MultiHeadComplexEMA(64, ndim=16).eval()
    p, q, g = cema.coeffs()
    po, qo, go = O.ema_coeffs_complex(cema.alpha.detach().numpy(), cema.delta.detach().numpy(),
                                      cema.theta.detach().numpy(), cema.gamma.detach().numpy())
    assert np.allclose(p.squeeze(-1).numpy(), po, atol=1e-6)
    assert np.allclose(q.squeeze(-1).numpy(), qo, atol=1e-6)
    assert np.allclose(g.numpy(), go, atol=1e-6)
    assert torch.all(cema.gamma[..., 1] == 0)
    assert cema.coeffs() is cema.coeffs()       # cached in eval mode
    cema.train()
    assert cema._coeffs is None
    ema = M.MultiHeadEMA(64, ndim=16).eval()
    p, q, g = ema.coeffs()
    po, qo, go = O.ema_coeffs_real(ema.alpha.detach().numpy(), ema.delta.detach().numpy(),
                                   ema.beta.detach().numpy(), ema.gamma.detach().numpy())
    assert np.allclose(p.squeeze(-1).numpy(), po, atol=1e-6) and np.allclose(q.squeeze(-1).numpy(), qo, atol=1e-6)
    b = ema.beta.detach().squeeze(-1)
    assert torch.all(b[:, 0::2] > 0.8) and torch.all(b[:, 1::2] < -0.8)


def test_incremental_state_keys_are_per_module():
    a, b = M.TimestepNorm(8, 2), M.TimestepNorm(8, 2)
    state = {}
    a.set_incremental_state(state, "norm_state", {"prev_count": 1})
    assert a.get_incremental_state(state, "norm_state") == {"prev_count": 1}
    assert b.get_incremental_state(state, "norm_state") is None
    key, = state.keys()
    assert key.endswith(".norm_state")
    e = M.MultiHeadComplexEMA(4, ndim=2)
    inc = {}
    e._set_input_buffer(inc, {"prev_state": torch.arange(6.).reshape(3, 2)})
    e.reorder_incremental_state(inc, torch.tensor([2, 0]))
    assert torch.equal(e._get_input_buffer(inc)["prev_state"], torch.tensor([[4., 5.], [0., 1.]]))


def test_configurations_without_a_backward_refuse_autograd():
    """The moving average (with a truncated kernel or a carried state through the chained operators),
    TimestepNorm and the attention have backward operators; what has none says so instead of returning tensors
    that silently carry no graph.  None of them has a CPU path: host tensors are refused by name."""
    e = M.MultiHeadComplexEMA(4, ndim=2, bidirectional=True, truncation=4)
    with pytest.raises(RuntimeError, match="no CPU path"):
        e(torch.zeros(1, 4, 8))
    layer = M.MovingAverageGatedAttention(8, 4, 8, 2, chunk_size=4, norm_num_groups=2)
    with pytest.raises(NotImplementedError, match="incremental state"):
        layer(torch.zeros(1, 4, 8), None, {})


def test_gated_attention_state_dict_matches_reference_names():
    """Parameter / buffer names and shapes a reference checkpoint of the layer holds
    (moving_average_gated_attention.py:84-113; complex_exponential_moving_average.py:31-36;
    norm_layer/timestep_norm.py:91-101; norm_layer/layer_norm.py:41-49; relative_positional_bias.py:55),
    so load_state_dict takes a reference state dict as is."""
    D, S, E, N, G = 16, 8, 24, 4, 4
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=8, moving_layer='cema', moving_act='rmsnorm',
                                          norm_num_groups=G)
    want = {
        "norm.prior_count": (), "norm.prior_mean": (G,), "norm.prior_logv": (G,), "norm.weight": (D,), "norm.bias": (D,),
        "move.alpha": (D, N, 1), "move.delta": (D, N, 1), "move.theta": (D, 1, 1), "move.gamma": (D, N, 2),
        "move.omega": (D, 1),
        "move_act.weight": (D,),
        "v_proj.weight": (E, D), "v_proj.bias": (E,),
        "mx_proj.weight": (S + E + 2 * D, D), "mx_proj.bias": (S + E + 2 * D,),
        "h_proj.weight": (D, E),
        "gamma": (2, S), "beta": (2, S),
        "rel_pos_bias.freqs": (S // 2,),
    }
    got = {k: tuple(v.shape) for k, v in layer.state_dict().items()}
    assert got == want
    ffn = M.NormalizedFeedForwardNetwork(D, 32, norm_type='rmsnorm')
    assert set(ffn.state_dict()) == {"norm.weight", "fc1.weight", "fc1.bias", "fc2.weight"}


def test_layer_constructor_follows_the_reference():
    """init_mode (moving_average_gated_attention.py:128-145) and the attention activations are checked at
    construction."""
    kw = dict(chunk_size=4, norm_num_groups=2)
    for mode in ('bert', 'he', 'xavier'):
        layer = M.MovingAverageGatedAttention(8, 4, 8, 2, init_mode=mode, **kw)
        assert layer.init_mode == mode and torch.all(layer.gamma == 0) and torch.all(layer.v_proj.bias == 0)
    with pytest.raises(ValueError, match="init mode"):
        M.MovingAverageGatedAttention(8, 4, 8, 2, init_mode='orthogonal', **kw)
    with pytest.raises(ValueError, match="attention activation"):
        M.MovingAverageGatedAttention(8, 4, 8, 2, attention_activation='gelu', **kw)
    assert 'chunk=4' in repr(M.MovingAverageGatedAttention(8, 4, 8, 2, **kw))


def test_eval_caches_follow_the_parameters():
    """Weights loaded (or edited in place) after a first eval-mode use: the cached coefficients, weight + 1 /
    bias and the prior state are recomputed, as the reference computes them on every call
    (timestep_norm.py:118-131) or from the parameters it was given (base_moving_average.py:52-58)."""
    import copy

    torch.manual_seed(3)
    ema = M.MultiHeadComplexEMA(8, ndim=4).eval()
    p0, q0, g0 = [t.clone() for t in ema.coeffs()]
    assert ema.coeffs()[0] is ema.coeffs()[0]                    # cached while nothing changes
    other = M.MultiHeadComplexEMA(8, ndim=4)
    ema.load_state_dict(copy.deepcopy(other.state_dict()))
    p1, q1, g1 = ema.coeffs()
    po, qo, go = other.eval().coeffs()
    assert torch.equal(p1, po) and torch.equal(q1, qo) and torch.equal(g1, go)
    assert not torch.equal(p1, p0)
    with torch.no_grad():
        ema.alpha.add_(0.5)
    assert not torch.equal(ema.coeffs()[0], p1)

    norm = M.TimestepNorm(16, 4, prior_count=2).eval()
    g_a, b_a = norm._affine()
    c_a, m_a, v_a = norm._prior_state(3)
    assert norm._affine()[0] is g_a and norm._prior_state(3)[1] is m_a
    sd = copy.deepcopy(norm.state_dict())
    sd["weight"] = torch.randn(16)
    sd["bias"] = torch.randn(16)
    sd["prior_mean"] = torch.randn(4)
    sd["prior_logv"] = torch.randn(4)
    norm.load_state_dict(sd)
    g_b, b_b = norm._affine()
    c_b, m_b, v_b = norm._prior_state(3)
    assert torch.equal(g_b, sd["weight"] + 1.0) and torch.equal(b_b, sd["bias"])
    assert torch.equal(m_b, sd["prior_mean"].expand(3, -1)) and torch.allclose(v_b, sd["prior_logv"].exp().expand(3, -1))


def test_bench_measures_one_gpu_only():
    """bench.py --gpus N with N > 1 exits with a message instead of starting ranks."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_split_keeps_its_gradient_buffer_or_concatenates():
    """SplitFunc / SplitGrads (the backward of the split of the mx_proj output): when every slice's gradient is the
    slot the buffer handed out, the buffer itself comes back (no copy); any other mix -- a slice nobody used, a
    gradient made elsewhere -- is concatenated, and the result equals torch.split's in both cases."""
    import torch

    from fairseq_apollo_amd.modules import SplitFunc, SplitGrads

    class IntoSlot(torch.autograd.Function):
        """y = 2 x whose backward writes into the slot it is given."""

        @staticmethod
        def forward(ctx, x, slot):
            ctx.slot = slot
            return 2 * x

        @staticmethod
        def backward(ctx, g):
            out = ctx.slot[0].slot(ctx.slot[1])
            out.copy_(2 * g)
            return out, None

    torch.manual_seed(0)
    widths = [3, 5, 4]
    base0 = torch.randn(2, 6, sum(widths))
    w = [torch.randn(2, 6, k) for k in widths]

    def reference(used):
        b = base0.clone().requires_grad_(True)
        parts = torch.split(b, widths, dim=-1)
        sum((2 * parts[i] * w[i]).sum() for i in used).backward()
        return b.grad

    # every slice through a consumer that writes its slot: the buffer comes back as it is
    b = base0.clone().requires_grad_(True)
    arena = SplitGrads(b, widths)
    parts = SplitFunc.apply(b, arena)
    before = SplitGrads.taken
    sum((IntoSlot.apply(parts[i], (arena, i)) * w[i]).sum() for i in range(3)).backward()
    assert SplitGrads.taken == before + 1 and arena.buf is None
    assert torch.equal(b.grad, reference(range(3)))
    # one slice unused, one gradient made by torch: concatenation, same values
    b = base0.clone().requires_grad_(True)
    arena = SplitGrads(b, widths)
    parts = SplitFunc.apply(b, arena)
    before = SplitGrads.taken
    ((IntoSlot.apply(parts[0], (arena, 0)) * w[0]).sum() + (2 * parts[2] * w[2]).sum()).backward()
    assert SplitGrads.taken == before and arena.buf is None
    assert torch.equal(b.grad, reference([0, 2]))
    # a second backward pass through a retained graph gets a buffer of its own
    b = base0.clone().requires_grad_(True)
    arena = SplitGrads(b, widths)
    parts = SplitFunc.apply(b, arena)
    loss = sum((IntoSlot.apply(parts[i], (arena, i)) * w[i]).sum() for i in range(3))
    loss.backward(retain_graph=True)
    first = b.grad.clone()
    loss.backward()
    assert torch.equal(b.grad, 2 * first)
