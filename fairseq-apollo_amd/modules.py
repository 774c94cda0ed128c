"""Module surface: drop-in counterparts of the reference's PyTorch modules for the
Mega/Mega2 sequence-mixing path, with the same constructor arguments, parameter names and
shapes (so reference checkpoints load) and the same incremental-state keys.

    MultiHeadEMA            fairseq/modules/exponential_moving_average.py:13-94
    MultiHeadComplexEMA     fairseq/modules/complex_exponential_moving_average.py:15-113
    (both on)  BaseMovingLayer  fairseq/modules/base_moving_average.py:18-197
    TimestepNorm            fairseq/modules/norm_layer/timestep_norm.py:71-167
    AttentionSoftmax        fairseq/modules/attention_softmax.py:44-56
    EfficientAttention      fairseq/modules/efficient_attention.py:45-63
    SwiGLU                  no counterpart in the reference (its FFN is
                            fairseq/modules/normalized_feedforward_network.py:77-93)

Every module works under autograd through the library's backward kernels (the autograd functions below);
what has no backward (incremental state under a graph) raises instead of silently detaching.
"""
from __future__ import annotations

import math
import uuid
from collections import OrderedDict
from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn
from torch.nn.parameter import Parameter

from . import ops


class IncrementalState(object):
    """Per-module namespacing of the shared incremental_state dict
    (fairseq/incremental_decoding_utils.py:12-50)."""

    def init_incremental_state(self):
        self._incremental_state_id = str(uuid.uuid4())

    def _get_full_incremental_state_key(self, key: str) -> str:
        return "{}.{}".format(self._incremental_state_id, key)

    def get_incremental_state(self, incremental_state, key: str):
        full_key = self._get_full_incremental_state_key(key)
        if incremental_state is None or full_key not in incremental_state:
            return None
        return incremental_state[full_key]

    def set_incremental_state(self, incremental_state, key: str, value):
        if incremental_state is not None:
            incremental_state[self._get_full_incremental_state_key(key)] = value
        return incremental_state


class MovingAverageFunc(torch.autograd.Function):
    """The whole moving-average layer (one- or two-sided) as one differentiable operator: the
    reference chains EMAParametersFunc (fused_ops/ema_parameters.py:11-33) and FFTConvFunc
    (fused_ops/fftconv.py:13-41) plus the residual; here neither the kernel nor its gradient is
    materialised.  Inputs (x [B, D, L], p, q, gamma, omega) as BaseMovingLayer holds them."""

    @staticmethod
    def forward(ctx, x, p, q, gamma, omega, padding_mask, out_layout, bidirectional=False, shift=True):
        layer = ops.PreparedEMA(p.squeeze(-1), q.squeeze(-1), gamma, omega.reshape(-1), bidirectional, None, shift)
        y, _ = layer(x, padding_mask, None, want_state=False, out_layout=out_layout)
        ctx.layer = layer
        ctx.save_for_backward(x, p, q, gamma, omega, padding_mask)
        return y

    @staticmethod
    def backward(ctx, y_grad):
        x, p, q, gamma, omega, padding_mask = ctx.saved_tensors
        dx, dp, dq, dg, dom = ops.ema_backward(y_grad, x, p.squeeze(-1), q.squeeze(-1), gamma, omega.reshape(-1),
                                               padding_mask, layer=ctx.layer)
        return (dx, dp.to(p.dtype).view_as(p), dq.to(q.dtype).view_as(q), dg.to(gamma.dtype).view_as(gamma),
                dom.to(omega.dtype).view_as(omega), None, None, None, None)


def _training_call(module: nn.Module, *tensors) -> bool:
    """True when the call must build an autograd graph."""
    return torch.is_grad_enabled() and (any(t is not None and t.requires_grad for t in tensors)
                                        or any(p.requires_grad for p in module.parameters()))


def _tensor_versions(*modules: nn.Module) -> tuple:
    """Storage address and in-place version of the modules' own parameters and buffers.  An eval-mode cache
    derived from them is stale once this tuple changes: load_state_dict copies into the parameters, an
    optimiser step or an in-place edit under no_grad bumps the version, `.to()` moves the storage.  (The
    reference recomputes weight + 1, the prior state and the q / k affine on every call,
    timestep_norm.py:118-131, and caches only the moving-average coefficients in eval mode,
    base_moving_average.py:52-58.)

    Limit: an edit through `param.data` (`p.data.copy_(...)`, `p.data.mul_(...)`, as some weight-averaging
    utilities do) changes neither the address nor the version counter of `p`, so it is not seen here; after such an
    edit call `module.train(); module.eval()` (every mode switch drops the caches) or edit under `torch.no_grad()`
    through the parameter itself."""
    return tuple((t.data_ptr(), t._version) for m in modules
                 for t in (*m._parameters.values(), *m._buffers.values()) if t is not None)


class EMACoeffsFunc(torch.autograd.Function):
    """(p, q, gamma, omega) of a moving-average layer from its stored parameters, one launch forwards and one
    backwards (the chain of torch operations of complex_exponential_moving_average.py:79-96 and
    exponential_moving_average.py:71-80, which `_calc_coeffs_torch` of the two classes keeps): parameters are read
    in their storage type, results are fp32 in the library's layout, parameter gradients come back in the
    storage type."""

    @staticmethod
    def forward(ctx, alpha, delta, third, gamma, omega, is_complex):
        p, q2, g2, om = ops.ema_coeffs_fwd(alpha, delta, third, gamma, omega, is_complex)
        ctx.save_for_backward(alpha, delta, third)
        ctx.is_complex = is_complex
        ctx.like = (gamma.shape, omega.shape)
        if is_complex:
            return p.unsqueeze(-1), torch.view_as_complex(q2).unsqueeze(-1), torch.view_as_complex(g2), om.view(omega.shape)
        return p.unsqueeze(-1), q2[..., 0].unsqueeze(-1), g2[..., 0], om.view(omega.shape)

    @staticmethod
    def backward(ctx, p_grad, q_grad, g_grad, om_grad):
        alpha, delta, third = ctx.saved_tensors
        if ctx.is_complex:
            q_grad = torch.view_as_real(q_grad.resolve_conj().contiguous())
            g_grad = torch.view_as_real(g_grad.resolve_conj().contiguous())
        gl = torch.empty(ctx.like[0], dtype=alpha.dtype, device="meta")
        ol = torch.empty(ctx.like[1], dtype=alpha.dtype, device="meta")
        da, dd, dt, dg, dom = ops.ema_coeffs_bwd(p_grad, q_grad, g_grad, om_grad, alpha, delta, third, gl, ol,
                                                 ctx.is_complex)
        return da, dd, dt, dg, dom, None


def _one_cuda_dtype(*ts) -> bool:
    return all(t.is_cuda for t in ts) and len({t.dtype for t in ts}) == 1 and \
        ts[0].dtype in (torch.float32, torch.bfloat16, torch.float16)


class NormParamsFunc(torch.autograd.Function):
    """(weight + 1, bias, prior mean and exp(prior log-variance) over the batch) in fp32 from TimestepNorm's
    parameters, one launch each way (timestep_norm.py:118-131)."""

    @staticmethod
    def forward(ctx, weight, bias, prior_mean, prior_logv, batch_size):
        ctx.save_for_backward(weight, prior_mean, prior_logv)
        ctx.batch_size = batch_size
        ctx.prior_needs_grad = prior_mean.requires_grad or prior_logv.requires_grad
        return ops.norm_params_fwd(weight, bias, prior_mean, prior_logv, batch_size)

    @staticmethod
    def backward(ctx, gamma_grad, beta_grad, mean_grad, var_grad):
        weight, prior_mean, prior_logv = ctx.saved_tensors
        dw, db, dpm, dpl = ops.norm_params_bwd(gamma_grad, beta_grad, mean_grad, var_grad, weight, prior_mean,
                                               prior_logv, ctx.batch_size, ctx.prior_needs_grad)
        return dw, db, dpm, dpl, None


class BaseMovingLayer(nn.Module, IncrementalState):
    """fairseq/modules/base_moving_average.py:18-197."""

    def __init__(self, bidirectional=False, truncation=None, shift=True):
        super().__init__()
        self.init_incremental_state()
        self._parameters_no_weight_decay = OrderedDict()
        self.complex = False
        self.bidirectional = bidirectional
        self.truncation = truncation
        self.shift = shift
        self._coeffs = None
        self._prepared = None
        self._cache_key = None
        assert self.bidirectional or (self.truncation is None or self.truncation < 1), \
            'one directional moving average should not have positive trunction: {}'.format(truncation)

    def register_parameters_no_weight_decay(self, name, param):
        self._parameters_no_weight_decay[name] = param

    def parameters_no_weight_decay(self):
        for name, param in self._parameters_no_weight_decay.items():
            yield name, param

    def _calc_coeffs(self):
        raise NotImplementedError

    def coeffs(self):
        """(p, q, gamma); cached in eval mode like the reference (base_moving_average.py:52-58)."""
        with torch.no_grad():           # forward only: coefficients never carry a graph
            if self.training:
                return self._calc_coeffs()
            self._drop_stale_cache()
            if self._coeffs is None:
                self._coeffs = self._calc_coeffs()
            return self._coeffs

    def _drop_stale_cache(self):
        """The eval-mode caches follow the parameters they were computed from."""
        key = _tensor_versions(self)
        if key != self._cache_key:
            self._coeffs = None
            self._prepared = None
            self._cache_key = key

    def train(self, mode: bool = True):
        self._coeffs = None
        self._prepared = None
        return super().train(mode)

    def _apply(self, fn, *args, **kwargs):
        # .to() / .cuda() / .half(): cached coefficients would stay on the old device
        self._coeffs = None
        self._prepared = None
        return super()._apply(fn, *args, **kwargs)

    def kernel(self, length: int, hx: Optional[Tensor] = None):
        """(k[K, Lk], bias[B, K, L] or None) -- the materialised convolution kernel; the forward
        pass does not use it (base_moving_average.py:60-62)."""
        kernel_size = length if self.truncation is None or self.truncation < 1 else min(self.truncation, length)
        p, q, gamma = self.coeffs()
        w, b, _ = ops.ema_parameters_fwd(p.squeeze(-1), torch.log(q.squeeze(-1).to(torch.complex64)),
                                         gamma.to(torch.complex64), hx, kernel_size)
        return w, b

    def one_step(self, x, hx=None):
        """x: [B, D, 1] -> (out [B, D, 1] without the residual, h [B, D, N])
        (base_moving_average.py:105-118)."""
        p, q, gamma = self.coeffs()
        zero = torch.zeros_like(self.omega.reshape(-1))
        y, h = ops.ema_step(x.squeeze(-1), p.squeeze(-1), q.squeeze(-1), gamma, zero, hx)
        return y.unsqueeze(-1), h

    def forward(self, x, padding_mask: Optional[Tensor] = None,
                incremental_state: Optional[Dict[str, Dict[str, Optional[Tensor]]]] = None,
                out_layout: str = "rows") -> Tensor:
        """x: [B, D, L]; padding_mask: [B, L] with 1 / True at padding; returns [B, D, L]: contiguous
        rows (what the reference returns) or, with out_layout="input", in x's own strides (a caller
        that hands over a transposed [B, L, D] view and transposes back gets a contiguous result)."""
        bsz, embed_dim, seq_len = x.size()
        assert embed_dim == self.embed_dim
        assert not self.bidirectional or incremental_state is None, \
            'Bidirectional EMA does not support incremental state'
        if torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters())):
            if incremental_state is not None or (self.truncation is not None and self.truncation >= 1):
                return self._chained_forward(x, padding_mask, incremental_state, out_layout)
            p, q, gamma, omega = self._calc_all()       # stays in the graph
            return MovingAverageFunc.apply(x, p, q, gamma, omega, padding_mask, out_layout, self.bidirectional,
                                           self.shift)
        layer = self._prepared_layer()
        if incremental_state is not None:
            saved_state = self._get_input_buffer(incremental_state)
            h = saved_state['prev_state'] if 'prev_state' in saved_state else None
            out, h = layer(x, padding_mask, h, want_state=True, out_layout=out_layout)
            saved_state['prev_state'] = h
            self._set_input_buffer(incremental_state, saved_state)
        else:
            out, _ = layer(x, padding_mask, None, want_state=False, out_layout=out_layout)
        return out

    def _chained_forward(self, x, padding_mask, incremental_state, out_layout):
        """Training with a carried state or a truncated kernel: the reference's own chain of differentiable
        operators (base_moving_average.py:139-171): kernel and state bias from ema_parameters, the explicit
        convolution, ema_hidden for the next state.  The kernel [K, L] is materialised here; the one-operator
        path of the common case (no state, no truncation) never forms it."""
        bsz, embed_dim, seq_len = x.size()
        p, q, gamma = self._calc_coeffs()
        p, q = p.squeeze(-1), q.squeeze(-1)
        residual = x * self.omega.reshape(1, -1, 1).to(x.dtype)
        xm = x if padding_mask is None else x * (1.0 - padding_mask.unsqueeze(1).to(x.dtype))
        if incremental_state is not None:
            saved_state = self._get_input_buffer(incremental_state)
            h = saved_state['prev_state'] if 'prev_state' in saved_state else None
            k, b = ops.ema_parameters(p, q, gamma, h, seq_len)
            out = ops.fftconv(xm, k)
            if b is not None:
                out = out + b.to(out.dtype)
            saved_state['prev_state'] = ops.ema_hidden(xm, p, q, h)
            self._set_input_buffer(incremental_state, saved_state)
        else:
            kernel_size = min(self.truncation, seq_len)
            k, _ = ops.ema_parameters(p, q, gamma, None, kernel_size)
            out = ops.bidirectional_fftconv(xm, k, self.shift) if self.bidirectional else ops.fftconv(xm, k)
        out = out + residual
        if out_layout == "input" and out.stride() != x.stride():
            y = torch.empty_like(x)                     # keeps x's strides
            y.copy_(out)
            return y
        return out

    def _prepared_layer(self) -> "ops.PreparedEMA":
        """Coefficients in the library's layout; kept while the eval-mode coefficient cache lives."""
        if not self.training:
            self._drop_stale_cache()
            if self._prepared is not None and self._coeffs is not None:
                return self._prepared
        p, q, gamma = self.coeffs()
        layer = ops.PreparedEMA(p.squeeze(-1), q.squeeze(-1), gamma, self.omega.reshape(-1), self.bidirectional,
                                self.truncation, self.shift)
        self._prepared = None if self.training else layer
        return layer

    def _get_input_buffer(self, incremental_state):
        result = self.get_incremental_state(incremental_state, "ema_state")
        return result if result is not None else {}

    def _set_input_buffer(self, incremental_state, buffer):
        return self.set_incremental_state(incremental_state, "ema_state", buffer)

    def reorder_incremental_state(self, incremental_state, new_order: Tensor):
        """Reorder the carried state for beam search (base_moving_average.py:185-197)."""
        input_buffer = self._get_input_buffer(incremental_state)
        if input_buffer is not None:
            for k in input_buffer.keys():
                if input_buffer[k] is not None:
                    input_buffer[k] = input_buffer[k].index_select(0, new_order)
            incremental_state = self._set_input_buffer(incremental_state, input_buffer)
        return incremental_state

    def extra_repr(self) -> str:
        return 'edim={}, ndim={}, bidirectional={}, trunction={}, shift={}'.format(
            self.embed_dim, self.ndim, self.bidirectional, self.truncation, self.shift)


class MultiHeadEMA(BaseMovingLayer):
    """Real-valued multi-dimensional damped EMA
    (fairseq/modules/exponential_moving_average.py:13-94).  The reference class is out of
    step with its base class in this snapshot; this one implements the formulas it states
    (q = 1 - s(alpha) s(delta), p = s(alpha) beta, gamma scaled by sqrt(1/N), omega per
    channel) behind the same interface as the complex layer."""

    def __init__(self, embed_dim, ndim=2, bidirectional=False, truncation=None, shift=True):
        super().__init__(bidirectional, truncation, shift)
        self.complex = False
        self.embed_dim = embed_dim
        self.ndim = ndim
        self.scale = math.sqrt(1.0 / self.ndim)
        kernel_dim = 2 * embed_dim if self.bidirectional else embed_dim
        self.alpha = nn.Parameter(torch.Tensor(kernel_dim, ndim, 1))
        self.delta = nn.Parameter(torch.Tensor(kernel_dim, ndim, 1))
        self.beta = nn.Parameter(torch.Tensor(kernel_dim, ndim, 1))
        self.gamma = nn.Parameter(torch.Tensor(kernel_dim, ndim))
        self.omega = nn.Parameter(torch.Tensor(embed_dim))
        self.register_parameters_no_weight_decay('alpha', self.alpha)
        self.register_parameters_no_weight_decay('delta', self.delta)
        self.reset_parameters()

    def reset_parameters(self):
        """alpha, delta ~ N(0, 0.2); beta = +1, -1, +1, ... along the states plus N(0, 0.02); gamma, omega ~ N(0, 1)
        (exponential_moving_average.py:47-69)."""
        with torch.no_grad():
            self.alpha.normal_(0.0, 0.2)
            self.delta.normal_(0.0, 0.2)
            signs = 1.0 - 2.0 * (torch.arange(self.ndim) % 2).to(self.beta.dtype)
            self.beta.normal_(0.0, 0.02).add_(signs.view(1, self.ndim, 1))
            self.gamma.normal_(0.0, 1.0)
            self.omega.normal_(0.0, 1.0)

    def _calc_coeffs(self):
        """p = sigmoid(alpha) beta, q = 1 - sigmoid(alpha) sigmoid(delta), gamma scaled by sqrt(1 / N)
        (exponential_moving_average.py:71-80); on the GPU one launch."""
        self._coeffs = None
        return self._calc_all()[:3]

    def _calc_all(self):
        """(p, q, gamma, omega): the coefficients and the residual weight as the kernels take them."""
        if _one_cuda_dtype(self.alpha, self.delta, self.beta, self.gamma, self.omega):
            return EMACoeffsFunc.apply(self.alpha, self.delta, self.beta, self.gamma, self.omega, False)
        return self._calc_coeffs_torch() + (self.omega,)

    def _calc_coeffs_torch(self):
        a = torch.sigmoid(self.alpha.float())
        return a * self.beta.float(), 1.0 - a * torch.sigmoid(self.delta.float()), self.gamma.float() * self.scale


class MultiHeadComplexEMA(BaseMovingLayer):
    """Complex EMA of Mega2 (fairseq/modules/complex_exponential_moving_average.py:15-113)."""

    def __init__(self, embed_dim, ndim=2, bidirectional=False, truncation=None, shift=True):
        super().__init__(bidirectional, truncation, shift)
        self.complex = True
        self.embed_dim = embed_dim
        self.ndim = ndim
        self.scale = math.sqrt(1.0 / self.ndim)
        kernel_dim = 2 * embed_dim if self.bidirectional else embed_dim
        self.alpha = nn.Parameter(torch.Tensor(kernel_dim, ndim, 1))
        self.delta = nn.Parameter(torch.Tensor(kernel_dim, ndim, 1))
        self.theta = nn.Parameter(torch.Tensor(kernel_dim, 1, 1))
        self.gamma = nn.Parameter(torch.Tensor(kernel_dim, ndim, 2))
        self.omega = nn.Parameter(torch.Tensor(embed_dim, 1))
        self.register_parameters_no_weight_decay('alpha', self.alpha)
        self.register_parameters_no_weight_decay('delta', self.delta)
        self.register_parameters_no_weight_decay('theta', self.theta)
        self.reset_parameters()

    def reset_parameters(self):
        """Initial values as the reference draws them (complex_exponential_moving_average.py:47-77): alpha, delta
        ~ N(0, 0.2); theta = logit of the base frequencies D^(-j / D), j = 1..D, shuffled over the channels (both
        directions of a two-sided layer share them); gamma real-valued ~ N(0, 1); omega ~ N(0, 1)."""
        D = self.embed_dim
        with torch.no_grad():
            self.alpha.normal_(0.0, 0.2)
            self.delta.normal_(0.0, 0.2)
            base = torch.exp(torch.arange(1, D + 1) * (-math.log(D) / D))
            base = base[torch.randperm(D)].to(self.theta).view(D, 1, 1)
            self.theta.copy_(torch.logit(base.repeat(2, 1, 1) if self.bidirectional else base))
            self.gamma.normal_(0.0, 1.0)
            self.gamma[..., 1].zero_()
            self.omega.normal_(0.0, 1.0)

    def _calc_coeffs(self):
        """p = sigmoid(alpha); q: state n of a channel shrinks by 1 - sigmoid(alpha) sigmoid(delta) and turns by
        (n + 1) sigmoid(theta) 2 pi / N per token; gamma complex, scaled by sqrt(1 / N)
        (complex_exponential_moving_average.py:79-96); on the GPU one launch."""
        self._coeffs = None
        return self._calc_all()[:3]

    def _calc_all(self):
        """(p, q, gamma, omega): the coefficients and the residual weight as the kernels take them."""
        if _one_cuda_dtype(self.alpha, self.delta, self.theta, self.gamma, self.omega):
            return EMACoeffsFunc.apply(self.alpha, self.delta, self.theta, self.gamma, self.omega, True)
        return self._calc_coeffs_torch() + (self.omega,)

    def _calc_coeffs_torch(self):
        a = torch.sigmoid(self.alpha.float())
        d = torch.sigmoid(self.delta.float())
        turn = torch.sigmoid(self.theta.float()) * (2.0 * math.pi / self.ndim)                      # [K, 1, 1]
        harmonic = torch.arange(1, self.ndim + 1, dtype=turn.dtype, device=turn.device).view(1, self.ndim, 1)
        q = torch.polar(1.0 - a * d, harmonic * turn)
        return a, q, torch.view_as_complex(self.gamma.float().contiguous()) * self.scale


class TimestepNormFunc(torch.autograd.Function):
    """fairseq/modules/norm_layer/timestep_norm.py:14-66: the forward keeps (group_mean,) cummean,
    cumrstd for the backward pass; count is an integer output without a gradient."""

    @staticmethod
    def forward(ctx, x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask=None, num_groups=None,
                eps: float = 1e-5):
        if num_groups is None:
            y, count, mean, var, cummean, cumrstd = ops.timestep_norm_fwd(x, prev_count, prev_mean, prev_var, gamma,
                                                                          beta, padding_mask, eps)
            ctx.save_for_backward(x, prev_mean, count, cummean, cumrstd, gamma, padding_mask)
        else:
            y, count, mean, var, group_mean, cummean, cumrstd = ops.group_timestep_norm_fwd(
                x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, num_groups, eps)
            ctx.save_for_backward(x, prev_mean, count, group_mean, cummean, cumrstd, gamma, padding_mask)
        ctx.num_groups = num_groups
        ctx.mark_non_differentiable(count)
        ctx.set_materialize_grads(False)        # unused final statistics: no zero tensors made for their gradients
        return y, count, mean, var

    @staticmethod
    def backward(ctx, y_grad, _, mean_grad, var_grad):
        if y_grad is None:
            y_grad = torch.zeros_like(ctx.saved_tensors[0])
        if ctx.num_groups is None:
            x, prev_mean, count, cummean, cumrstd, gamma, padding_mask = ctx.saved_tensors
            grads = ops.timestep_norm_bwd(y_grad, mean_grad, var_grad, x, prev_mean, count, cummean, cumrstd, gamma,
                                          padding_mask)
        else:
            x, prev_mean, count, group_mean, cummean, cumrstd, gamma, padding_mask = ctx.saved_tensors
            grads = ops.group_timestep_norm_bwd(y_grad, mean_grad, var_grad, x, prev_mean, count, group_mean, cummean,
                                                cumrstd, gamma, padding_mask, ctx.num_groups)
        x_grad, prev_mean_grad, prev_var_grad, gamma_grad, beta_grad = grads
        return (x_grad, None, prev_mean_grad.to(prev_mean.dtype).view_as(prev_mean), prev_var_grad.view_as(prev_mean),
                gamma_grad.to(gamma.dtype), beta_grad, None, None, None)


timestep_norm = TimestepNormFunc.apply


class TimestepNorm(nn.Module, IncrementalState):
    """Streaming cumulative (group) normalisation with a carried (count, mean, var) state
    (fairseq/modules/norm_layer/timestep_norm.py:71-167).  mean / var are carried in fp32."""

    def __init__(self, num_features: int, num_groups: Optional[int] = None, prior_count: int = 0,
                 eps: float = 1e-5) -> None:
        super().__init__()
        self.init_incremental_state()
        self.num_features = num_features
        self.num_groups = num_groups
        self._prior_count = prior_count
        self._prior_cache = {}
        self._affine_cache = None
        self._cache_key = None
        if num_groups is None or num_groups == num_features:
            num_groups = num_features
            assert prior_count > 1
        else:
            assert self.num_features % num_groups == 0
        self.register_buffer("prior_count", torch.tensor(prior_count, dtype=torch.int64))
        if prior_count > 0:
            self.register_parameter("prior_mean", Parameter(torch.zeros(num_groups), requires_grad=True))
            self.register_parameter("prior_logv", Parameter(torch.zeros(num_groups), requires_grad=True))
        else:
            self.register_buffer("prior_mean", torch.zeros(num_groups))
            self.register_buffer("prior_logv", torch.zeros(num_groups))
        self.register_parameter("weight", Parameter(torch.zeros(num_features), requires_grad=True))
        self.register_parameter("bias", Parameter(torch.zeros(num_features), requires_grad=True))
        self.eps = eps

    def forward(self, x: Tensor, padding_mask: Optional[Tensor] = None,
                incremental_state: Optional[Dict[str, Dict[str, Optional[Tensor]]]] = None) -> Tensor:
        batch_size = x.size(0)
        train = torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.parameters()))
        prev_mean = prev_var = prev_count = None
        saved_state = None
        if incremental_state is not None:
            saved_state = self._get_input_buffer(incremental_state)
            if 'prev_mean' in saved_state:
                prev_mean = saved_state['prev_mean']
                assert 'prev_var' in saved_state and 'prev_count' in saved_state
                prev_var = saved_state['prev_var']
                prev_count = saved_state['prev_count']
        norm_gamma = norm_beta = None
        if train and prev_count is None and prev_mean is None and prev_var is None:
            prev_count, norm_gamma, norm_beta, prev_mean, prev_var = self._training_operands(batch_size)
        if prev_count is None or prev_mean is None or prev_var is None:
            d_count, d_mean, d_var = self._prior_state(batch_size, train)
            prev_count = d_count if prev_count is None else prev_count
            prev_mean = d_mean if prev_mean is None else prev_mean
            prev_var = d_var if prev_var is None else prev_var
        if train:
            # the autograd path of the reference (timestep_norm.py:129-136): prior, weight + 1 and
            # bias stay in the graph; statistics for the backward pass are kept
            if norm_gamma is None:
                norm_gamma, norm_beta = self.weight.float() + 1.0, self.bias.float()
            out, count, mean, var = timestep_norm(x, prev_count, prev_mean, prev_var, norm_gamma, norm_beta,
                                                  padding_mask, self.num_groups, self.eps)
            if incremental_state is not None:
                saved_state['prev_mean'], saved_state['prev_var'], saved_state['prev_count'] = mean, var, count
                self._set_input_buffer(incremental_state, saved_state)
            return out
        gamma, beta = self._affine()
        if self.num_groups is None:
            out, count, mean, var, _, _ = ops.timestep_norm_fwd(x, prev_count, prev_mean, prev_var, gamma, beta,
                                                                padding_mask, self.eps, need_stats=False)
        else:
            out, count, mean, var, _, _, _ = ops.group_timestep_norm_fwd(x, prev_count, prev_mean, prev_var, gamma,
                                                                         beta, padding_mask, self.num_groups,
                                                                         self.eps, need_stats=False)
        if incremental_state is not None:
            saved_state['prev_mean'] = mean
            saved_state['prev_var'] = var
            saved_state['prev_count'] = count
            self._set_input_buffer(incremental_state, saved_state)
        return out

    def _training_operands(self, batch_size: int):
        """(count [B], weight + 1 [H], bias [H], prior mean [B, G], prior variance [B, G]) with the last four in the
        autograd graph (timestep_norm.py:118-131): one launch on the GPU, torch operations elsewhere."""
        count = self.prior_count.expand(batch_size).contiguous()
        if _one_cuda_dtype(self.weight, self.bias) and _one_cuda_dtype(self.prior_mean, self.prior_logv):
            return (count,) + tuple(NormParamsFunc.apply(self.weight, self.bias, self.prior_mean, self.prior_logv,
                                                         batch_size))
        _, mean, var = self._prior_state(batch_size, differentiable=True)
        return count, self.weight.float() + 1.0, self.bias.float(), mean, var

    def _prior_state(self, batch_size: int, differentiable: bool = False):
        """(count[B], mean[B,G], var[B,G]) of the prior (timestep_norm.py:122-127); cached in eval mode."""
        if differentiable:
            return (self.prior_count.expand(batch_size).contiguous(),
                    self.prior_mean.float().expand(batch_size, -1),
                    torch.exp(self.prior_logv.float()).expand(batch_size, -1))
        key = batch_size
        if not self.training:
            self._drop_stale_cache()
            if key in self._prior_cache:
                return self._prior_cache[key]
        with torch.no_grad():
            st = (self.prior_count.expand(batch_size).contiguous(),
                  self.prior_mean.float().expand(batch_size, -1).contiguous(),
                  torch.exp(self.prior_logv.float()).expand(batch_size, -1).contiguous())
        if not self.training:
            self._prior_cache[key] = st
        return st

    def _affine(self):
        """(weight + 1, bias) in fp32, as the reference passes them (timestep_norm.py:129-131)."""
        if not self.training:
            self._drop_stale_cache()
            if self._affine_cache is not None:
                return self._affine_cache
        with torch.no_grad():
            ab = (self.weight.float() + 1.0, self.bias.float().contiguous())
        self._affine_cache = None if self.training else ab
        return ab

    def _drop_stale_cache(self):
        """The eval-mode caches follow the parameters and buffers they were computed from."""
        key = _tensor_versions(self)
        if key != self._cache_key:
            self._prior_cache = {}
            self._affine_cache = None
            self._cache_key = key

    def train(self, mode: bool = True):
        self._prior_cache = {}
        self._affine_cache = None
        return super().train(mode)

    def _apply(self, fn, *args, **kwargs):
        self._prior_cache = {}
        self._affine_cache = None
        return super()._apply(fn, *args, **kwargs)

    def _get_input_buffer(self, incremental_state):
        result = self.get_incremental_state(incremental_state, "norm_state")
        return result if result is not None else {}

    def _set_input_buffer(self, incremental_state, buffer):
        return self.set_incremental_state(incremental_state, "norm_state", buffer)

    def reorder_incremental_state(self, incremental_state, new_order: Tensor):
        input_buffer = self._get_input_buffer(incremental_state)
        if input_buffer is not None:
            for k in input_buffer.keys():
                if input_buffer[k] is not None:
                    input_buffer[k] = input_buffer[k].index_select(0, new_order)
            incremental_state = self._set_input_buffer(incremental_state, input_buffer)
        return incremental_state

    def extra_repr(self) -> str:
        return 'num_features={num_features}, num_groups={num_groups}, prior_count={_prior_count}, eps={eps}'.format(
            **self.__dict__)


class NormThenMoveFunc(torch.autograd.Function):
    """x = norm(x); mx = move(x^T) as one differentiable operator whose forward is one library call
    (moving_average_gated_attention.py:304-315; the reference chains GroupTimestepNormFunc,
    norm_layer/timestep_norm.py:14-66, EMAParametersFunc and FFTConvFunc).  The forward keeps x, xn and the
    norm's running statistics; the backward runs the moving average backwards in time on mx's gradient, adds
    the result to xn's own gradient and hands the sum to the norm's backward pass."""

    ENABLED = True          # False: training runs the two modules' own operators one after the other

    @staticmethod
    def forward(ctx, x, prev_count, prev_mean, prev_var, norm_gamma, norm_beta, p, q, gamma, omega, padding_mask,
                num_groups, eps, out_layout, shift):
        layer = ops.PreparedEMA(p.squeeze(-1), q.squeeze(-1), gamma, omega.reshape(-1), False, None, shift)
        xn, y, count, _, _, _, cummean, cumrstd = layer.norm_forward(
            x, prev_count, prev_mean, prev_var, norm_gamma, norm_beta, num_groups, eps, padding_mask, None,
            want_state=False, out_layout=out_layout, want_stats=True)
        ctx.layer = layer
        ctx.num_groups = num_groups
        ctx.save_for_backward(x, xn, prev_mean, count, cummean, cumrstd, norm_gamma, p, q, gamma, omega, padding_mask)
        return xn, y

    @staticmethod
    def backward(ctx, xn_grad, y_grad):
        x, xn, prev_mean, count, cummean, cumrstd, norm_gamma, p, q, gamma, omega, padding_mask = ctx.saved_tensors
        total = xn_grad
        dp = dq = dg = dom = None
        if y_grad is not None:
            dxe, dp, dq, dg, dom = ops.ema_backward(y_grad, xn.transpose(1, 2), p.squeeze(-1), q.squeeze(-1), gamma,
                                                    omega.reshape(-1), padding_mask, layer=ctx.layer)
            dxe = dxe.transpose(1, 2)
            total = dxe if total is None else total + dxe
            dp, dq = dp.to(p.dtype).view_as(p), dq.to(q.dtype).view_as(q)
            dg, dom = dg.to(gamma.dtype).view_as(gamma), dom.to(omega.dtype).view_as(omega)
        x_grad, pm_grad, pv_grad, ng_grad, nb_grad = ops.group_timestep_norm_bwd(
            total.contiguous(), None, None, x, prev_mean, count, None, cummean, cumrstd, norm_gamma, padding_mask,
            ctx.num_groups)
        return (x_grad, None, pm_grad.to(prev_mean.dtype).view_as(prev_mean), pv_grad.view_as(prev_mean),
                ng_grad.to(norm_gamma.dtype), nb_grad, dp, dq, dg, dom, None, None, None, None, None)


def norm_then_move(norm: nn.Module, move: nn.Module, x: Tensor, padding_mask: Optional[Tensor] = None,
                   incremental_state: Optional[Dict[str, Dict[str, Optional[Tensor]]]] = None,
                   out_layout: str = "rows") -> Tuple[Tensor, Tensor]:
    """x = norm(x); mx = move(x^T), the head of the layer (moving_average_gated_attention.py:304-315).
    x: [B, L, D] -> (xn [B, L, D], mx [B, D, L] in `out_layout`).  A group TimestepNorm in front of a
    one-sided layer without kernel truncation, called without autograd, goes to the library as one call
    (x is read once, xn and mx are written once); both modules' incremental state is kept exactly as the
    two calls keep it.  Under autograd the same call is one differentiable operator (NormThenMoveFunc) when no
    state is carried.  Every other combination runs the two modules one after the other."""
    one_call = (isinstance(norm, TimestepNorm) and norm.num_groups is not None and isinstance(move, BaseMovingLayer)
                and not move.bidirectional and (move.truncation is None or move.truncation < 1)
                and x.is_cuda and x.dim() == 3 and x.size(0) > 0 and x.size(1) > 0)
    training = one_call and (_training_call(norm, x) or _training_call(move, x))
    if training and incremental_state is None and NormThenMoveFunc.ENABLED:
        prev_count, norm_gamma, norm_beta, prev_mean, prev_var = norm._training_operands(x.size(0))
        p, q, gamma, omega = move._calc_all()           # stay in the graph
        return NormThenMoveFunc.apply(x, prev_count, prev_mean, prev_var, norm_gamma, norm_beta, p, q, gamma, omega,
                                      padding_mask, norm.num_groups, norm.eps, out_layout, move.shift)
    if not one_call or training:
        xn = norm(x, padding_mask=padding_mask, incremental_state=incremental_state)
        return xn, move(xn.transpose(1, 2), padding_mask, incremental_state, out_layout=out_layout)
    batch_size = x.size(0)
    norm_state = move_state = None
    prev_count = prev_mean = prev_var = h = None
    if incremental_state is not None:
        norm_state = norm._get_input_buffer(incremental_state)
        if 'prev_mean' in norm_state:
            prev_mean, prev_var, prev_count = norm_state['prev_mean'], norm_state['prev_var'], norm_state['prev_count']
        move_state = move._get_input_buffer(incremental_state)
        h = move_state.get('prev_state')
    if prev_count is None or prev_mean is None or prev_var is None:
        d_count, d_mean, d_var = norm._prior_state(batch_size)
        prev_count = d_count if prev_count is None else prev_count
        prev_mean = d_mean if prev_mean is None else prev_mean
        prev_var = d_var if prev_var is None else prev_var
    gamma, beta = norm._affine()
    xn, y, count, mean, var, h_out = move._prepared_layer().norm_forward(
        x, prev_count, prev_mean, prev_var, gamma, beta, norm.num_groups, norm.eps, padding_mask, h,
        want_state=incremental_state is not None, out_layout=out_layout)
    if incremental_state is not None:
        norm_state['prev_mean'], norm_state['prev_var'], norm_state['prev_count'] = mean, var, count
        norm._set_input_buffer(incremental_state, norm_state)
        move_state['prev_state'] = h_out
        move._set_input_buffer(incremental_state, move_state)
    return xn, y


class SequenceNormFunc(torch.autograd.Function):
    """fairseq/modules/norm_layer/sequence_norm.py:12-49."""

    @staticmethod
    def forward(ctx, x, gamma, beta, padding_mask=None, num_groups=None, eps: float = 1e-5, length_last: bool = False):
        G = (x.shape[1] if length_last else x.shape[2]) if num_groups is None else num_groups
        y, count, mean, rstd = ops.group_sequence_norm_fwd(x, gamma, beta, padding_mask, G, eps, length_last)
        ctx.save_for_backward(x, count, mean, rstd, gamma, padding_mask)
        ctx.groups = G
        ctx.length_last = length_last
        return y

    @staticmethod
    def backward(ctx, y_grad):
        x, count, mean, rstd, gamma, padding_mask = ctx.saved_tensors
        dx, dg, db = ops.group_sequence_norm_bwd(y_grad, x, count, mean, rstd, gamma, padding_mask, ctx.groups,
                                                 ctx.length_last)
        return dx, dg.to(gamma.dtype), db, None, None, None, None


sequence_norm = SequenceNormFunc.apply


class SequenceNorm(nn.Module):
    """Whole-sequence (group) normalisation of bidirectional layers
    (fairseq/modules/norm_layer/sequence_norm.py:54-74): x [B, H, L], statistics per (row, group)
    over the unmasked tokens."""

    def __init__(self, num_features: int, num_groups: Optional[int] = None, eps: float = 1e-5) -> None:
        super().__init__()
        self.num_features = num_features
        self.num_groups = num_groups
        assert self.num_groups is None or self.num_features % self.num_groups == 0
        self.register_parameter("weight", Parameter(torch.zeros(num_features), requires_grad=True))
        self.register_parameter("bias", Parameter(torch.zeros(num_features), requires_grad=True))
        self.eps = eps

    def forward(self, x: Tensor, padding_mask: Optional[Tensor] = None, length_last: bool = True) -> Tensor:
        if _training_call(self, x):
            return sequence_norm(x, self.weight.float() + 1.0, self.bias.float(), padding_mask, self.num_groups,
                                 self.eps, length_last)
        gamma, beta = self.weight.float() + 1.0, self.bias.float()
        if self.num_groups is None:
            return ops.sequence_norm_fwd(x, gamma, beta, padding_mask, self.eps, length_last)[0]
        return ops.group_sequence_norm_fwd(x, gamma, beta, padding_mask, self.num_groups, self.eps, length_last)[0]

    def extra_repr(self) -> str:
        return 'num_features={num_features}, num_groups={num_groups}, eps={eps}'.format(**self.__dict__)


class SplitGrads(object):
    """The gradients of the slices of one split tensor, written in place.  `torch.split` hands every slice's
    gradient to a concatenation in its backward pass (the mx_proj output of
    moving_average_gated_attention.py:319 is split four ways: a 142 MB copy per step at the Mega2 layer's size).
    The backward kernels of the slices' consumers instead write into the slices of one buffer that this
    object hands out (`slot(i)`), and SplitFunc's backward returns that buffer when every gradient it receives
    is the slot it handed out, and concatenates otherwise.  A new buffer per backward pass."""

    taken = 0        # backward passes that needed no concatenation (all objects; read by the tests)

    def __init__(self, like: Tensor, widths):
        self.shape, self.dtype, self.device = like.shape, like.dtype, like.device
        self.widths = list(widths)
        self.offsets = [sum(self.widths[:i]) for i in range(len(self.widths))]
        self.buf = None

    def slot(self, i: int) -> Tensor:
        if self.buf is None:
            self.buf = torch.empty(self.shape, dtype=self.dtype, device=self.device)
        return self.buf.narrow(-1, self.offsets[i], self.widths[i])

    def take(self, grads) -> Optional[Tensor]:
        """The buffer, if `grads` are exactly its slots; the buffer is released either way."""
        buf, self.buf = self.buf, None
        if buf is None or len(grads) != len(self.widths):
            return None
        for i, g in enumerate(grads):
            if g is None or g.dtype != buf.dtype or g.shape[:-1] != buf.shape[:-1] or g.shape[-1] != self.widths[i] \
                    or g.stride() != buf.stride() \
                    or g.data_ptr() != buf.data_ptr() + self.offsets[i] * buf.element_size():
                return None
        SplitGrads.taken += 1
        return buf


class SplitFunc(torch.autograd.Function):
    """torch.split(base, widths, -1) whose backward takes the slices' gradients from a SplitGrads buffer."""

    @staticmethod
    def forward(ctx, base, arena):
        ctx.arena = arena
        return tuple(base.narrow(-1, o, w) for o, w in zip(arena.offsets, arena.widths))

    @staticmethod
    def backward(ctx, *grads):
        arena = ctx.arena
        buf = arena.take(grads)
        if buf is not None:
            return buf, None
        parts = [g if g is not None else torch.zeros(arena.shape[:-1] + (w,), dtype=arena.dtype, device=arena.device)
                 for g, w in zip(grads, arena.widths)]
        return torch.cat(parts, dim=-1), None


class GateQKFunc(torch.autograd.Function):
    """q, k = rotary(normalize(z) * (gamma + 1) + beta) in one pass over z, with one backward pass
    (moving_average_gated_attention.py:324-328, relative_positional_bias.py:86-97).  gamma, beta are
    the layer's [2, S] parameters; freqs holds zeros when the layer does not rotate."""

    @staticmethod
    def forward(ctx, z, gamma, beta, freqs, num_heads, chunk, slot=None):
        g1 = gamma.detach().float() + 1.0
        ctx.save_for_backward(z, g1, freqs)
        ctx.num_heads, ctx.chunk, ctx.slot = num_heads, chunk, slot
        ctx.param_dtypes = (gamma.dtype, beta.dtype)
        return ops.gate_qk_fwd(z, g1, beta.detach().float(), freqs, num_heads, chunk)

    @staticmethod
    def backward(ctx, q_grad, k_grad):
        z, g1, freqs = ctx.saved_tensors
        out = None if ctx.slot is None else ctx.slot[0].slot(ctx.slot[1])
        dz, dgamma, dbeta = ops.gate_qk_bwd(q_grad, k_grad, z, g1, freqs, ctx.num_heads, ctx.chunk, z_grad_out=out)
        return dz, dgamma.to(ctx.param_dtypes[0]), dbeta.to(ctx.param_dtypes[1]), None, None, None, None


class GateMulFunc(torch.autograd.Function):
    """a * silu(r) with its own backward (moving_average_gated_attention.py:330, 407)."""

    @staticmethod
    def forward(ctx, a, r, slot=None):
        ctx.save_for_backward(a, r)
        ctx.slot = slot
        return ops.gate_mul_fwd(a, r)

    @staticmethod
    def backward(ctx, y_grad):
        out = None if ctx.slot is None else ctx.slot[0].slot(ctx.slot[1])
        da, dr = ops.gate_mul_bwd(y_grad, *ctx.saved_tensors, r_grad_out=out)
        return da, dr, None


class GateOutFunc(torch.autograd.Function):
    """residual + sigmoid(u) * (silu(hx + hp) - residual) with its own backward
    (moving_average_gated_attention.py:322, 409, 412)."""

    @staticmethod
    def forward(ctx, residual, u, hx, hp, slots=None):
        ctx.save_for_backward(residual, u, hx, hp)
        ctx.slots = slots
        return ops.gate_out_fwd(residual, u, hx, hp)

    @staticmethod
    def backward(ctx, y_grad):
        uo = ho = None
        if ctx.slots is not None:
            arena, iu, ih = ctx.slots
            uo, ho = arena.slot(iu), arena.slot(ih)
        dres, du, dh = ops.gate_out_bwd(y_grad, *ctx.saved_tensors, u_grad_out=uo, h_grad_out=ho)
        return dres, du, dh, dh, None


class SiluFunc(torch.autograd.Function):
    """F.silu with the library's kernels both ways."""

    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return ops.silu(x)

    @staticmethod
    def backward(ctx, y_grad):
        return ops.silu_bwd(y_grad, ctx.saved_tensors[0])


def silu(x: Tensor) -> Tensor:
    """silu(x): the library's kernels on the GPU (with their own backward under autograd), F.silu elsewhere."""
    if not x.is_cuda:
        return F.silu(x)
    if torch.is_grad_enabled() and x.requires_grad:
        return SiluFunc.apply(x)
    return ops.silu(x)


class LinearFunc(torch.autograd.Function):
    """F.linear whose backward takes the bias gradient from the library's column sums (torch's sum over the tokens
    runs at a third of the memory rate on matrices this wide); the three products stay library GEMMs, and a
    row-strided output gradient (a slice of a wider gradient buffer) is read in place."""

    @staticmethod
    def forward(ctx, x, weight, bias):
        ctx.save_for_backward(x, weight)
        ctx.has_bias = bias is not None
        return F.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, y_grad):
        x, weight = ctx.saved_tensors
        g2 = y_grad.reshape(-1, y_grad.shape[-1])
        x2 = x.reshape(-1, x.shape[-1])
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = torch.mm(g2, weight).view(x.shape)
        if ctx.needs_input_grad[1]:
            dw = torch.mm(g2.t(), x2)
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = ops.colsum(y_grad, weight.dtype)
        return dx, dw, db


def linear(lin: nn.Linear, x: Tensor) -> Tensor:
    """lin(x); under autograd on the GPU with the bias gradient as the library's column sums."""
    if lin.bias is not None and x.is_cuda and x.dtype == lin.weight.dtype and torch.is_grad_enabled() and \
            (x.requires_grad or lin.weight.requires_grad):
        return LinearFunc.apply(x, lin.weight, lin.bias)
    return lin(x)


class SwiGLUFunc(torch.autograd.Function):
    """silu(a) * b with its own backward."""

    @staticmethod
    def forward(ctx, a, b):
        ctx.save_for_backward(a, b)
        return ops.swiglu(a, b)

    @staticmethod
    def backward(ctx, y_grad):
        return ops.swiglu_bwd(y_grad, *ctx.saved_tensors)


class AttentionSoftmaxFunc(torch.autograd.Function):
    """fairseq/modules/attention_softmax.py:11-39.  The saved output already holds zeros at the
    dropped keys, so the backward needs no mask.  `seed` (not in the reference) pins the mask."""

    @staticmethod
    def forward(ctx, x, dropout: float = 0.0, use_causal_mask: bool = True, training: bool = True, seed=None):
        y = ops.attention_softmax_fwd(x, dropout if training else 0.0, use_causal_mask, seed)
        ctx.save_for_backward(y)
        ctx.use_causal_mask = use_causal_mask
        return y

    @staticmethod
    def backward(ctx, y_grad):
        y, = ctx.saved_tensors
        return ops.attention_softmax_bwd(y_grad, y, ctx.use_causal_mask), None, None, None, None


class AttentionFunc(torch.autograd.Function):
    """fairseq/modules/efficient_attention.py:11-40.  The reference's forward keeps the L x L weights (after
    DropKey) for the backward pass.  Here they are kept only with DropKey or outside the matrix-core envelope;
    otherwise the forward is the one-kernel attention (no L x L array at all), q, k, v and y are saved, and the backward
    forms the weights again in scratch memory before its four products: B Nh L^2 elements less to hold per layer
    between the passes (134 MB at configs[4]), the same gradients.  `KEEP_WEIGHTS = True` restores the reference's
    behaviour.  `seed` (not in the reference) pins the DropKey mask."""

    KEEP_WEIGHTS = False

    @staticmethod
    def forward(ctx, q, k, v, scale: float = 1.0, dropout: float = 0.0, use_causal_mask: bool = True,
                training: bool = True, seed=None):
        drop = dropout if training else 0.0
        ctx.scale = scale
        ctx.use_causal_mask = use_causal_mask
        if not AttentionFunc.KEEP_WEIGHTS and ops.attention_keeps_no_weights(q, k, v, drop):
            y, _ = ops.attention_fwd(q, k, v, scale, 0.0, use_causal_mask, need_weights=False)
            ctx.save_for_backward(q, k, v, y)
            ctx.has_weights = False
            return y
        y, w = ops.attention_fwd(q, k, v, scale, drop, use_causal_mask, need_weights=True, seed=seed)
        ctx.save_for_backward(q, k, v, w, y)          # y: lets the backward form the softmax's row sums as y_grad . y
        ctx.has_weights = True
        return y

    @staticmethod
    def backward(ctx, y_grad):
        if ctx.has_weights:
            q, k, v, w, y = ctx.saved_tensors
        else:
            q, k, v, y = ctx.saved_tensors
            _, w = ops.attention_fwd(q, k, v, ctx.scale, 0.0, ctx.use_causal_mask, weights_only=True)
        q_grad, k_grad, v_grad = ops.attention_bwd(y_grad, q, k, v, w, ctx.scale, ctx.use_causal_mask, y=y)
        return q_grad, k_grad, v_grad, None, None, None, None, None


attention_softmax = AttentionSoftmaxFunc.apply
attention = AttentionFunc.apply


def _wants_grad(*tensors) -> bool:
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


class AttentionSoftmax(nn.Module):
    """fairseq/modules/attention_softmax.py:44-56."""

    def __init__(self, dropout: float = 0.0, use_causal_mask: bool = False) -> None:
        super().__init__()
        self._dropout = dropout
        self._causal = use_causal_mask

    def forward(self, x: Tensor) -> Tensor:
        if _wants_grad(x):
            return attention_softmax(x, self._dropout, self._causal, self.training)
        return ops.attention_softmax_fwd(x, self._dropout if self.training else 0.0, self._causal)

    def extra_repr(self) -> str:
        return 'causal={}, dropout={}'.format(self._causal, self._dropout)


class EfficientAttention(nn.Module):
    """fairseq/modules/efficient_attention.py:45-63: q, k: [B, L, H1], v: [B, L, H2]
    (single head), or the 4-D [B, L, Nh, H] layout of the op itself."""

    def __init__(self, scale: float = 1.0, dropout: float = 0.0, use_causal_mask: bool = True) -> None:
        super().__init__()
        self._scale = scale
        self._dropout = dropout
        self._causal = use_causal_mask

    def forward(self, q: Tensor, k: Tensor, v: Tensor) -> Tensor:
        squeeze = q.dim() == 3
        if squeeze:
            q, k, v = q.unsqueeze(2), k.unsqueeze(2), v.unsqueeze(2)
        if _wants_grad(q, k, v):
            out = attention(q, k, v, self._scale, self._dropout, self._causal, self.training)
        else:
            out, _ = ops.attention_fwd(q, k, v, self._scale, self._dropout if self.training else 0.0, self._causal)
        return out.squeeze(2) if squeeze else out

    def extra_repr(self) -> str:
        return 'causal={}, dropout={}'.format(self._causal, self._dropout)


def linear_residual(lin: nn.Linear, h: Tensor, residual: Optional[Tensor], consume: bool = False) -> Tensor:
    """lin(h) + residual as one library GEMM (the residual is the accumulator's start, rounded once with the
    product); lin(h) when there is no residual.  consume: the caller owns `residual` and has no further use for
    it, so outside autograd the product is accumulated into it in place (the out-of-place form first copies the
    residual into its result: one more pass over the activations)."""
    if residual is None:
        return lin(h)
    if lin.bias is not None or residual.dtype != h.dtype or not residual.is_contiguous():
        return lin(h) + residual
    r2, h2 = residual.reshape(-1, residual.shape[-1]), h.reshape(-1, h.shape[-1])
    if consume and not torch.is_grad_enabled() and not residual.requires_grad:
        r2.addmm_(h2, lin.weight.t())
        return residual
    return torch.addmm(r2, h2, lin.weight.t()).view(residual.shape)


class SwiGLU(nn.Module):
    """W2 (silu(W1 x) * W3 x) with the gate evaluated by the HIP kernel; the three
    projections are library GEMMs."""

    def __init__(self, embed_dim: int, hidden_dim: int, bias: bool = False) -> None:
        super().__init__()
        self.w1 = nn.Linear(embed_dim, hidden_dim, bias=bias)
        self.w3 = nn.Linear(embed_dim, hidden_dim, bias=bias)
        self.w2 = nn.Linear(hidden_dim, embed_dim, bias=bias)

    def forward(self, x: Tensor, residual: Optional[Tensor] = None, consume_residual: bool = False) -> Tensor:
        """W2 (silu(W1 x) * W3 x) (+ residual, which then enters the last product as its accumulator start: no
        separate addition pass over the activations; consume_residual: see linear_residual)."""
        gate = SwiGLUFunc.apply(self.w1(x), self.w3(x)) if _training_call(self, x) else ops.swiglu(self.w1(x), self.w3(x))
        return linear_residual(self.w2, gate, residual, consume_residual)
