"""Layer glue around the HIP ops: the caller of the hot path in the reference,
`MovingAverageGatedAttention` (fairseq/modules/moving_average_gated_attention.py:26-470),
restricted to the rotary softmax attention through the fused ops (causal with TimestepNorm and a
one-sided EMA / CEMA, or bidirectional with SequenceNorm and a two-sided one), plus the north-star
SwiGLU FFN.

The projections are library GEMMs (torch -> hipBLASLt); normalisation, moving average,
attention and the SwiGLU gate run in libmega_hip.so.  Under autograd the normalisation, the
moving average and the attention (softmax backward in libmega_hip.so, batched library GEMMs) keep
their own backward operators, and so do the r gate, the output gate and the SwiGLU gate; the
remaining element-wise steps (q / k map, activations of v and of the moving average) run as torch
operations so that the graph is complete.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn
from torch.nn import Parameter

from . import ops
from .modules import (AttentionSoftmax, EfficientAttention, GateMulFunc, GateOutFunc, GateQKFunc, IncrementalState,
                      MultiHeadComplexEMA, MultiHeadEMA, SequenceNorm, SplitFunc, SplitGrads, SwiGLU, TimestepNorm,
                      _tensor_versions, _training_call, linear, linear_residual, norm_then_move, silu)


class RMSNorm(nn.Module):
    """x / sqrt(mean(x^2) + eps) * (weight + 1): the parameter is stored as the offset from one and starts at zero, as
    in the reference (fairseq/modules/norm_layer/layer_norm.py:41-59: FusedRMSNorm.reset_parameters zeroes it and
    forward passes `self.weight + 1.0`), so a reference checkpoint's `*.weight` loads unchanged.  One wave per token
    in the HIP library."""

    def __init__(self, dim: int, elementwise_affine: bool = True, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        if elementwise_affine:
            self.weight = Parameter(torch.zeros(dim))
        else:
            self.register_parameter("weight", None)

    def forward(self, x: Tensor) -> Tensor:
        w = None if self.weight is None else self.weight.float() + 1.0
        if _training_call(self, x):
            y = x.float()
            y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + self.eps)
            if w is not None:
                y = y * w
            return y.to(x.dtype)
        return ops.rms_norm_fwd(x, w, self.eps)


class LayerNorm(nn.Module):
    """Layer normalisation with the affine weight stored as its offset from one (zero-initialised weight and bias,
    `weight + 1` in the forward): fairseq/modules/norm_layer/layer_norm.py:85-111 (FairseqLayerNorm; the fused
    variant at :19-39 does the same).  A torch operation: it is not on the measured path."""

    def __init__(self, dim: int, eps: float = 1e-5, elementwise_affine: bool = True):
        super().__init__()
        self.normalized_shape = (dim,)
        self.eps = eps
        if elementwise_affine:
            self.weight = Parameter(torch.zeros(dim))
            self.bias = Parameter(torch.zeros(dim))
        else:
            self.register_parameter("weight", None)
            self.register_parameter("bias", None)

    def forward(self, x: Tensor) -> Tensor:
        w = None if self.weight is None else self.weight + 1.0
        return F.layer_norm(x, self.normalized_shape, w, self.bias, self.eps)


class NormalizedFeedForwardNetwork(nn.Module):
    """The reference's position-wise block, `x + fc2(silu(fc1(norm(x))))` with an optional
    per-feature layer scale (fairseq/modules/normalized_feedforward_network.py:13-93; same
    constructor arguments, parameter names and initialisation; the two dropouts act in training
    mode only).  The two projections are library GEMMs; norm and activation are elementwise glue."""

    def __init__(self, embed_dim, ffn_hidden_dim, dropout=0.0, hidden_dropout=0.0, norm_type='layernorm',
                 norm_affine=True, norm_eps=1e-5, layer_scale=None, init_mode='bert', export=False):
        super().__init__()
        self.embedding_dim = embed_dim
        self.hidden_dim = ffn_hidden_dim
        self.act_fn = 'silu'
        self.init_mode = init_mode
        self.layer_scale = layer_scale
        self.dropout_p, self.hidden_dropout_p = float(dropout), float(hidden_dropout)
        if norm_type == 'layernorm':
            self.norm = LayerNorm(embed_dim, eps=norm_eps, elementwise_affine=norm_affine)
        elif norm_type == 'rmsnorm':
            self.norm = RMSNorm(embed_dim, elementwise_affine=norm_affine, eps=norm_eps)
        else:
            raise ValueError('unknown norm type: {}'.format(norm_type))
        self.fc1 = nn.Linear(embed_dim, ffn_hidden_dim, bias=True)
        self.fc2 = nn.Linear(ffn_hidden_dim, embed_dim, bias=False)
        if layer_scale is None:
            self.register_parameter('layerscale_weight', None)
        else:
            assert layer_scale > 0., 'Layer scale init value should be positive.'
            self.layerscale_weight = Parameter(torch.Tensor(embed_dim))
        assert init_mode in ['bert', 'xavier', 'he']
        self.reset_parameters(init_mode)

    def reset_parameters(self, mode):
        """'bert': N(0, 0.02); 'he': Kaiming normal with a = sqrt(5); otherwise Xavier uniform; zero bias; the layer
        scale starts at its given value (normalized_feedforward_network.py:56-75)."""
        init = {'bert': lambda w: nn.init.normal_(w, mean=0.0, std=0.02),
                'he': lambda w: nn.init.kaiming_normal_(w, a=math.sqrt(5.0))}.get(mode, nn.init.xavier_uniform_)
        for lin in (self.fc1, self.fc2):
            init(lin.weight)
        nn.init.zeros_(self.fc1.bias)
        if self.layerscale_weight is not None:
            nn.init.constant_(self.layerscale_weight, self.layer_scale)

    def forward(self, x: Tensor, consume_input: bool = False) -> Tensor:
        """consume_input: the caller owns x and does not use it again (the residual sum may be formed in it)."""
        # hidden dropout acts whenever the module is in training mode, with or without a graph
        # (normalized_feedforward_network.py:81-83)
        if _training_call(self, x) or (self.training and self.hidden_dropout_p > 0):
            h = F.dropout(silu(linear(self.fc1, self.norm(x))), self.hidden_dropout_p, self.training)
        else:
            h = ops.silu(self.fc1(self.norm(x)), inplace=True)
        if self.layerscale_weight is None and not (self.training and self.dropout_p > 0):
            return linear_residual(self.fc2, h, x, consume_input)      # the residual rides in the product
        h = F.dropout(self.fc2(h), self.dropout_p, self.training)
        if self.layerscale_weight is not None:
            h = h * self.layerscale_weight
        return h + x

    def extra_repr(self) -> str:
        return 'edim={}, hdim={}, act={}, init={}, layerscale={}'.format(self.embedding_dim, self.hidden_dim,
                                                                         self.act_fn, self.init_mode, self.layer_scale)


class RotaryEmbedding(nn.Module):
    """fairseq/modules/relative_positional_bias.py:47-97: features (2i, 2i+1) rotate by
    t * base^(-2i/dim); q may start at an offset (incremental decoding)."""

    def __init__(self, embed_dim: int, max_positions: int, base: Optional[float] = None):
        super().__init__()
        assert embed_dim % 2 == 0
        self.embed_dim = embed_dim
        self.max_positions = max_positions
        self.base = 10000 if base is None else base
        freqs = 1.0 / torch.tensor([self.base ** (j / embed_dim) for j in range(0, embed_dim, 2)], dtype=torch.float32)
        self.register_buffer("freqs", freqs)
        self._cis: Optional[Tensor] = None

    def _freqs_cis(self, start: int, end: int) -> Tensor:
        if self._cis is None or self._cis.shape[0] < end or self._cis.device != self.freqs.device:
            n = max(end, self.max_positions)
            t = torch.arange(n, dtype=torch.float32, device=self.freqs.device)
            ang = torch.outer(t, self.freqs.float())
            self._cis = torch.polar(torch.ones_like(ang), ang)
        return self._cis[start:end]

    def rotary(self, x: Tensor, sidx: int) -> Tensor:
        """x: [..., C, dim] with positions along the second to last axis."""
        cis = self._freqs_cis(sidx, sidx + x.shape[-2])
        x_ = torch.view_as_complex(x.float().reshape(*x.shape[:-1], -1, 2))
        return torch.view_as_real(x_ * cis).flatten(-2).to(x.dtype)

    def forward(self, xq: Tensor, xk: Tensor, qidx: int = 0) -> Tuple[Tensor, Tensor]:
        return self.rotary(xq, qidx), self.rotary(xk, 0)


class SimpleRelativePositionalBias(nn.Module):
    """fairseq/modules/relative_positional_bias.py:13-45: one learned bias per relative offset;
    forward(L) is the L x L Toeplitz matrix with entry (i, j) = rel_pos_bias[max_positions - 1 + j - i]."""

    def __init__(self, max_positions: int):
        super().__init__()
        self.max_positions = max_positions
        self.rel_pos_bias = Parameter(torch.Tensor(2 * max_positions - 1))
        nn.init.normal_(self.rel_pos_bias, mean=0, std=0.02)

    def forward(self, seq_len: int) -> Tensor:
        if seq_len > self.max_positions:
            raise ValueError('Sequence length {} going beyond max length {}'.format(seq_len, self.max_positions))
        pos = torch.arange(seq_len, device=self.rel_pos_bias.device)
        return self.rel_pos_bias[(self.max_positions - 1) + pos[None, :] - pos[:, None]]

    def extra_repr(self) -> str:
        return 'max positions={}'.format(self.max_positions)


class MovingAverageGatedAttention(nn.Module, IncrementalState):
    """Gated attention with a moving-average pre-mixer.  Constructor arguments follow the
    reference (moving_average_gated_attention.py:31-53) for the supported subset; `num_heads`
    (default 1 = the reference) splits q, k and v into heads in the [B, L, Nh, H] layout of the
    fused attention op."""

    def __init__(self, embed_dim, zdim, hdim, ndim, chunk_size=-1, moving_layer='cema', moving_act='rmsnorm',
                 norm_num_groups=None, norm_affine=True, norm_eps=1e-5, max_positions=1024, num_heads=1,
                 efficient_attn=True, rel_pos_bias='rotary', bidirectional=False, attention_activation='softmax',
                 truncation=None, dropout=0.0, attention_dropout=0.0, hidden_dropout=0.0, init_mode='bert'):
        super().__init__()
        self.init_incremental_state()
        self.init_mode = init_mode
        # efficient_attn=False (moving_average_gated_attention.py:66-79) changes one thing: the attention
        # dropout is plain dropout on the softmax weights instead of DropKey inside the softmax
        self._weight_dropout = (not efficient_attn) and attention_activation == 'softmax' and attention_dropout > 0
        # moving_average_gated_attention.py:64-79: element dropout after the output activation and on the
        # two hidden activations, DropKey inside the attention softmax; all three act in training mode only
        self.dropout_p, self.hidden_dropout_p = float(dropout), float(hidden_dropout)
        self.attention_dropout_p = float(attention_dropout)
        if attention_activation not in ('softmax', 'relu2', 'laplace'):
            raise ValueError('Unknown attention activation function: {}'.format(attention_activation))
        self.attention_activation = attention_activation
        if rel_pos_bias not in ('rotary', 'simple'):
            raise ValueError('unknown relative position bias: {}'.format(rel_pos_bias))
        assert zdim % num_heads == 0 and hdim % num_heads == 0 and (zdim // num_heads) % 2 == 0
        self.embed_dim, self.zdim, self.hdim, self.ndim = embed_dim, zdim, hdim, ndim
        self._qk_cache = None
        self._qk_key = None
        self._keep_weights, self._last_weights = False, None
        self.chunk_size = chunk_size
        self.num_heads = num_heads
        self.bidirectional = bidirectional
        # causal layers: the fused causal op; bidirectional layers (moving_average_gated_attention.py:70-75,
        # 84-92): full softmax over every chunk, SequenceNorm, a two-sided moving average
        dropkey = 0.0 if not efficient_attn else attention_dropout
        self.efficient_attn = EfficientAttention(dropout=dropkey, use_causal_mask=not bidirectional, scale=1.0)
        self.attn_softmax = AttentionSoftmax(dropout=dropkey, use_causal_mask=not bidirectional)
        if bidirectional:
            self.norm = SequenceNorm(embed_dim, num_groups=norm_num_groups, eps=norm_eps)
        else:
            self.norm = TimestepNorm(embed_dim, num_groups=norm_num_groups, eps=norm_eps)
        if moving_layer == 'ema':
            self.move = MultiHeadEMA(embed_dim, ndim=ndim, bidirectional=bidirectional, truncation=truncation)
        elif moving_layer == 'cema':
            self.move = MultiHeadComplexEMA(embed_dim, ndim=ndim, bidirectional=bidirectional, truncation=truncation)
        else:
            raise ValueError("Unknown moving type: {}".format(moving_layer))
        assert moving_act in ['rmsnorm', 'silu']
        self.move_act = RMSNorm(embed_dim, norm_affine, norm_eps) if moving_act == 'rmsnorm' else nn.SiLU()
        self.v_proj = nn.Linear(embed_dim, hdim, bias=True)
        self.mx_proj = nn.Linear(embed_dim, zdim + hdim + 2 * embed_dim, bias=True)
        self.h_proj = nn.Linear(hdim, embed_dim, bias=False)
        self.gamma = Parameter(torch.zeros(2, zdim))
        self.beta = Parameter(torch.zeros(2, zdim))
        self.max_positions = max_positions if chunk_size < 0 else chunk_size
        if rel_pos_bias == 'rotary':
            self.rel_pos_bias = RotaryEmbedding(zdim // num_heads, self.max_positions)
        else:
            # moving_average_gated_attention.py:109-110, 212-219: scores = q k^T + bias[j - i], no rotation
            self.rel_pos_bias = SimpleRelativePositionalBias(self.max_positions)
            self.register_buffer("_no_rotation", torch.zeros(zdim // num_heads // 2), persistent=False)
        self.reset_parameters(init_mode)

    def reset_parameters(self, mode='bert'):
        """moving_average_gated_attention.py:128-151."""
        for lin in (self.v_proj, self.mx_proj, self.h_proj):
            if mode == 'bert':
                nn.init.normal_(lin.weight, mean=0.0, std=0.02)
            elif mode == 'he':
                nn.init.kaiming_normal_(lin.weight, a=math.sqrt(5.0))
            elif mode == 'xavier':
                nn.init.xavier_uniform_(lin.weight)
            else:
                raise ValueError('Unknown init mode: {}'.format(mode))
        nn.init.constant_(self.v_proj.bias, 0.0)
        nn.init.constant_(self.mx_proj.bias, 0.0)
        nn.init.constant_(self.gamma, 0.0)
        nn.init.constant_(self.beta, 0.0)

    def forward(self, x: Tensor, padding_mask: Optional[Tensor] = None,
                incremental_state: Optional[Dict[str, Dict[str, Optional[Tensor]]]] = None,
                need_weights: bool = False, attn_mask: Optional[Tensor] = None, before_attn_fn: bool = False):
        """x: [B, L, D] -> ([B, L, D], weights or None); the reference's signature
        (moving_average_gated_attention.py:263-271).  One-sided layers mask the future themselves, so the
        `attn_mask` the reference's decoder hands them (models/mega_lm.py:353-360: always that mask) is not
        looked at; need_weights returns the [B * chunks, (Nh,) C, C] weights of a whole-sequence call."""
        if before_attn_fn:
            raise NotImplementedError("MovingAverageGatedAttention: before_attn_fn (raw scores) is not built")
        if attn_mask is not None and self.bidirectional:
            raise NotImplementedError("MovingAverageGatedAttention: attn_mask on a bidirectional layer is not built")
        if need_weights:
            if incremental_state is not None:
                raise NotImplementedError("MovingAverageGatedAttention: need_weights with incremental state")
            self._keep_weights = True
            try:
                out = self._forward_autograd(x, padding_mask, None)
                w = self._last_weights
            finally:
                self._keep_weights, self._last_weights = False, None
            return out, (w.squeeze(1) if self.num_heads == 1 else w)
        if _training_call(self, x) or (self.training and self._drops()):
            return self._forward_autograd(x, padding_mask, incremental_state), None
        bsz, seq_len, embed_dim = x.size()
        assert embed_dim == self.embed_dim
        saved_state = self._get_input_buffer(incremental_state) if incremental_state is not None else None
        residual = x
        if self.bidirectional:
            assert incremental_state is None, 'a bidirectional layer has no incremental state'
            x = self.norm(x, padding_mask, length_last=False)      # the statistics do not depend on the layout
            mx = None
        else:
            x, mx = norm_then_move(self.norm, self.move, x, padding_mask, incremental_state, out_layout="input")
        v = ops.silu(self.v_proj(x), inplace=True)
        if mx is None:
            mx = self.move(x.transpose(1, 2), padding_mask, incremental_state, out_layout="input")
        mx = mx.transpose(1, 2)
        mx = self.move_act(mx) if isinstance(self.move_act, RMSNorm) else ops.silu(mx, inplace=True)
        base = self.mx_proj(mx)
        u, z, r, hx = torch.split(base, [self.embed_dim, self.zdim, self.hdim, self.embed_dim], dim=-1)
        Nh = self.num_heads
        if saved_state is None:
            # whole chunks, nothing cached: q, k come out of one pass over z (normalise, the two
            # affine maps, rotary with positions restarting in every chunk)
            C = self.chunk_size if 1 < self.chunk_size < seq_len else seq_len
            nc = seq_len // C
            simple = isinstance(self.rel_pos_bias, SimpleRelativePositionalBias)
            qk_gamma, qk_beta, freqs = self._qk_constants(simple)
            q, k = ops.gate_qk_fwd(z, qk_gamma, qk_beta, freqs, Nh, C)
            q4, k4, v4 = q.view(bsz * nc, C, Nh, -1), k.view(bsz * nc, C, Nh, -1), v.reshape(bsz * nc, C, Nh, -1)
            if self.attention_activation != 'softmax':
                attn = self._element_attention(q4, k4, v4, None if padding_mask is None
                                               else padding_mask.reshape(bsz * nc, C))
            elif simple or (self.bidirectional and padding_mask is not None):
                attn = self._padded_attention(q4, k4, v4, None if padding_mask is None or not self.bidirectional
                                              else padding_mask.reshape(bsz * nc, C))
            else:
                attn = self.efficient_attn(q4, k4, v4)
        else:
            attn = self._cached_attention(z, v, saved_state, incremental_state)
        # the gates are applied where their operands are consumed: r on the way into the output
        # projection, u and the residual mix after it
        hp = self.h_proj(ops.gate_mul_fwd(attn.reshape(bsz, seq_len, self.hdim), r))
        return ops.gate_out_fwd(residual, u, hx, hp), None

    def _drops(self) -> bool:
        return self.dropout_p > 0 or self.hidden_dropout_p > 0 or self.attention_dropout_p > 0

    def _qk_constants(self, simple: bool):
        """(gamma + 1, beta, rotation frequencies) in fp32 for the q / k kernel; kept in eval mode
        (dropped by train() and by .to() / .half())."""
        if not self.training:
            key = _tensor_versions(self, self.rel_pos_bias)
            if key != self._qk_key:
                self._qk_cache, self._qk_key = None, key
            if self._qk_cache is not None:
                return self._qk_cache
        with torch.no_grad():
            freqs = self._no_rotation if simple else self.rel_pos_bias.freqs      # zero angles: no rotation
            c = ((self.gamma.float() + 1.0).contiguous(), self.beta.float().contiguous(), freqs.float().contiguous())
        self._qk_cache = None if self.training else c
        return c

    def train(self, mode: bool = True):
        self._qk_cache = None
        return super().train(mode)

    def _apply(self, fn, *args, **kwargs):
        self._qk_cache = None
        return super()._apply(fn, *args, **kwargs)

    def _padded_attention(self, q4: Tensor, k4: Tensor, v4: Tensor, key_padding: Tensor) -> Tensor:
        """Softmax attention outside the fused op (moving_average_gated_attention.py:210-256): the
        learned relative bias is added to the scores, scores of padded keys are -inf except in chunks
        that consist of padding only; library GEMMs around the softmax op (causal for one-sided
        layers)."""
        s = torch.einsum('bqnh,bknh->bnqk', q4, k4)
        if isinstance(self.rel_pos_bias, SimpleRelativePositionalBias):
            s = s + self.rel_pos_bias(q4.size(1)).to(s.dtype)
        if key_padding is not None:
            pad = key_padding.to(torch.bool)
            pad = torch.logical_and(pad, ~pad.all(dim=-1, keepdim=True))
            s = s.masked_fill(pad[:, None, None, :], float('-inf'))
        return torch.einsum('bnqk,bknh->bqnh', self.attn_softmax(s), v4)

    def _element_attention(self, q4: Tensor, k4: Tensor, v4: Tensor, key_padding: Optional[Tensor]) -> Tensor:
        """The element-wise attention of moving_average_gated_attention.py:153-208 (relu2 / laplace in place
        of the softmax): scores scaled by 1 / sqrt(number of keys a query sees), the learned bias added for
        the simple position encoding, weights of padded keys and, in one-sided layers, of future keys set
        to zero after the activation; plain dropout on the weights.  Library GEMMs and torch element-wise
        operations."""
        C = q4.size(1)
        s = torch.einsum('bqnh,bknh->bnqk', q4, k4)
        if not self.bidirectional:
            # the reference's lower-triangular attn_mask (models/mega_lm.py:391-410): query i sees i + 1 keys
            scale = torch.rsqrt(torch.arange(1, C + 1, device=s.device, dtype=torch.float32)).to(s.dtype)[:, None]
        elif key_padding is not None:
            lengths = C - key_padding.to(torch.float32).sum(dim=-1)
            scale = torch.rsqrt(lengths.clamp(min=1.0)).to(s.dtype)[:, None, None, None]
        else:
            scale = 1.0 / math.sqrt(C)
        s = s * scale
        if isinstance(self.rel_pos_bias, SimpleRelativePositionalBias):
            s = s + self.rel_pos_bias(C).to(s.dtype)
        if self.attention_activation == 'relu2':
            w = torch.square(F.relu(s))
        else:
            # fairseq/utils.py:451-457: the logistic approximation of the Laplace attention function
            w = torch.sigmoid((s - 0.707107) * (1.702 / 0.282095))
        if key_padding is not None:
            w = w * (~key_padding.to(torch.bool)).to(w.dtype)[:, None, None, :]
        if not self.bidirectional:
            w = w * torch.ones(C, C, device=w.device, dtype=w.dtype).tril_()
        w = F.dropout(w, self.attention_dropout_p, self.training)
        if self._keep_weights:
            self._last_weights = w
        return torch.einsum('bnqk,bknh->bqnh', w, v4)

    def _forward_autograd(self, x: Tensor, padding_mask: Optional[Tensor], incremental_state) -> Tensor:
        """The same layer with a complete autograd graph (moving_average_gated_attention.py:263-417,
        whole chunks, no cache): TimestepNorm, the moving average and the attention carry their own
        backward operators, the element-wise steps are torch operations."""
        if incremental_state is not None:
            raise NotImplementedError("MovingAverageGatedAttention: incremental state is an inference feature; "
                                      "call it under torch.no_grad()")
        bsz, seq_len, _ = x.size()
        residual = x
        if self.bidirectional:
            x = self.norm(x, padding_mask, length_last=False)
            mx = self.move(x.transpose(1, 2), padding_mask, None, out_layout="input").transpose(1, 2)
        else:
            x, mx = norm_then_move(self.norm, self.move, x, padding_mask, None, out_layout="input")
            mx = mx.transpose(1, 2)
        v = silu(linear(self.v_proj, x))
        mx = self.move_act(mx) if isinstance(self.move_act, RMSNorm) else silu(mx)
        base = linear(self.mx_proj, F.dropout(mx, self.hidden_dropout_p, self.training))
        # the four slices' gradients are written into one buffer by the backward kernels of their consumers
        arena = SplitGrads(base, [self.embed_dim, self.zdim, self.hdim, self.embed_dim])
        u, z, r, hx = SplitFunc.apply(base, arena)
        Nh = self.num_heads
        C = self.chunk_size if 1 < self.chunk_size < seq_len else seq_len
        nc = seq_len // C
        simple = isinstance(self.rel_pos_bias, SimpleRelativePositionalBias)
        v4 = v.reshape(bsz * nc, C, Nh, -1)
        vec = 16 // z.element_size()
        if self.zdim % vec == 0 and self.zdim <= 128 * vec:
            # one kernel forward, one backward (rows of whole 16-byte vectors, at most two per lane)
            freqs = self._no_rotation if simple else self.rel_pos_bias.freqs
            q, k = GateQKFunc.apply(z, self.gamma, self.beta, freqs.detach().float().contiguous(), Nh, C, (arena, 1))
            q4 = q.view(bsz * nc, C, Nh, -1)
            k4 = k.view(bsz * nc, C, Nh, -1)
        else:
            # rows the q / k kernel does not take: torch operations, in fp32 like the kernel (in fp16 the backward of
            # the division by a norm clamped at 1e-5 squares a subnormal and returns NaN), results back in z's type
            zt = F.normalize(z.float(), p=2, dim=-1, eps=1e-5)
            zt = zt.unsqueeze(2) * (self.gamma.float() + 1.0) + self.beta.float()
            q, k = torch.unbind(zt, dim=2)
            q4 = q.reshape(bsz * nc, C, Nh, -1)
            k4 = k.reshape(bsz * nc, C, Nh, -1)
            if not simple:
                q4 = self.rel_pos_bias.rotary(q4.transpose(1, 2), 0).transpose(1, 2)
                k4 = self.rel_pos_bias.rotary(k4.transpose(1, 2), 0).transpose(1, 2)
            q4, k4 = q4.to(z.dtype), k4.to(z.dtype)
        if self.attention_activation != 'softmax':
            attn = self._element_attention(q4, k4, v4, None if padding_mask is None
                                           else padding_mask.reshape(bsz * nc, C))
        elif simple or self._keep_weights or (self.bidirectional and padding_mask is not None) or \
                (self._weight_dropout and self.training):
            s = torch.einsum('bqnh,bknh->bnqk', q4, k4)
            if simple:
                s = s + self.rel_pos_bias(C).to(s.dtype)
            if self.bidirectional and padding_mask is not None:
                pad = padding_mask.reshape(bsz * nc, C).to(torch.bool)
                pad = torch.logical_and(pad, ~pad.all(dim=-1, keepdim=True))
                s = s.masked_fill(pad[:, None, None, :], float('-inf'))
            w = self.attn_softmax(s)
            if self._weight_dropout:
                w = F.dropout(w, self.attention_dropout_p, self.training)
            if self._keep_weights:
                self._last_weights = w
            attn = torch.einsum('bnqk,bknh->bqnh', w, v4)
        else:
            attn = self.efficient_attn(q4, k4, v4)
        gated = GateMulFunc.apply(attn.reshape(bsz, seq_len, self.hdim), r, (arena, 2))
        hp = linear(self.h_proj, F.dropout(gated, self.hidden_dropout_p, self.training))
        if self.training and self.dropout_p > 0:
            # the output dropout sits between the activation and the residual mix
            # (moving_average_gated_attention.py:409-412), so the fused gate is taken apart
            h = F.dropout(F.silu(hx + hp), self.dropout_p, True)
            return torch.addcmul(residual, torch.sigmoid(u), h - residual)
        return GateOutFunc.apply(residual, u, hx, hp, (arena, 0, 3))

    def _cached_attention(self, z: Tensor, v: Tensor, saved_state, incremental_state) -> Tensor:
        """Attention with the partial-chunk key / value cache
        (moving_average_gated_attention.py:332-372): keys are cached before the rotation, so the
        whole context is rotated again at every call."""
        simple = isinstance(self.rel_pos_bias, SimpleRelativePositionalBias)
        bsz, seq_len = z.shape[:2]
        Nh = self.num_heads
        z = F.normalize(z, p=2, dim=-1, eps=1e-5)
        z = z.unsqueeze(2) * (self.gamma + 1.0) + self.beta
        q, k = torch.unbind(z, dim=2)
        if "prev_key" in saved_state:
            k = torch.cat([saved_state["prev_key"], k], dim=1)
            v = torch.cat([saved_state["prev_value"], v], dim=1)
        if self.chunk_size < 0 or k.size(1) % self.chunk_size != 0:
            saved_state["prev_key"], saved_state["prev_value"] = k, v
        else:
            saved_state.pop("prev_key", None)
            saved_state.pop("prev_value", None)
        self._set_input_buffer(incremental_state, saved_state)
        ctx_len = k.size(1)
        if 1 < self.chunk_size < seq_len:
            nc = seq_len // self.chunk_size
            q = q.reshape(bsz * nc, self.chunk_size, self.zdim)
        if 1 < self.chunk_size < ctx_len:
            nc = ctx_len // self.chunk_size
            k = k.reshape(bsz * nc, self.chunk_size, self.zdim)
            v = v.reshape(bsz * nc, self.chunk_size, self.hdim)
        # [B', C, Nh, H]; rotary positions run along C per head and restart in every chunk
        q4 = q.reshape(q.size(0), q.size(1), Nh, -1)
        k4 = k.reshape(k.size(0), k.size(1), Nh, -1)
        v4 = v.reshape(v.size(0), v.size(1), Nh, -1)
        qidx = k4.size(1) - q4.size(1)
        if not simple:
            q4 = self.rel_pos_bias.rotary(q4.transpose(1, 2), qidx).transpose(1, 2)
            k4 = self.rel_pos_bias.rotary(k4.transpose(1, 2), 0).transpose(1, 2)
            if q4.size(1) == k4.size(1) and self.attention_activation == 'softmax':
                return self.efficient_attn(q4, k4, v4)
        # new queries at positions qidx .. ctx-1 against the cached context (a whole chunk when qidx = 0):
        # right-aligned causal weights; the bias rows are those of the query positions
        # (moving_average_gated_attention.py:170-178, 212-221: `bias[-1:]` for one new token)
        ctx = k4.size(1)
        s = torch.einsum('bqnh,bknh->bnqk', q4.float(), k4.float())
        if self.attention_activation != 'softmax':
            s = s * torch.rsqrt(torch.arange(qidx + 1, ctx + 1, device=s.device, dtype=torch.float32))[:, None]
        if simple:
            s = s + self.rel_pos_bias(ctx)[qidx:].float()
        if self.attention_activation == 'softmax':
            w = ops.attention_softmax_fwd(s.to(q4.dtype), 0.0, True).float()
        else:
            w = torch.square(F.relu(s)) if self.attention_activation == 'relu2' else \
                torch.sigmoid((s - 0.707107) * (1.702 / 0.282095))
            w = w * torch.ones(ctx, ctx, device=w.device, dtype=w.dtype).tril_()[qidx:]
        return torch.einsum('bnqk,bknh->bqnh', w, v4.float()).to(v4.dtype)

    def _get_input_buffer(self, incremental_state):
        result = self.get_incremental_state(incremental_state, "attn_state")
        return result if result is not None else {}

    def _set_input_buffer(self, incremental_state, buffer):
        return self.set_incremental_state(incremental_state, "attn_state", buffer)

    def reorder_incremental_state(self, incremental_state, new_order: Tensor):
        """The cached keys / values follow a beam reordering
        (moving_average_gated_attention.py:430-443); the norm and the moving average reorder their
        own entries."""
        input_buffer = self._get_input_buffer(incremental_state)
        for name in list(input_buffer.keys()):
            if input_buffer[name] is not None:
                input_buffer[name] = input_buffer[name].index_select(0, new_order)
        return self._set_input_buffer(incremental_state, input_buffer)

    def extra_repr(self) -> str:
        return 'edim={}, zdim={}, hdim={}, ndim={}, chunk={}, heads={}, bidir={}'.format(
            self.embed_dim, self.zdim, self.hdim, self.ndim, self.chunk_size, self.num_heads, self.bidirectional)


class Mega2Layer(nn.Module):
    """One Mega2 block of the north-star configuration: gated attention (TimestepNorm -> CEMA ->
    chunked causal attention) followed by a pre-normalised SwiGLU FFN with a residual."""

    def __init__(self, embed_dim, zdim, hdim, ndim, ffn_dim, chunk_size, norm_num_groups=16, num_heads=1,
                 moving_act='silu'):
        super().__init__()
        self.attn = MovingAverageGatedAttention(embed_dim, zdim, hdim, ndim, chunk_size=chunk_size,
                                                norm_num_groups=norm_num_groups, num_heads=num_heads,
                                                moving_act=moving_act)
        self.ffn_norm = TimestepNorm(embed_dim, num_groups=norm_num_groups)
        self.ffn = SwiGLU(embed_dim, ffn_dim, bias=False)
        for lin in (self.ffn.w1, self.ffn.w2, self.ffn.w3):
            nn.init.normal_(lin.weight, mean=0.0, std=0.02)

    def forward(self, x: Tensor, padding_mask: Optional[Tensor] = None, incremental_state=None) -> Tensor:
        x, _ = self.attn(x, padding_mask, incremental_state)
        # x is this layer's own intermediate: the feed-forward block may accumulate into it
        return self.ffn(self.ffn_norm(x, padding_mask, incremental_state), residual=x, consume_residual=True)


def _arg(args, name, default):
    return getattr(args, name, default)


class MegaDecoderLayer(nn.Module):
    """fairseq/modules/mega_layer.py:81-202 without the cross attention (a language-model layer):
    `mega_layer` (causal MovingAverageGatedAttention) followed by `nffn`
    (NormalizedFeedForwardNetwork) when args.decoder_ffn_embed_dim > 0.  `args` is the reference's
    namespace (fairseq/models/mega_lm.py:51-121); submodule names, and therefore state-dict keys,
    are the reference's."""

    def __init__(self, args, no_cross_attention: bool = True, layer_scale: Optional[float] = None):
        super().__init__()
        if not no_cross_attention:
            raise NotImplementedError("MegaDecoderLayer: the gated cross attention is not built")
        self.embed_dim = args.decoder_embed_dim
        trunc = _arg(args, 'truncation_length', 0)
        self.mega_layer = MovingAverageGatedAttention(
            self.embed_dim, args.decoder_z_dim, args.decoder_hidden_dim, args.decoder_n_dim,
            chunk_size=_arg(args, 'decoder_chunk_size', -1), moving_layer=_arg(args, 'moving_layer', 'cema'),
            moving_act=_arg(args, 'moving_act', 'rmsnorm'), norm_num_groups=_arg(args, 'norm_num_groups', None),
            norm_affine=not _arg(args, 'no_affine_norm', False), norm_eps=_arg(args, 'norm_eps', 1e-5),
            max_positions=_arg(args, 'max_target_positions', 1024), num_heads=_arg(args, 'num_heads', 1),
            efficient_attn=_arg(args, 'efficient_attention', True), rel_pos_bias=_arg(args, 'rel_pos_bias', 'rotary'),
            bidirectional=False, attention_activation=_arg(args, 'attention_activation_fn', 'softmax'),
            truncation=trunc if trunc and trunc > 0 else None, dropout=_arg(args, 'dropout', 0.0),
            attention_dropout=_arg(args, 'attention_dropout', 0.0), hidden_dropout=_arg(args, 'hidden_dropout', 0.0),
            init_mode=_arg(args, 'init_mode', 'bert'))
        self.cross_attn = None
        if _arg(args, 'decoder_ffn_embed_dim', 0) > 0:
            self.nffn = NormalizedFeedForwardNetwork(
                self.embed_dim, args.decoder_ffn_embed_dim, dropout=_arg(args, 'dropout', 0.0),
                hidden_dropout=_arg(args, 'activation_dropout', 0.0), norm_type=_arg(args, 'norm_type', 'layernorm'),
                norm_affine=not _arg(args, 'no_affine_norm', False), norm_eps=_arg(args, 'norm_eps', 1e-5),
                layer_scale=layer_scale, init_mode=_arg(args, 'init_mode', 'bert'))
        else:
            self.nffn = None

    def forward(self, x: Tensor, encoder_out=None, encoder_padding_mask=None, incremental_state=None, attn_mask=None,
                decoder_padding_mask: Optional[Tensor] = None, need_attn: bool = False):
        """x: [B, L, D] -> (x, None, None), the reference's return triple."""
        x, attn = self.mega_layer(x, decoder_padding_mask, incremental_state, need_weights=need_attn)
        if self.nffn is not None:
            x = self.nffn(x, consume_input=True)      # x is this layer's own intermediate
        return x, attn, None


class MegaEncoderLayer(nn.Module):
    """fairseq/modules/mega_layer.py:11-78: bidirectional `mega_layer` followed by `nffn`."""

    def __init__(self, args, layer_scale: Optional[float] = None):
        super().__init__()
        self.embed_dim = args.encoder_embed_dim
        trunc = _arg(args, 'truncation_length', 0)
        self.mega_layer = MovingAverageGatedAttention(
            self.embed_dim, args.encoder_z_dim, args.encoder_hidden_dim, args.encoder_n_dim,
            chunk_size=_arg(args, 'encoder_chunk_size', -1), moving_layer=_arg(args, 'moving_layer', 'cema'),
            moving_act=_arg(args, 'moving_act', 'rmsnorm'), norm_num_groups=_arg(args, 'norm_num_groups', None),
            norm_affine=not _arg(args, 'no_affine_norm', False), norm_eps=_arg(args, 'norm_eps', 1e-5),
            max_positions=_arg(args, 'max_source_positions', 1024), num_heads=_arg(args, 'num_heads', 1),
            efficient_attn=_arg(args, 'efficient_attention', True), rel_pos_bias=_arg(args, 'rel_pos_bias', 'rotary'),
            bidirectional=True, attention_activation=_arg(args, 'attention_activation_fn', 'softmax'),
            truncation=trunc if trunc and trunc > 0 else None, dropout=_arg(args, 'dropout', 0.0),
            attention_dropout=_arg(args, 'attention_dropout', 0.0), hidden_dropout=_arg(args, 'hidden_dropout', 0.0),
            init_mode=_arg(args, 'init_mode', 'bert'))
        if _arg(args, 'encoder_ffn_embed_dim', 0) > 0:
            self.nffn = NormalizedFeedForwardNetwork(
                self.embed_dim, args.encoder_ffn_embed_dim, dropout=_arg(args, 'dropout', 0.0),
                hidden_dropout=_arg(args, 'activation_dropout', 0.0), norm_type=_arg(args, 'norm_type', 'layernorm'),
                norm_affine=not _arg(args, 'no_affine_norm', False), norm_eps=_arg(args, 'norm_eps', 1e-5),
                layer_scale=layer_scale, init_mode=_arg(args, 'init_mode', 'bert'))
        else:
            self.nffn = None

    def forward(self, x: Tensor, encoder_padding_mask: Optional[Tensor] = None) -> Tensor:
        x, _ = self.mega_layer(x, encoder_padding_mask)
        if self.nffn is not None:
            x = self.nffn(x, consume_input=True)      # x is this layer's own intermediate
        return x


def streamed_forward(layers, x: Tensor, chunk_size: int, padding_mask: Optional[Tensor] = None) -> Tensor:
    """Run a stack of decoder layers over x [B, L, D] chunk by chunk with carried state, the way the
    reference's validation streams documents (fairseq_cli/train.py:406-417: one incremental-state
    dictionary per document, consecutive slices of `chunk_size` tokens).  Equals the one-shot result
    for causal layers."""
    incremental_states: Dict[str, Dict[str, Optional[Tensor]]] = {}
    outs = []
    for a in range(0, x.size(1), chunk_size):
        h = x[:, a:a + chunk_size]
        pm = None if padding_mask is None else padding_mask[:, a:a + chunk_size]
        for layer in layers:
            out = layer(h, incremental_state=incremental_states, decoder_padding_mask=pm)
            h = out[0] if isinstance(out, tuple) else out
        outs.append(h)
    if x.is_cuda:
        ops.check_lookback("streamed_forward")
    return torch.cat(outs, dim=1)
