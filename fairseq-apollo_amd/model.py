"""Decoder-only Mega language-model body: token embedding -> MegaDecoderLayer stack ->
TimestepNorm -> output projection, with the reference's submodule names so that the `decoder.*`
entries of a reference `mega_lm` checkpoint load with `load_state_dict`
(fairseq/models/mega_lm.py:188-300, MegaDecoderNoCrossAttn).  Dictionary handling, adaptive softmax
and the fairseq task / trainer plumbing are not part of it.
"""
from __future__ import annotations

import math
from collections import OrderedDict
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from . import ops
from .layers import MegaDecoderLayer, _arg
from .modules import TimestepNorm


class MegaDecoderNoCrossAttn(nn.Module):
    """fairseq/models/mega_lm.py:188-412.  `args` is the reference's namespace (decoder_embed_dim,
    decoder_layers, decoder_z_dim, decoder_hidden_dim, decoder_n_dim, decoder_ffn_embed_dim,
    decoder_chunk_size, norm_num_groups, norm_eps, layer_scale, share_decoder_input_output_embed,
    no_scale_embedding, representation_dim, ...); `embed_tokens` an nn.Embedding with padding_idx."""

    def __init__(self, args, vocab_size: int, embed_tokens: nn.Embedding):
        super().__init__()
        self.args = args
        self.register_buffer("version", torch.Tensor([3]))
        embed_dim = args.decoder_embed_dim
        self.embed_dim = embed_dim
        self.share_input_output_embed = _arg(args, 'share_decoder_input_output_embed', False)
        self.padding_idx = embed_tokens.padding_idx
        self.max_target_positions = _arg(args, 'max_target_positions', 1024)
        self.chunk_size = _arg(args, 'decoder_chunk_size', -1)
        self.embed_tokens = embed_tokens
        self.embed_scale = None if _arg(args, 'no_scale_embedding', False) else math.sqrt(embed_dim)
        self.embedding_dropout = nn.Dropout(_arg(args, 'dropout', 0.0))
        depth = args.decoder_layers
        lsw = [0.1 * (0.5 ** i) for i in range(depth)] if _arg(args, 'layer_scale', False) else [None] * depth
        self.layers = nn.ModuleList([MegaDecoderLayer(args, no_cross_attention=True, layer_scale=lsw[i])
                                     for i in range(depth)])
        self.num_layers = depth
        self.final_norm = TimestepNorm(embed_dim, num_groups=_arg(args, 'norm_num_groups', None),
                                       eps=_arg(args, 'norm_eps', 1e-5))
        rep = _arg(args, 'representation_dim', None)
        if rep is not None:
            self.num_features = rep
            self.pre_logits = nn.Sequential(OrderedDict([('fc', nn.Linear(embed_dim, rep, bias=True)),
                                                         ('act', nn.SiLU()),
                                                         ('dropout', nn.Dropout(_arg(args, 'dropout', 0.0)))]))
        else:
            self.num_features = embed_dim
            self.pre_logits = nn.Identity()
        if _arg(args, 'adaptive_softmax_cutoff', None) is not None:
            raise NotImplementedError("MegaDecoderNoCrossAttn: adaptive softmax is not built")
        if self.share_input_output_embed:
            self.output_projection = nn.Linear(embed_tokens.weight.shape[1], embed_tokens.weight.shape[0], bias=False)
            self.output_projection.weight = embed_tokens.weight
        else:
            self.output_projection = nn.Linear(self.num_features, vocab_size, bias=False)
            nn.init.normal_(self.output_projection.weight, mean=0, std=1.0 / math.sqrt(self.num_features))

    def forward(self, prev_output_tokens: Tensor,
                incremental_state: Optional[Dict[str, Dict[str, Optional[Tensor]]]] = None,
                features_only: bool = False) -> Tuple[Tensor, Dict[str, List[Tensor]]]:
        x, extra = self.extract_features(prev_output_tokens, incremental_state)
        if not features_only:
            x = self.output_layer(x)
        return x, extra

    def output_layer(self, features: Tensor) -> Tensor:
        """Project features to the vocabulary (mega_lm.py:379-385)."""
        return self.output_projection(features)

    def max_positions(self) -> int:
        """Longest sequence the decoder is configured for (mega_lm.py:387-389)."""
        return self.max_target_positions

    def extract_features(self, prev_output_tokens: Tensor, incremental_state=None):
        """mega_lm.py:313-386: tokens are padded up to a whole number of chunks, padded positions are
        masked in every layer and zeroed at the end."""
        bsz, seq_len = prev_output_tokens.size()
        num_paddings = 0
        if seq_len > self.chunk_size > 0 and seq_len % self.chunk_size != 0:
            num_paddings = math.ceil(seq_len / self.chunk_size) * self.chunk_size - seq_len
            prev_output_tokens = F.pad(prev_output_tokens, (0, num_paddings), value=self.padding_idx)
        x = self.embed_tokens(prev_output_tokens)
        if self.embed_scale is not None:
            x = self.embed_scale * x
        decoder_padding_mask = prev_output_tokens.eq(self.padding_idx) if self.padding_idx is not None else None
        if decoder_padding_mask is not None and not decoder_padding_mask.any():
            decoder_padding_mask = None
        x = self.embedding_dropout(x)
        inner_states: List[Tensor] = [x]
        for layer in self.layers:
            x, _, _ = layer(x, incremental_state=incremental_state, decoder_padding_mask=decoder_padding_mask)
            inner_states.append(x)
        x = self.final_norm(x, padding_mask=decoder_padding_mask, incremental_state=incremental_state)
        x = self.pre_logits(x)
        if decoder_padding_mask is not None:
            x = x * (~decoder_padding_mask).to(x.dtype).unsqueeze(-1)
        if num_paddings > 0:
            x = x[:, :seq_len]
        return x, {"inner_states": inner_states}

    def reorder_incremental_state(self, incremental_state, new_order: Tensor) -> None:
        """Beam search keeps a subset / permutation of the streams: every module that carries state
        reorders its own entries (fairseq/models/fairseq_incremental_decoder.py:82-96 walks the
        module tree the same way)."""
        for module in self.modules():
            if module is not self and hasattr(module, 'reorder_incremental_state'):
                module.reorder_incremental_state(incremental_state, new_order)

    def streamed(self, tokens: Tensor, chunk_size: Optional[int] = None) -> Tensor:
        """Logits of a document evaluated slice by slice with one incremental-state dictionary
        (fairseq_cli/train.py:406-417)."""
        chunk = chunk_size or self.chunk_size
        state: Dict[str, Dict[str, Optional[Tensor]]] = {}
        outs = [self(tokens[:, a:a + chunk], incremental_state=state)[0] for a in range(0, tokens.size(1), chunk)]
        return torch.cat(outs, dim=1)


def validate_stream(model: MegaDecoderNoCrossAttn, src_tokens: Tensor, target: Tensor, pad_idx: int,
                    chunk_size: Optional[int] = None) -> Tuple[Tensor, Tensor]:
    """Chunk-wise evaluation of one batch of documents the way the reference validates a Mega language
    model (fairseq_cli/train.py:395-417): consecutive slices of `chunk_size` tokens go through the
    model with one incremental-state dictionary per batch, and every slice adds its summed negative
    log-likelihood and its count of non-padding targets.  -> (nll_sum, ntokens); perplexity is
    exp(nll_sum / ntokens) (base e)."""
    chunk = chunk_size or model.chunk_size
    if chunk <= 0:
        chunk = src_tokens.size(1)
    state: Dict[str, Dict[str, Optional[Tensor]]] = {}
    nll = torch.zeros((), dtype=torch.float64, device=src_tokens.device)
    ntok = torch.zeros((), dtype=torch.int64, device=src_tokens.device)
    with torch.no_grad():
        for a in range(0, src_tokens.size(1), chunk):
            logits = model(src_tokens[:, a:a + chunk], incremental_state=state)[0]
            tgt = target[:, a:a + chunk]
            lp = F.log_softmax(logits.float(), dim=-1)
            nll += F.nll_loss(lp.reshape(-1, lp.size(-1)), tgt.reshape(-1), ignore_index=pad_idx,
                              reduction='sum').double()
            ntok += tgt.ne(pad_idx).sum()
    if src_tokens.is_cuda:
        ops.check_lookback("validate_stream")
    return nll, ntok
