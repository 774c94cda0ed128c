"""Logits of the decoder-only language model (MegaDecoderNoCrossAttn, fairseq/models/mega_lm.py:188-412) against the
fp64 oracle of the whole model (oracle.mega_lm_decoder: embedding, the layers, the final TimestepNorm, pre_logits, the
projection), for the argument sets of tests/golden/mega_lm_state_dict.json: one shot, for a length that is not a whole
number of chunks, and streamed slice by slice with one incremental-state dictionary.  The oracle's inputs are taken from
the model's state dict by name, the way a reference checkpoint would provide them, and turned into moving-average
coefficients by the oracle's own restatement, not by the package."""
import json
import os
import types

import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import rel_err
from gpu_util import DEV, host
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu

TABLE = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "mega_lm_state_dict.json")))


def _build(name, seed):
    a = dict(TABLE[name]["args"])
    vocab = a.pop("vocab")
    args = types.SimpleNamespace(dropout=0.0, attention_dropout=0.0, hidden_dropout=0.0, activation_dropout=0.0,
                                 truncation_length=None, init_mode="bert", adaptive_softmax_cutoff=None, **a)
    torch.manual_seed(seed)
    emb = torch.nn.Embedding(vocab, args.decoder_embed_dim, padding_idx=1)
    model = M.MegaDecoderNoCrossAttn(args, vocab, emb)
    with torch.no_grad():                       # away from the initial values, where several terms vanish
        for k, v in model.state_dict().items():
            if k.endswith(("norm.weight", "norm.bias", "move_act.weight", ".gamma", ".beta", "rel_pos_bias.rel_pos_bias",
                           "fc1.bias", "v_proj.bias", "mx_proj.bias")) and "move." not in k:
                v.normal_(0, 0.1)
            elif k.endswith(("v_proj.weight", "mx_proj.weight", "h_proj.weight", "fc1.weight", "fc2.weight", "fc.weight")):
                v.normal_(0, 0.12)
        model.embed_tokens.weight[1].zero_()
    return model.to(DEV).eval(), args, vocab


def _oracle_params(sd, args):
    g = lambda k: sd[k].detach().double().cpu().numpy()
    layers = []
    for i in range(args.decoder_layers):
        m = f"layers.{i}.mega_layer."
        if args.moving_layer == "cema":
            p, q, eg = O.ema_coeffs_complex(g(m + "move.alpha"), g(m + "move.delta"), g(m + "move.theta"),
                                            g(m + "move.gamma"))
        else:
            p, q, eg = O.ema_coeffs_real(g(m + "move.alpha"), g(m + "move.delta"), g(m + "move.beta"),
                                         g(m + "move.gamma"))
        A = dict(norm_weight=g(m + "norm.weight"), norm_bias=g(m + "norm.bias"), p=p, q=q, ema_gamma=eg,
                 omega=g(m + "move.omega").reshape(-1), v_w=g(m + "v_proj.weight"), v_b=g(m + "v_proj.bias"),
                 mx_w=g(m + "mx_proj.weight"), mx_b=g(m + "mx_proj.bias"), h_w=g(m + "h_proj.weight"),
                 gamma=g(m + "gamma"), beta=g(m + "beta"))
        if m + "move_act.weight" in sd:
            A["rms_weight"] = g(m + "move_act.weight")
        if m + "rel_pos_bias.rel_pos_bias" in sd:
            A["simple_bias"] = g(m + "rel_pos_bias.rel_pos_bias")
        F_ = None
        n = f"layers.{i}.nffn."
        if n + "fc1.weight" in sd:
            F_ = dict(norm_weight=g(n + "norm.weight") if n + "norm.weight" in sd else None,
                      norm_bias=g(n + "norm.bias") if n + "norm.bias" in sd else None,
                      fc1_w=g(n + "fc1.weight"), fc1_b=g(n + "fc1.bias"), fc2_w=g(n + "fc2.weight"),
                      layerscale=g(n + "layerscale_weight") if n + "layerscale_weight" in sd else None)
        layers.append(dict(attn=A, ffn=F_))
    P = dict(embed=g("embed_tokens.weight"), layers=layers, final_weight=g("final_norm.weight"),
             final_bias=g("final_norm.bias"), out_w=g("output_projection.weight"))
    if "pre_logits.fc.weight" in sd:
        P["pre_w"], P["pre_b"] = g("pre_logits.fc.weight"), g("pre_logits.fc.bias")
    return P


def _oracle(model, args, tokens):
    chunk = args.decoder_chunk_size
    return O.mega_lm_decoder(host(tokens), _oracle_params(model.state_dict(), args), chunk, 1, args.norm_num_groups,
                             None if args.no_scale_embedding else float(np.sqrt(args.decoder_embed_dim)),
                             moving_act="rmsnorm", norm_type=args.norm_type, eps=args.norm_eps,
                             simple_bias=args.rel_pos_bias == "simple",
                             attention_activation=args.attention_activation_fn)


@pytest.mark.parametrize("name,T,T_odd", [("cema_rotary_rmsnorm_layerscale_tied", 128, 80),
                                          ("ema_simple_layernorm_representation", 64, 40),
                                          ("cema_no_ffn_no_affine", 48, 33)])
def test_logits_one_shot_against_the_model_oracle(name, T, T_odd):
    model, args, vocab = _build(name, 5)
    tokens = torch.randint(2, vocab, (2, T), device=DEV)
    for t in (T, T_odd):                                  # T_odd: padded up to whole chunks inside, cut back
        with torch.no_grad():
            got = model(tokens[:, :t])[0]
        want = _oracle(model, args, tokens[:, :t])
        assert got.shape == want.shape == (2, t, vocab)
        assert rel_err(host(got), want) < 5e-4, (name, t, rel_err(host(got), want))
    assert M.ops.timestep_norm_status() == 0


@pytest.mark.parametrize("name,T", [("cema_rotary_rmsnorm_layerscale_tied", 112),
                                    ("ema_simple_layernorm_representation", 56)])
def test_logits_streamed_against_the_model_oracle(name, T):
    """Slices of one chunk (the last one shorter) with one incremental-state dictionary, the reference's validation
    loop (fairseq_cli/train.py:406-417): every slice continues the norms' statistics and the moving average's state
    and attends inside itself, which is what the one-shot forward computes chunk by chunk.  T is a whole number of
    chunks plus a remainder; the one-shot oracle of the first whole chunks and of the remainder's positions agree with
    the stream except for the one-shot path's end padding, which only follows the compared positions."""
    model, args, vocab = _build(name, 6)
    tokens = torch.randint(2, vocab, (3, T), device=DEV)
    with torch.no_grad():
        got = model.streamed(tokens)
    want = _oracle(model, args, tokens)
    assert rel_err(host(got), want) < 5e-4, (name, rel_err(host(got), want))
    assert M.ops.timestep_norm_status() == 0
