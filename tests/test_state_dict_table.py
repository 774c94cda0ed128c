"""Checkpoint compatibility of the decoder-only Mega language model: for every argument set of
tests/golden/mega_lm_state_dict.json (every `decoder.*` entry the reference's MegaLanguageModel creates, read off
fairseq/models/mega_lm.py:198-266 and the constructors below it by tests/golden/make_state_dict_table.py) the model
built here holds exactly those entries -- same names, shapes and dtypes, nothing missing, nothing extra -- so that
`load_state_dict(strict=True)` takes a reference checkpoint's decoder as it is.  CPU only: nothing is computed."""
import json
import os
import types

import pytest
import torch

import fairseq_apollo_amd as M

TABLE = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "mega_lm_state_dict.json")))


@pytest.mark.parametrize("name", sorted(TABLE))
def test_decoder_state_dict_equals_the_reference_table(name):
    a = dict(TABLE[name]["args"])
    vocab = a.pop("vocab")
    args = types.SimpleNamespace(dropout=0.0, attention_dropout=0.0, hidden_dropout=0.0, activation_dropout=0.0,
                                 truncation_length=None, init_mode="bert", adaptive_softmax_cutoff=None, **a)
    emb = torch.nn.Embedding(vocab, args.decoder_embed_dim, padding_idx=1)
    model = M.MegaDecoderNoCrossAttn(args, vocab, emb)
    got = {"decoder." + k: (list(v.shape), str(v.dtype).replace("torch.", "")) for k, v in model.state_dict().items()}
    want = {e["name"]: (e["shape"], e["dtype"]) for e in TABLE[name]["entries"]}
    assert sorted(set(want) - set(got)) == [], "entries of a reference checkpoint this model lacks"
    assert sorted(set(got) - set(want)) == [], "entries this model holds that a reference checkpoint lacks"
    assert got == want
    # a state dict with the table's names and shapes loads strictly
    sd = {k[len("decoder."):]: torch.zeros(s, dtype=getattr(torch, d)) for k, (s, d) in want.items()}
    model.load_state_dict(sd, strict=True)
    if args.share_decoder_input_output_embed:
        assert model.output_projection.weight is model.embed_tokens.weight


def test_norm_weights_are_stored_as_offsets_from_one():
    """A reference checkpoint stores `weight - 1` for TimestepNorm, RMSNorm and LayerNorm (zero-initialised, `+ 1.0` in
    the forward: norm_layer/timestep_norm.py:96,118; norm_layer/layer_norm.py:24-33, 47-56, 105-111): fresh modules hold
    zeros there."""
    for mod in (M.TimestepNorm(8, 2), M.RMSNorm(8), M.layers.LayerNorm(8)):
        assert torch.count_nonzero(mod.weight) == 0
    ln = M.layers.LayerNorm(8)
    x = torch.randn(3, 8)
    assert torch.allclose(ln(x), torch.nn.functional.layer_norm(x, (8,)), atol=1e-6)
    with torch.no_grad():
        ln.weight.fill_(1.0)
    assert torch.allclose(ln(x), 2 * torch.nn.functional.layer_norm(x, (8,)), atol=1e-6)
