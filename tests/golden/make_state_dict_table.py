"""Writes tests/golden/mega_lm_state_dict.json: every `decoder.*` state-dict entry (name -> shape, dtype) that the
reference's MegaLanguageModel creates for a few stated argument sets.

    python tests/golden/make_state_dict_table.py

The reference model cannot be constructed here (importing fairseq needs its CUDA extension), so the table is read off
the constructors, registration by registration; every entry names the line that creates it (paths relative to the
reference tree).  nn.Module.state_dict lists, per module, parameters, then persistent buffers, then the submodules in
the order they were assigned; the order is kept so that the fixture reads like a real checkpoint, but the test
compares names, shapes and dtypes as a mapping.
"""
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))

ARG_SETS = {
    # the Mega2 recipe's shape in small: complex EMA, rotary, RMSNorm feed-forward, layer scale, tied embeddings
    "cema_rotary_rmsnorm_layerscale_tied": dict(
        vocab=100, decoder_embed_dim=64, decoder_layers=2, decoder_z_dim=16, decoder_hidden_dim=96, decoder_n_dim=4,
        decoder_ffn_embed_dim=128, decoder_chunk_size=32, norm_num_groups=4, norm_eps=1e-5, layer_scale=True,
        share_decoder_input_output_embed=True, no_scale_embedding=False, representation_dim=None,
        moving_layer="cema", rel_pos_bias="rotary", attention_activation_fn="softmax", norm_type="rmsnorm",
        no_affine_norm=False, max_target_positions=1024, efficient_attention=True),
    # real EMA, learned relative bias, LayerNorm feed-forward, own output projection, a representation layer
    "ema_simple_layernorm_representation": dict(
        vocab=60, decoder_embed_dim=32, decoder_layers=1, decoder_z_dim=8, decoder_hidden_dim=48, decoder_n_dim=2,
        decoder_ffn_embed_dim=64, decoder_chunk_size=16, norm_num_groups=2, norm_eps=1e-5, layer_scale=False,
        share_decoder_input_output_embed=False, no_scale_embedding=True, representation_dim=40,
        moving_layer="ema", rel_pos_bias="simple", attention_activation_fn="laplace", norm_type="layernorm",
        no_affine_norm=False, max_target_positions=128, efficient_attention=False),
    # no feed-forward block, no affine in the RMSNorm of the moving average, whole-sequence attention
    "cema_no_ffn_no_affine": dict(
        vocab=30, decoder_embed_dim=16, decoder_layers=3, decoder_z_dim=4, decoder_hidden_dim=24, decoder_n_dim=8,
        decoder_ffn_embed_dim=0, decoder_chunk_size=-1, norm_num_groups=8, norm_eps=1e-5, layer_scale=False,
        share_decoder_input_output_embed=False, no_scale_embedding=False, representation_dim=None,
        moving_layer="cema", rel_pos_bias="simple", attention_activation_fn="softmax", norm_type="rmsnorm",
        no_affine_norm=True, max_target_positions=64, efficient_attention=False),
}


def timestep_norm(prefix, D, G):
    """fairseq/modules/norm_layer/timestep_norm.py:71-97: weight, bias parameters; prior_count (int64 scalar),
    prior_mean, prior_logv buffers (prior_count = 0 in every Mega recipe, so they are buffers, :88-94)."""
    return [(prefix + "weight", [D], "float32"), (prefix + "bias", [D], "float32"),
            (prefix + "prior_count", [], "int64"), (prefix + "prior_mean", [G], "float32"),
            (prefix + "prior_logv", [G], "float32")]


def layer_entries(prefix, a, layer_scale):
    D, S, E, N = a["decoder_embed_dim"], a["decoder_z_dim"], a["decoder_hidden_dim"], a["decoder_n_dim"]
    out = []
    m = prefix + "mega_layer."
    # MovingAverageGatedAttention.__init__, fairseq/modules/moving_average_gated_attention.py:32-117, called without
    # moving_act from mega_layer.py:105-126, i.e. with the default 'rmsnorm' (:45)
    out += [(m + "gamma", [2, S], "float32"), (m + "beta", [2, S], "float32")]                       # :103-104
    out += timestep_norm(m + "norm.", D, a["norm_num_groups"])                                         # :84
    if a["moving_layer"] == "cema":      # complex_exponential_moving_average.py:36-41
        out += [(m + "move.alpha", [D, N, 1], "float32"), (m + "move.delta", [D, N, 1], "float32"),
                (m + "move.theta", [D, 1, 1], "float32"), (m + "move.gamma", [D, N, 2], "float32"),
                (m + "move.omega", [D, 1], "float32")]
    else:                                # exponential_moving_average.py:34-38
        out += [(m + "move.alpha", [D, N, 1], "float32"), (m + "move.delta", [D, N, 1], "float32"),
                (m + "move.beta", [D, N, 1], "float32"), (m + "move.gamma", [D, N], "float32"),
                (m + "move.omega", [D], "float32")]
    if not a["no_affine_norm"]:          # :95 RMSNorm -> FusedRMSNorm: one `weight` (norm_layer/layer_norm.py:41-50)
        out += [(m + "move_act.weight", [D], "float32")]
    out += [(m + "v_proj.weight", [E, D], "float32"), (m + "v_proj.bias", [E], "float32"),             # :99
            (m + "mx_proj.weight", [S + E + 2 * D, D], "float32"), (m + "mx_proj.bias", [S + E + 2 * D], "float32"),  # :100
            (m + "h_proj.weight", [D, E], "float32")]                                                  # :101
    mp = a["max_target_positions"] if a["decoder_chunk_size"] < 0 else a["decoder_chunk_size"]        # :107
    if a["rel_pos_bias"] == "simple":    # relative_positional_bias.py:18
        out += [(m + "rel_pos_bias.rel_pos_bias", [2 * mp - 1], "float32")]
    else:                                # relative_positional_bias.py:53: the `freqs` buffer
        out += [(m + "rel_pos_bias.freqs", [S // 2], "float32")]
    if a["decoder_ffn_embed_dim"] > 0:   # mega_layer.py:98-101; normalized_feedforward_network.py:38-52
        n = prefix + "nffn."
        F_ = a["decoder_ffn_embed_dim"]
        if layer_scale:
            out += [(n + "layerscale_weight", [D], "float32")]                                        # :50
        if not a["no_affine_norm"]:
            out += [(n + "norm.weight", [D], "float32")]
            if a["norm_type"] == "layernorm":                                                         # layer_norm.py:97-98
                out += [(n + "norm.bias", [D], "float32")]
        out += [(n + "fc1.weight", [F_, D], "float32"), (n + "fc1.bias", [F_], "float32"),            # :45
                (n + "fc2.weight", [D, F_], "float32")]                                               # :46
    return out


def decoder_entries(a):
    """MegaDecoderNoCrossAttn.__init__, fairseq/models/mega_lm.py:198-266."""
    D, V = a["decoder_embed_dim"], a["vocab"]
    out = [("decoder.version", [1], "float32"),                                                      # :201
           ("decoder.embed_tokens.weight", [V, D], "float32")]                                        # :213
    for i in range(a["decoder_layers"]):                                                              # :217-220
        out += layer_entries(f"decoder.layers.{i}.", a, a["layer_scale"])
    out += timestep_norm("decoder.final_norm.", D, a["norm_num_groups"])                              # :224
    feat = D
    if a["representation_dim"] is not None:                                                           # :226-232
        feat = a["representation_dim"]
        out += [("decoder.pre_logits.fc.weight", [feat, D], "float32"), ("decoder.pre_logits.fc.bias", [feat], "float32")]
    out += [("decoder.output_projection.weight", [V, feat], "float32")]                               # :252-262
    return out


def main():
    table = {}
    for name, a in ARG_SETS.items():
        table[name] = {"args": a, "entries": [{"name": n, "shape": s, "dtype": d} for n, s, d in decoder_entries(a)]}
    path = os.path.join(HERE, "mega_lm_state_dict.json")
    with open(path, "w") as f:
        json.dump(table, f, indent=1)
    print("wrote", path, {k: len(v["entries"]) for k, v in table.items()})


if __name__ == "__main__":
    main()
