"""The gated-attention layer (the caller of the hot path) and the full Mega2 block against the
fp64 oracle restatement of moving_average_gated_attention.py:263-417."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import rel_err
from gpu_util import DEV, host
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu


def _params(layer):
    p, q, g = layer.move.coeffs()
    P = dict(norm_weight=host(layer.norm.weight), norm_bias=host(layer.norm.bias), p=host(p.squeeze(-1)),
             q=host(q.squeeze(-1)), ema_gamma=host(g), omega=host(layer.move.omega).reshape(-1),
             v_w=host(layer.v_proj.weight), v_b=host(layer.v_proj.bias), mx_w=host(layer.mx_proj.weight),
             mx_b=host(layer.mx_proj.bias), h_w=host(layer.h_proj.weight), gamma=host(layer.gamma),
             beta=host(layer.beta))
    if isinstance(layer.move_act, M.RMSNorm):
        P['rms_weight'] = host(layer.move_act.weight)
    return P


def _chain_ok(y, yo, tol):
    """A layer chains ~10 roundings to the activation type, so the per-op bound (2e-2 for bf16) is
    applied to the root-mean-square error and a 4x wider bound to the worst element."""
    e = host(y) - yo
    rms = np.sqrt(np.mean(yo ** 2))
    return rel_err(host(y), yo) < 4 * tol and np.sqrt(np.mean(e ** 2)) < tol * rms


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("heads,act,moving", [(1, 'rmsnorm', 'cema'), (4, 'silu', 'cema'), (1, 'silu', 'ema')])
def test_gated_attention_layer(dtype, tol, heads, act, moving):
    torch.manual_seed(7)
    B, L, D, S, E, N, C = 2, 512, 64, 32, 128, 16, 256
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_layer=moving, moving_act=act,
                                          norm_num_groups=8, num_heads=heads).to(DEV).eval()
    with torch.no_grad():
        for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
            prm.normal_(0, 0.15)
        layer.gamma.normal_(0, 0.1); layer.beta.normal_(0, 0.1)
        layer.norm.weight.normal_(0, 0.1); layer.norm.bias.normal_(0, 0.1)
        if act == 'rmsnorm':
            layer.move_act.weight.normal_(0, 0.2)        # stored as the offset from one
    P = _params(layer)                       # fp32 master copy of the parameters
    if dtype != torch.float32:               # the module rounds its projection weights to the activation type
        for k_ in ('v_w', 'v_b', 'mx_w', 'mx_b', 'h_w', 'gamma', 'beta', 'norm_weight', 'norm_bias', 'rms_weight'):
            if k_ in P:
                P[k_] = torch.from_numpy(np.asarray(P[k_], np.float32)).to(dtype).double().numpy()
    layer = layer.to(dtype)
    x = torch.randn(B, L, D, device=DEV).to(dtype)
    with torch.no_grad():
        y, _ = layer(x)
    yo = O.gated_attention_layer(host(x), P, chunk=C, num_heads=heads, moving_act=act, num_groups=8)
    assert _chain_ok(y, yo, tol) if dtype != torch.float32 else rel_err(host(y), yo) < tol


def test_incremental_chunks_match_one_shot():
    torch.manual_seed(8)
    B, L, D, S, E, N, C = 2, 512, 64, 32, 64, 16, 128
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_act='silu', norm_num_groups=8).to(DEV).eval()
    x = torch.randn(B, L, D, device=DEV)
    with torch.no_grad():
        full, _ = layer(x)
        state = {}
        parts = [layer(x[:, a:a + C], None, state)[0] for a in range(0, L, C)]
        state2 = {}
        odd = [layer(x[:, a:b], None, state2)[0] for a, b in ((0, 100), (100, 128), (128, 131), (131, 256))]
    assert rel_err(host(torch.cat(parts, 1)), host(full)) < 1e-4
    assert rel_err(host(torch.cat(odd, 1)), host(full[:, :256])) < 1e-4


def test_config4_full_mega2_layer_bf16():
    """B=1, L=8192, D=2048, z=512, v=4096, chunk 2048, 4 heads, SwiGLU 5632, bf16."""
    torch.manual_seed(1238)
    B, L, D, S, E, N, C, Hf = 1, 8192, 2048, 512, 4096, 16, 2048, 5632
    blk = M.Mega2Layer(D, S, E, N, Hf, C, norm_num_groups=16, num_heads=4, moving_act='silu').to(DEV).eval()
    P = _params(blk.attn)
    w1, w2, w3 = host(blk.ffn.w1.weight), host(blk.ffn.w2.weight), host(blk.ffn.w3.weight)
    blk = blk.to(torch.bfloat16)
    x = torch.randn(B, L, D, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        y = blk(x)
        a, _ = blk.attn(x)
    torch.cuda.synchronize()
    assert M.ops.timestep_norm_status() == 0
    # oracle on the first two chunks (causal: they do not see the rest), bf16-rounded weights
    Lo = 2 * C
    rb = lambda a_: torch.from_numpy(np.asarray(a_, np.float32)).to(torch.bfloat16).double().numpy()
    Pb = {k_: (rb(v_) if k_ in ('v_w', 'v_b', 'mx_w', 'mx_b', 'h_w', 'gamma', 'beta', 'norm_weight', 'norm_bias')
               else v_) for k_, v_ in P.items()}
    ao = O.gated_attention_layer(host(x[:, :Lo]), Pb, chunk=C, num_heads=4, moving_act='silu', num_groups=16)
    assert _chain_ok(a[:, :Lo], ao, 2e-2)
    xn, _, _, _ = O.timestep_norm(ao, np.zeros(B, np.int64), np.zeros((B, 16)), np.ones((B, 16)), np.ones(D),
                                  np.zeros(D), None, 16, 1e-5)
    yo = ao + O.swiglu_ffn(xn, rb(w1), rb(w3), rb(w2))
    assert _chain_ok(y[:, :Lo], yo, 2e-2)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("norm_type,layer_scale", [("rmsnorm", None), ("layernorm", 0.1)])
def test_normalized_feed_forward(dtype, tol, norm_type, layer_scale):
    """The reference's position-wise block against the oracle (normalized_feedforward_network.py:77-93)."""
    torch.manual_seed(11)
    B, L, D, Hd = 2, 96, 64, 160
    ffn = M.NormalizedFeedForwardNetwork(D, Hd, norm_type=norm_type, layer_scale=layer_scale, init_mode='xavier')
    with torch.no_grad():
        ffn.fc1.bias.normal_(0, 0.1)
        ffn.norm.weight.normal_(0, 0.2)                   # away from the initial zero (= a multiplier of one)
    ffn = ffn.to(DEV).to(dtype).eval()
    x = torch.randn(B, L, D).to(dtype).to(DEV)
    with torch.no_grad():
        y = ffn(x)
    x64 = host(x)
    if norm_type == "rmsnorm":
        xn = O.rms_norm(x64, host(ffn.norm.weight) + 1.0)          # stored as the offset from one (layer_norm.py:47-56)
    else:
        mu = x64.mean(-1, keepdims=True)
        xn = (x64 - mu) / np.sqrt(x64.var(-1, keepdims=True) + 1e-5) * (host(ffn.norm.weight) + 1.0) + host(ffn.norm.bias)
    w2 = host(ffn.fc2.weight)
    if layer_scale is not None:
        w2 = w2 * host(ffn.layerscale_weight)[:, None]
    yo = O.silu_ffn(xn, host(ffn.fc1.weight), host(ffn.fc1.bias), w2, 0.0) - xn + x64
    assert _chain_ok(y, yo, tol)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("heads,act,moving,masked", [(1, 'rmsnorm', 'cema', True), (2, 'silu', 'cema', False),
                                                     (1, 'silu', 'ema', True)])
def test_bidirectional_gated_attention_layer(dtype, tol, heads, act, moving, masked):
    """The encoder form of the layer: SequenceNorm, two-sided moving average, full softmax per
    chunk with padded keys excluded (one row ends in a chunk that is padding only)."""
    torch.manual_seed(9)
    B, L, D, S, E, N, C = 2, 512, 64, 32, 128, 16, 128
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_layer=moving, moving_act=act,
                                          norm_num_groups=8, num_heads=heads, bidirectional=True).to(DEV).eval()
    with torch.no_grad():
        for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
            prm.normal_(0, 0.15)
        layer.gamma.normal_(0, 0.1); layer.beta.normal_(0, 0.1)
        layer.norm.weight.normal_(0, 0.1); layer.norm.bias.normal_(0, 0.1)
    P = _params(layer)
    if dtype != torch.float32:
        for k_ in ('v_w', 'v_b', 'mx_w', 'mx_b', 'h_w', 'gamma', 'beta', 'norm_weight', 'norm_bias', 'rms_weight'):
            if k_ in P:
                P[k_] = torch.from_numpy(np.asarray(P[k_], np.float32)).to(dtype).double().numpy()
    layer = layer.to(dtype)
    x = torch.randn(B, L, D, device=DEV).to(dtype)
    mask = None
    if masked:
        mask = np.zeros((B, L), bool)
        mask[0, 300:] = True                   # the last chunk of row 0 is padding only
        mask[1, 500:] = True
    with torch.no_grad():
        y, _ = layer(x, None if mask is None else torch.from_numpy(mask).to(DEV))
    yo = O.gated_attention_layer(host(x), P, chunk=C, num_heads=heads, moving_act=act, num_groups=8,
                                 bidirectional=True, padding_mask=mask)
    keep = np.ones((B, L), bool) if mask is None else ~mask     # padded positions carry no meaning
    got, ref = host(y)[keep], yo[keep]
    if dtype == torch.float32:
        assert rel_err(got, ref) < tol
    else:
        e = got - ref
        rms = np.sqrt((ref ** 2).mean())
        assert np.sqrt((e ** 2).mean()) < tol * rms and np.abs(e).max() < 4 * tol * max(rms, np.abs(ref).max())


def _lm_args(**kw):
    import types
    base = dict(decoder_embed_dim=64, decoder_z_dim=32, decoder_hidden_dim=128, decoder_n_dim=16,
                decoder_chunk_size=128, decoder_ffn_embed_dim=160, norm_num_groups=8, norm_type='rmsnorm',
                moving_layer='cema', moving_act='rmsnorm', efficient_attention=True, rel_pos_bias='rotary')
    base.update(kw)
    return types.SimpleNamespace(**base)


def test_decoder_stack_streams_like_the_reference_validation():
    """Three MegaDecoderLayers: a document streamed in chunk-sized slices with one incremental-state
    dictionary equals the one-shot forward (fp32: the recurrences agree to ~1e-5), also when the
    slices are half chunks."""
    torch.manual_seed(21)
    args = _lm_args()
    layers = torch.nn.ModuleList([M.MegaDecoderLayer(args) for _ in range(3)]).to(DEV).eval()
    with torch.no_grad():
        for lyr in layers:
            for prm in (lyr.mega_layer.v_proj.weight, lyr.mega_layer.mx_proj.weight, lyr.mega_layer.h_proj.weight,
                        lyr.nffn.fc1.weight, lyr.nffn.fc2.weight):
                prm.normal_(0, 0.1)
    x = torch.randn(2, 512, 64, device=DEV)
    with torch.no_grad():
        full = x
        for lyr in layers:
            full = lyr(full)[0]
        streamed = M.streamed_forward(layers, x, 128)
        halves = M.streamed_forward(layers, x, 64)
    assert rel_err(host(streamed), host(full)) < 5e-5
    assert rel_err(host(halves), host(full)) < 5e-5
    assert M.ops.timestep_norm_status() == 0


def test_decoder_and_encoder_layer_names_and_training():
    args = _lm_args()
    dec = M.MegaDecoderLayer(args).to(DEV).train()
    keys = set(dec.state_dict())
    assert {"mega_layer.norm.weight", "mega_layer.move.alpha", "mega_layer.mx_proj.weight", "mega_layer.gamma",
            "mega_layer.move_act.weight", "mega_layer.rel_pos_bias.freqs", "nffn.norm.weight", "nffn.fc1.weight",
            "nffn.fc1.bias", "nffn.fc2.weight"} <= keys
    x = torch.randn(2, 256, 64, device=DEV, requires_grad=True)
    dec(x)[0].square().mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in dec.parameters())
    import types
    eargs = types.SimpleNamespace(encoder_embed_dim=64, encoder_z_dim=32, encoder_hidden_dim=128, encoder_n_dim=16,
                                  encoder_chunk_size=128, encoder_ffn_embed_dim=160, norm_num_groups=8,
                                  norm_type='layernorm', moving_act='silu')
    enc = M.MegaEncoderLayer(eargs).to(DEV).train()
    assert isinstance(enc.mega_layer.norm, M.SequenceNorm) and enc.mega_layer.move.bidirectional
    mask = torch.zeros(2, 256, dtype=torch.bool, device=DEV)
    mask[1, 200:] = True
    xe = torch.randn(2, 256, 64, device=DEV, requires_grad=True)
    (enc(xe, mask) * (~mask)[..., None]).square().mean().backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in enc.parameters())
    assert torch.isfinite(xe.grad).all()


@pytest.mark.parametrize("bidir", [False, True])
def test_simple_relative_bias_layer(bidir):
    """rel_pos_bias='simple' (moving_average_gated_attention.py:109-110): scores = q k^T + bias[j - i],
    no rotation; forward against the layer oracle and a training step against central differences
    of the bias parameter."""
    torch.manual_seed(31)
    B, L, D, S, E, N, C = 2, 128, 32, 16, 48, 8, 64
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_act='silu', norm_num_groups=4,
                                          rel_pos_bias='simple', bidirectional=bidir).to(DEV).eval()
    with torch.no_grad():
        for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
            prm.normal_(0, 0.2)
        layer.gamma.normal_(0, 0.3); layer.beta.normal_(0, 0.3)
        layer.rel_pos_bias.rel_pos_bias.normal_(0, 0.5)
    P = _params(layer)
    sb = host(layer.rel_pos_bias.rel_pos_bias)
    assert sb.shape == (2 * C - 1,)
    x = torch.randn(B, L, D, device=DEV)
    okw = dict(chunk=C, num_heads=1, moving_act='silu', num_groups=4, bidirectional=bidir)
    with torch.no_grad():
        y, _ = layer(x)
    assert rel_err(host(y), O.gated_attention_layer(host(x), P, simple_bias=sb, **okw)) < 2e-4
    w = torch.randn(B, L, D, device=DEV)
    layer.train()
    out, _ = layer(x)
    (out * w).sum().backward()
    g = host(layer.rel_pos_bias.rel_pos_bias.grad)
    rng = np.random.default_rng(3)
    for _ in range(4):
        i = int(rng.integers(C - 20, C + 19))              # offsets that occur often
        sp, sm = sb.copy(), sb.copy()
        sp[i] += 1e-5; sm[i] -= 1e-5
        fd = ((O.gated_attention_layer(host(x), P, simple_bias=sp, **okw) * host(w)).sum()
              - (O.gated_attention_layer(host(x), P, simple_bias=sm, **okw) * host(w)).sum()) / 2e-5
        assert abs(fd - g[i]) < 3e-3 * (np.abs(g).max() + 1e-6), (i, fd, g[i])


def test_decoder_model_names_streaming_and_training():
    """MegaDecoderNoCrossAttn: reference state-dict names, logits streamed chunk by chunk equal to
    the one-shot logits (also for a length that is not a whole number of chunks), and a
    cross-entropy training step."""
    torch.manual_seed(41)
    args = _lm_args(decoder_layers=2, share_decoder_input_output_embed=True, layer_scale=True, norm_eps=1e-5)
    vocab, pad = 50, 1
    emb = torch.nn.Embedding(vocab, 64, padding_idx=pad)
    model = M.MegaDecoderNoCrossAttn(args, vocab, emb).to(DEV).eval()
    keys = set(model.state_dict())
    assert {"version", "embed_tokens.weight", "layers.0.mega_layer.norm.weight", "layers.1.mega_layer.move.alpha",
            "layers.0.nffn.fc1.weight", "layers.1.nffn.layerscale_weight", "final_norm.weight", "final_norm.bias",
            "output_projection.weight"} <= keys
    assert model.output_projection.weight is model.embed_tokens.weight
    with torch.no_grad():
        for lyr in model.layers:
            for prm in (lyr.mega_layer.v_proj.weight, lyr.mega_layer.mx_proj.weight, lyr.mega_layer.h_proj.weight):
                prm.normal_(0, 0.1)
    tokens = torch.randint(2, vocab, (2, 512), device=DEV)
    with torch.no_grad():
        full = model(tokens)[0]
        streamed = model.streamed(tokens)
        odd = model(tokens[:, :300])[0]                  # padded up to 384 tokens inside, cut back to 300
    assert full.shape == (2, 512, vocab) and rel_err(host(streamed), host(full)) < 5e-5
    assert odd.shape == (2, 300, vocab) and rel_err(host(odd[:, :256]), host(full[:, :256])) < 5e-5
    model.train()
    logits = model(tokens[:, :-1])[0]
    loss = torch.nn.functional.cross_entropy(logits.reshape(-1, vocab).float(), tokens[:, 1:].reshape(-1))
    loss.backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in model.parameters())


def test_layer_dropouts_act_in_training_only():
    """dropout / hidden_dropout / attention_dropout (moving_average_gated_attention.py:64-79, 316,
    407-410): identity in eval mode; in training mode they change the output, follow torch's seed,
    and with all three at zero the training path equals the inference path."""
    torch.manual_seed(3)
    D, S, E, N, C = 32, 16, 48, 4, 16
    kw = dict(chunk_size=C, norm_num_groups=4, moving_act='silu')
    plain = M.MovingAverageGatedAttention(D, S, E, N, **kw).to(DEV)
    drop = M.MovingAverageGatedAttention(D, S, E, N, dropout=0.1, attention_dropout=0.2, hidden_dropout=0.1,
                                         **kw).to(DEV)
    drop.load_state_dict(plain.state_dict())
    x = torch.randn(2, 64, D, device=DEV)
    with torch.no_grad():
        ref = plain.eval()(x)[0]
        assert torch.equal(drop.eval()(x)[0], ref)
        torch.manual_seed(7)
        a = drop.train()(x)[0]
        torch.manual_seed(7)
        b = drop(x)[0]
        assert torch.equal(a, b) and not torch.allclose(a, ref, atol=1e-4)
        assert torch.isfinite(a).all()
    # each dropout alone reaches the output, and gradients flow through the dropped layer
    for name in ('dropout', 'attention_dropout', 'hidden_dropout'):
        one = M.MovingAverageGatedAttention(D, S, E, N, **{name: 0.3}, **kw).to(DEV).train()
        one.load_state_dict(plain.state_dict())
        xg = x.clone().requires_grad_(True)
        y = one(xg)[0]
        assert not torch.allclose(y.detach(), ref, atol=1e-5), name
        y.square().sum().backward()
        assert torch.isfinite(xg.grad).all() and all(torch.isfinite(p.grad).all() for p in one.parameters()
                                                     if p.grad is not None)
    f = M.NormalizedFeedForwardNetwork(D, 64, dropout=0.2, hidden_dropout=0.2).to(DEV)
    assert torch.equal(f.eval()(x), f(x)) and not torch.equal(f.train()(x), f.eval()(x))
    # efficient_attn=False: plain dropout on the softmax weights instead of DropKey (:66-79, 244-247)
    wd = M.MovingAverageGatedAttention(D, S, E, N, attention_dropout=0.3, efficient_attn=False, **kw).to(DEV)
    wd.load_state_dict(plain.state_dict())
    with torch.no_grad():
        assert torch.equal(wd.eval()(x)[0], ref)
        _, w = wd.train()(x, need_weights=True)
    zeros = (w.tril() == 0) & (torch.ones_like(w).tril() > 0)
    assert 0.2 < zeros.float().sum() / torch.ones_like(w).tril().sum() < 0.4
    assert (w.sum(-1) - 1).abs().max() > 0.05           # survivors are scaled by 1 / (1 - p), rows no longer sum to one


def test_decoder_model_beam_reorder():
    """reorder_incremental_state: after some tokens the streams are permuted / duplicated as beam
    search does (fairseq_incremental_decoder.py:82-96); decoding on equals decoding the reordered
    streams from the start.  Single tokens, so the K/V chunk cache, the norm state and the
    moving-average state all carry entries."""
    torch.manual_seed(43)
    args = _lm_args(decoder_layers=2, norm_eps=1e-5)
    vocab = 40
    model = M.MegaDecoderNoCrossAttn(args, vocab, torch.nn.Embedding(vocab, 64, padding_idx=1)).to(DEV).eval()
    tokens = torch.randint(2, vocab, (3, 40), device=DEV)
    order = torch.tensor([2, 0, 2], device=DEV)
    with torch.no_grad():
        state = {}
        for t in range(25):
            model(tokens[:, t:t + 1], incremental_state=state)
        model.reorder_incremental_state(state, order)
        got = torch.cat([model(tokens[order][:, t:t + 1], incremental_state=state)[0] for t in range(25, 40)], dim=1)
        ref_state = {}
        ref = torch.cat([model(tokens[order][:, t:t + 1], incremental_state=ref_state)[0] for t in range(40)], dim=1)
    assert rel_err(host(got), host(ref[:, 25:])) < 1e-5


@pytest.mark.parametrize("act", ['laplace', 'relu2'])
@pytest.mark.parametrize("bidir,bias,masked", [(False, 'rotary', False), (True, 'simple', True), (True, 'rotary', True),
                                               (False, 'simple', True)])
def test_element_attention_layer(act, bidir, bias, masked):
    """attention_activation = relu2 / laplace (moving_average_gated_attention.py:153-208): forward in
    inference and in training mode against the layer oracle, and the gradient of the q / k scale
    against central differences of the oracle."""
    torch.manual_seed(37)
    B, L, D, S, E, N, C = 2, 128, 32, 16, 48, 8, 64
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_act='silu', norm_num_groups=4,
                                          rel_pos_bias=bias, bidirectional=bidir,
                                          attention_activation=act).to(DEV).eval()
    with torch.no_grad():
        for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
            prm.normal_(0, 0.2)
        layer.gamma.normal_(0, 0.5); layer.beta.normal_(0, 0.5)
        if bias == 'simple':
            layer.rel_pos_bias.rel_pos_bias.normal_(0, 0.5)
    P = _params(layer)
    sb = host(layer.rel_pos_bias.rel_pos_bias) if bias == 'simple' else None
    x = torch.randn(B, L, D, device=DEV)
    mask = None
    if masked:
        mask = np.zeros((B, L), bool)
        mask[0, 100:] = True
        mask[1, 60:] = True                     # the second chunk of row 1 is padding only
    tm = None if mask is None else torch.from_numpy(mask).to(DEV)
    okw = dict(chunk=C, num_heads=1, moving_act='silu', num_groups=4, bidirectional=bidir, padding_mask=mask,
               simple_bias=sb, attention_activation=act)
    yo = O.gated_attention_layer(host(x), P, **okw)
    keep = np.ones((B, L), bool) if mask is None else ~mask
    with torch.no_grad():
        y, _ = layer(x, tm)
    assert rel_err(host(y)[keep], yo[keep]) < 2e-4
    layer.train()
    w = torch.randn(B, L, D, device=DEV) * torch.from_numpy(keep).to(DEV)[..., None]
    out, _ = layer(x, tm)
    assert rel_err(host(out)[keep], yo[keep]) < 2e-4
    (out * w).sum().backward()
    g = host(layer.gamma.grad)
    for (a, i) in [(0, 3), (1, 11)]:
        Pp, Pm = dict(P), dict(P)
        Pp['gamma'] = P['gamma'].copy(); Pm['gamma'] = P['gamma'].copy()
        Pp['gamma'][a, i] += 1e-5; Pm['gamma'][a, i] -= 1e-5
        fd = ((O.gated_attention_layer(host(x), Pp, **okw) * host(w)).sum()
              - (O.gated_attention_layer(host(x), Pm, **okw) * host(w)).sum()) / 2e-5
        assert abs(fd - g[a, i]) < 3e-3 * (np.abs(g).max() + 1e-6), (a, i, fd, g[a, i])


@pytest.mark.parametrize("heads", [1, 2])
def test_need_weights_returns_the_chunk_attention(heads):
    """need_weights (moving_average_gated_attention.py:266, 414-417): same output as the fused call, weights
    per chunk with rows that sum to one and no weight on future keys."""
    torch.manual_seed(39)
    B, L, D, S, E, N, C = 2, 128, 32, 16, 48, 8, 64
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_act='silu', norm_num_groups=4,
                                          num_heads=heads).to(DEV).eval()
    with torch.no_grad():
        for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
            prm.normal_(0, 0.2)
        x = torch.randn(B, L, D, device=DEV)
        y0, none = layer(x)
        y1, w = layer(x, need_weights=True, attn_mask=torch.ones(C, C, device=DEV).tril())
    assert none is None and rel_err(host(y1), host(y0)) < 1e-5
    assert w.shape == ((B * L // C, C, C) if heads == 1 else (B * L // C, heads, C, C))
    assert torch.allclose(w.sum(-1), torch.ones_like(w.sum(-1)), atol=1e-5)
    assert torch.all(w.triu(1) == 0)
    dec = M.MegaDecoderLayer(_lm_args()).to(DEV).eval()
    with torch.no_grad():
        out, attn, _ = dec(torch.randn(1, 256, 64, device=DEV), need_attn=True)
    assert attn.shape == (2, 128, 128)
    with pytest.raises(NotImplementedError):
        layer(x, before_attn_fn=True)


def test_chunkwise_validation_equals_one_shot_loss():
    """validate_stream (fairseq_cli/train.py:395-417): the summed loss over chunk-wise slices with carried
    state equals the loss of the whole documents in one forward; padded targets are not counted."""
    torch.manual_seed(45)
    args = _lm_args(decoder_layers=2, norm_eps=1e-5)
    vocab, pad = 40, 1
    model = M.MegaDecoderNoCrossAttn(args, vocab, torch.nn.Embedding(vocab, 64, padding_idx=pad)).to(DEV).eval()
    tokens = torch.randint(2, vocab, (3, 513), device=DEV)
    src, tgt = tokens[:, :-1].clone(), tokens[:, 1:].clone()
    src[1, 400:] = pad
    tgt[1, 399:] = pad                                   # a document that ends early
    nll, ntok = M.validate_stream(model, src, tgt, pad)
    with torch.no_grad():
        logits = model(src)[0]
    ref = torch.nn.functional.cross_entropy(logits.reshape(-1, vocab).float(), tgt.reshape(-1), ignore_index=pad,
                                            reduction='sum')
    assert int(ntok) == int(tgt.ne(pad).sum()) == 2 * 512 + 399
    assert abs(float(nll) - float(ref)) < 1e-4 * float(ref)


@pytest.mark.parametrize("bias,act", [('simple', 'softmax'), ('rotary', 'laplace'), ('simple', 'relu2')])
@pytest.mark.parametrize("step", [1, 16, 64])
def test_incremental_decoding_with_learned_bias_and_element_attention(bias, act, step):
    """The key / value chunk cache with the learned position bias (rows of the new positions,
    moving_average_gated_attention.py:212-221) and with the element-wise attention: a sequence fed in
    slices of `step` tokens (1: token by token; 64: whole chunks) equals the one-shot forward."""
    torch.manual_seed(47)
    B, L, D, S, E, N, C = 2, 160, 32, 16, 48, 8, 64
    layer = M.MovingAverageGatedAttention(D, S, E, N, chunk_size=C, moving_act='silu', norm_num_groups=4,
                                          rel_pos_bias=bias, attention_activation=act).to(DEV).eval()
    with torch.no_grad():
        for prm in (layer.v_proj.weight, layer.mx_proj.weight, layer.h_proj.weight):
            prm.normal_(0, 0.2)
        layer.gamma.normal_(0, 0.5); layer.beta.normal_(0, 0.5)
        if bias == 'simple':
            layer.rel_pos_bias.rel_pos_bias.normal_(0, 0.5)
        x = torch.randn(B, 128, D, device=DEV)
        full, _ = layer(x)
        state = {}
        parts = [layer(x[:, a:a + step], incremental_state=state)[0] for a in range(0, 128, step)]
    assert rel_err(host(torch.cat(parts, dim=1)), host(full)) < 2e-5


def test_weights_loaded_after_an_eval_forward_take_effect():
    """The eval-mode caches (moving-average coefficients and operand images, weight + 1 / bias of the norm,
    the q / k affine) are rebuilt when load_state_dict or an in-place edit changes the parameters."""
    B, L, D, S, E, N, C = 1, 1024, 64, 32, 128, 16, 256
    mk = lambda seed: (torch.manual_seed(seed), M.MovingAverageGatedAttention(
        D, S, E, N, chunk_size=C, norm_num_groups=1).to(DEV).to(torch.bfloat16).eval())[1]
    a, b = mk(11), mk(12)
    with torch.no_grad():
        for layer in (a, b):
            layer.gamma.normal_(0, 0.1); layer.beta.normal_(0, 0.1)
            layer.norm.weight.normal_(0, 0.1); layer.norm.bias.normal_(0, 0.1)
    x = torch.randn(B, L, D, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        ya, _ = a(x)
        yb, _ = b(x)
        assert not torch.equal(ya, yb)
        a.load_state_dict(b.state_dict())
        ya2, _ = a(x)
        assert torch.equal(ya2, yb)
        a.move.alpha.add_(0.3); b.move.alpha.add_(0.3)
        a.norm.weight.mul_(0.5); b.norm.weight.mul_(0.5)
        b.train(); b.eval()                  # b recomputes everything
        ya3, _ = a(x)
        yb3, _ = b(x)
        assert torch.equal(ya3, yb3) and not torch.equal(ya3, ya2)


def test_residual_product_in_place():
    """linear_residual: outside autograd a residual the caller gives up takes the product in place (no copy of the
    residual first); under autograd, or without `consume`, the residual is left as it was."""
    torch.manual_seed(3)
    lin = torch.nn.Linear(96, 64, bias=False).to(DEV).to(torch.bfloat16)
    h = torch.randn(2, 40, 96, device=DEV).to(torch.bfloat16)
    res = torch.randn(2, 40, 64, device=DEV).to(torch.bfloat16)
    with torch.no_grad():
        ref = M.modules.linear_residual(lin, h, res)
        assert ref.data_ptr() != res.data_ptr()
        mine = res.clone()
        out = M.modules.linear_residual(lin, h, mine, consume=True)
        assert out.data_ptr() == mine.data_ptr() and torch.equal(out, ref)
    keep = res.clone()
    out = M.modules.linear_residual(lin, h, res, consume=True)          # autograd on: lin.weight requires grad
    assert out.data_ptr() != res.data_ptr() and torch.equal(res, keep) and torch.equal(out, ref)
