"""A time tile that gives up waiting for an earlier tile: the outputs and statistics that depended on the
missing words are NaN (never a partial sum), the status word is set, the next call of the entry point raises
once, and the call after that is correct again.  The condition is forced from the host (the first tile of a
row publishes nothing, the poll limit is tiny), so every kernel exits normally."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import mega_init_complex
from gpu_util import DEV, dev
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu
BF = torch.bfloat16


@pytest.fixture
def hooks():
    lib = M._lib.load()
    torch.cuda.synchronize()
    assert lib.mega_lookback_status(0) == 0
    yield lib
    torch.cuda.synchronize()
    lib.mega_test_lookback(0, 0, 0)
    lib.mega_lookback_status(1)
    M.ops.timestep_norm_status(clear=True)


def _state(B, G):
    return (torch.zeros(B, dtype=torch.int64, device=DEV), torch.zeros(B, G, device=DEV), torch.ones(B, G, device=DEV))


@pytest.mark.parametrize("L", [4096, 32768])
def test_group_norm_tile_that_gives_up(hooks, L):
    """4096 tokens: every tile looks back over the tiles themselves; 32768 tokens (512 tiles a row): over block
    records, which a block's last tile withholds when it gave up itself, so that the later blocks give up too."""
    lib = hooks
    B, D, G = 2, 256, 4
    torch.manual_seed(61)
    x = torch.randn(B, L, D, device=DEV).to(BF)
    gamma, beta = torch.ones(D, device=DEV), torch.zeros(D, device=DEV)
    run = lambda: M.ops.group_timestep_norm_fwd(x, *_state(B, G), gamma, beta, None, G, 1e-5, need_stats=False)
    good = run()
    torch.cuda.synchronize()
    print("forced give-up: group_timestep_norm_fwd", flush=True)
    lib.mega_test_lookback(64, 1, 0)
    bad = run()
    torch.cuda.synchronize()
    lib.mega_test_lookback(0, 0, 0)
    y, count, mean, var = bad[0], bad[1], bad[2], bad[3]
    nan_tok = torch.isnan(y.float()).any(-1)                     # [B, L]
    assert nan_tok.any() and not nan_tok[:, 0].any()
    first = int(nan_tok[0].float().argmax())                     # the first tile is whole, the rest is NaN throughout
    assert first > 0 and nan_tok[:, first:].all() and not nan_tok[:, :first].any()
    assert torch.equal(y[:, :first], good[0][:, :first])
    assert torch.isnan(mean).all() and count.tolist() == [-1] * B
    assert M.ops.lookback_status() == 1 and M.ops.timestep_norm_status() != 0
    with pytest.raises(RuntimeError, match="gave up"):
        run()
    assert M.ops.lookback_status() == 0
    again = run()
    torch.cuda.synchronize()
    assert torch.equal(again[0], good[0]) and torch.equal(again[2], good[2]) and again[1].tolist() == [L] * B
    assert M.ops.lookback_status() == 0


def test_one_kernel_block_that_gives_up(hooks):
    lib = hooks
    B, L, G, N = 2, 4096, 2, 16
    D = 64 * G
    rng = np.random.default_rng(62)
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(rng.normal(size=D)))
    x = torch.randn(B, L, D, device=DEV).to(BF)
    gamma, beta = torch.ones(D, device=DEV), torch.zeros(D, device=DEV)
    run = lambda: layer.norm_forward(x, *_state(B, G), gamma, beta, G, 1e-5, want_state=True)
    good = run()
    torch.cuda.synchronize()
    print("forced give-up: norm_ema_fwd", flush=True)
    lib.mega_test_lookback(64, 1, 0)
    xn, y, count, mean, var, h = run()
    torch.cuda.synchronize()
    lib.mega_test_lookback(0, 0, 0)
    assert torch.equal(xn[:, :1024], good[0][:, :1024]) and torch.equal(y[..., :1024], good[1][..., :1024])
    assert torch.isnan(xn[:, 1024:].float()).all() and torch.isnan(y[..., 1024:].float()).all()
    assert torch.isnan(mean).all() and count.tolist() == [-1] * B
    assert torch.isnan(torch.view_as_real(h)).any()
    assert M.ops.lookback_status() == 1
    with pytest.raises(RuntimeError, match="gave up"):
        run()
    again = run()
    torch.cuda.synchronize()
    assert torch.equal(again[0], good[0]) and torch.equal(again[1], good[1]) and torch.equal(again[3], good[3])
    assert M.ops.lookback_status() == 0


@pytest.mark.parametrize("L", [4096, 8192])
def test_norm_backward_tile_that_gives_up(hooks, L):
    """The one-launch TimestepNorm backward walks a row from its last tile to its first: with the row's last tile
    publishing nothing, every other tile gives up (4096 tokens: 128 tiles that look back over the tiles themselves;
    8192: block records, which a block's first tile withholds when it gave up itself)."""
    lib = hooks
    B, D, G = 2, 1024, 16
    torch.manual_seed(64)
    x = torch.randn(B, L, D, device=DEV).to(BF)
    dy = torch.randn(B, L, D, device=DEV).to(BF)
    gamma, beta = torch.ones(D, device=DEV), torch.zeros(D, device=DEV)
    y, cnt, mu, var, gm, cm, cr = M.ops.group_timestep_norm_fwd(x, *_state(B, G), gamma, beta, None, G, 1e-5)
    pm = torch.zeros(B, G, device=DEV)
    run = lambda: M.ops.group_timestep_norm_bwd(dy, None, None, x, pm, cnt, gm, cm, cr, gamma, None, G)
    good = run()
    torch.cuda.synchronize()
    print("forced give-up: group_timestep_norm_bwd", flush=True)
    lib.mega_test_lookback(64, 1, 0)
    bad = run()
    torch.cuda.synchronize()
    lib.mega_test_lookback(0, 0, 0)
    nan_tok = torch.isnan(bad[0].float()).any(-1)                # [B, L]
    assert nan_tok[:, :L - 32].all() and not nan_tok[:, L - 32:].any()
    assert torch.equal(bad[0][:, L - 32:], good[0][:, L - 32:])   # the last tile waits for nobody
    assert torch.isnan(bad[1]).all() and torch.isnan(bad[2]).all()
    assert M.ops.lookback_status() == 1
    with pytest.raises(RuntimeError, match="gave up"):
        run()
    assert M.ops.lookback_status() == 0
    again = run()
    torch.cuda.synchronize()
    for a, b_ in zip(again, good):
        assert torch.equal(a, b_)
    assert M.ops.lookback_status() == 0


def test_checked_mode_reports_the_give_up_of_the_same_call(hooks):
    """With checked mode on, the call whose launch gave up raises itself (after waiting for its stream); nothing is
    left over for the next call."""
    lib = hooks
    B, L, G, N = 2, 4096, 2, 16
    D = 64 * G
    rng = np.random.default_rng(63)
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, D, N))
    layer = M.ops.PreparedEMA(dev(p), dev(q), dev(g), dev(rng.normal(size=D)))
    x = torch.randn(B, L, D, device=DEV).to(BF)
    gamma, beta = torch.ones(D, device=DEV), torch.zeros(D, device=DEV)
    block = lambda: layer.norm_forward(x, *_state(B, G), gamma, beta, G, 1e-5)
    norm = lambda: M.ops.group_timestep_norm_fwd(x, *_state(B, G), gamma, beta, None, G, 1e-5, need_stats=False)
    good_b, good_n = block(), norm()
    torch.cuda.synchronize()
    M.ops.lookback_checked(True)
    try:
        for run, good in ((block, good_b), (norm, good_n)):
            print("forced give-up in checked mode", flush=True)
            lib.mega_test_lookback(64, 1, 0)
            with pytest.raises(RuntimeError, match="this launch gave up"):
                run()
            lib.mega_test_lookback(0, 0, 0)
            assert M.ops.lookback_status() == 0
            again = run()                                    # nothing pending: the next call runs, and is right
            torch.cuda.synchronize()
            assert torch.equal(again[0], good[0]) and torch.equal(again[1], good[1])
    finally:
        M.ops.lookback_checked(False)
