"""HIP TimestepNorm against the fp64 oracle (group and per-feature variants)."""
import numpy as np
import pytest
import torch

import fairseq_apollo_amd as M
from conftest import rel_err
from gpu_util import DEV, TOL, dev, host, rounded
from oracle import mega_oracle as O

pytestmark = pytest.mark.gpu


def _case(seed, B, L, H, G, dtype, masked, prior):
    rng = np.random.default_rng(seed)
    x, x64 = rounded(rng.normal(size=(B, L, H)) * 1.5 + 0.3, dtype)
    Gs = H if G is None else G
    mask = (rng.random((B, L)) < 0.25) if masked else None
    if prior:
        pc = rng.integers(2, 9, size=B).astype(np.int64)
        pm = rng.normal(size=(B, Gs)).astype(np.float32) * 0.3
        pv = (rng.random((B, Gs)) + 0.5).astype(np.float32)
    else:
        pc = np.zeros(B, np.int64); pm = np.zeros((B, Gs), np.float32); pv = np.ones((B, Gs), np.float32)
    gamma = (rng.normal(size=H) * 0.2 + 1).astype(np.float32)
    beta = (rng.normal(size=H) * 0.2).astype(np.float32)
    return x, x64, mask, pc, pm, pv, gamma, beta


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,L,H,G", [(2, 37, 64, 4), (3, 300, 256, 16), (1, 1, 128, 8), (2, 129, 96, 2),
                                     (1, 70, 2048, 16), (2, 50, 48, 12)])
@pytest.mark.parametrize("masked,prior", [(False, False), (True, True)])
def test_group_matches_oracle(dtype, B, L, H, G, masked, prior):
    print(f"case dtype={dtype} B={B} L={L} H={H} G={G} masked={masked} prior={prior}", flush=True)
    x, x64, mask, pc, pm, pv, gamma, beta = _case(1, B, L, H, G, dtype, masked, prior)
    out = M.ops.group_timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma), dev(beta),
                                        None if mask is None else dev(mask, torch.bool), G, 1e-5)
    torch.cuda.synchronize()
    assert M.ops.timestep_norm_status() == 0
    y, c, mu, v = O.timestep_norm(x64, pc, pm, pv, gamma, beta, mask, G, 1e-5)
    assert rel_err(host(out[0]), y) < TOL[dtype]
    assert np.array_equal(host(out[1]), c)
    assert rel_err(host(out[2]), mu) < 1e-4 and rel_err(host(out[3]), v) < 1e-4
    if mask is not None:
        assert torch.all(out[0][dev(mask, torch.bool)] == 0)
    # statistics saved for a backward pass: running mean / rstd after each unmasked step
    _, muc, varc = O.timestep_norm_closed_form(x64, mask, G) if not prior else (None, None, None)
    if muc is not None and mask is None:
        assert rel_err(host(out[5]), muc) < 1e-4
        assert rel_err(host(out[6]), 1 / np.sqrt(varc + 1e-5)) < 1e-4
        assert rel_err(host(out[4]), x64.reshape(B, L, G, -1).mean(-1)) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,H,G,masked,prior", [(2, 3000, 256, 32, True, True), (1, 2100, 384, 48, False, False),
                                                  (2, 1500, 512, 256, True, False), (1, 9000, 128, 64, False, True)])
def test_more_than_sixteen_groups_over_many_tiles(dtype, B, L, H, G, masked, prior):
    """Groups are handled 16 at a time.  Every set's aggregates are published before the first look-back (a tile does
    not wait for the earlier tiles with its later sets still unpublished), and a look-back reads only its set's words
    of the records; 9000 tokens: block records as well.  Also a bound on the time, which a row that turned into a
    chain of tiles misses by two orders of magnitude."""
    print(f"case dtype={dtype} B={B} L={L} H={H} G={G} masked={masked} prior={prior}", flush=True)
    x, x64, mask, pc, pm, pv, gamma, beta = _case(11, B, L, H, G, dtype, masked, prior)
    run = lambda: M.ops.group_timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma), dev(beta),
                                                None if mask is None else dev(mask, torch.bool), G, 1e-5)
    out = run()
    torch.cuda.synchronize()
    assert M.ops.timestep_norm_status() == 0
    y, c, mu, v = O.timestep_norm(x64, pc, pm, pv, gamma, beta, mask, G, 1e-5)
    assert rel_err(host(out[0]), y) < TOL[dtype]
    assert np.array_equal(host(out[1]), c)
    assert rel_err(host(out[2]), mu) < 1e-4 and rel_err(host(out[3]), v) < 1e-4
    if not prior and mask is None:
        _, muc, varc = O.timestep_norm_closed_form(x64, mask, G)
        assert rel_err(host(out[5]), muc) < 1e-4
        assert rel_err(host(out[6]), 1 / np.sqrt(varc + 1e-5)) < 1e-4
    a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(5):
        run()
    b_.record()
    torch.cuda.synchronize()
    assert a.elapsed_time(b_) / 5 < 2.0, "milliseconds per call"


def test_chunked_streaming_equals_one_shot():
    rng = np.random.default_rng(5)
    B, L, H, G = 2, 256, 128, 8
    tn = M.TimestepNorm(H, G).to(DEV).eval()
    with torch.no_grad():
        tn.weight.copy_(dev(rng.normal(size=H) * 0.1)); tn.bias.copy_(dev(rng.normal(size=H) * 0.1))
        x, x64 = rounded(rng.normal(size=(B, L, H)), torch.float32)
        full = tn(x)
        state = {}
        parts = [tn(x[:, a:b], None, state) for a, b in ((0, 100), (100, 101), (101, 256))]
    assert rel_err(host(torch.cat(parts, 1)), host(full)) < 1e-5
    saved = tn._get_input_buffer(state)
    assert saved["prev_count"].tolist() == [L, L]
    y, _, mu, v = O.timestep_norm(x64, np.zeros(B, np.int64), np.zeros((B, G)), np.ones((B, G)),
                                  host(tn.weight) + 1, host(tn.bias), None, G, 1e-5)
    assert rel_err(host(full), y) < 1e-4 and rel_err(host(saved["prev_mean"]), mu) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feature_variant_matches_oracle(dtype):
    x, x64, mask, pc, pm, pv, gamma, beta = _case(7, 2, 90, 40, None, dtype, True, True)
    out = M.ops.timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma), dev(beta),
                                  dev(mask, torch.bool), 1e-5)
    y, c, mu, v = O.timestep_norm(x64, pc, pm, pv, gamma, beta, mask, None, 1e-5)
    assert rel_err(host(out[0]), y) < TOL[dtype] and np.array_equal(host(out[1]), c)
    assert rel_err(host(out[2]), mu) < 1e-4 and rel_err(host(out[3]), v) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,L,H,masked", [(2, 700, 96, True), (3, 129, 40, False), (1, 4096, 300, True)])
def test_feature_variant_parallel_over_time(dtype, B, L, H, masked):
    """Sequences longer than two time tiles run the per-feature variant as three kernels parallel over tiles of 64
    tokens: against the fp64 oracle (cumulative statistics included), and against the one-thread-per-feature
    kernel, which the same entry point runs for short rows when it gets no workspace."""
    print(f"case {dtype} B={B} L={L} H={H} masked={masked}", flush=True)
    x, x64, mask, pc, pm, pv, gamma, beta = _case(9, B, L, H, None, dtype, masked, True)
    if masked:
        mask[0, 64:128] = True                                   # a whole tile without a token
        mask[-1, :70] = True                                     # a row that starts masked
    tm = dev(mask, torch.bool) if masked else None
    out = M.ops.timestep_norm_fwd(x, dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma), dev(beta), tm, 1e-5)
    y, c, mu, v = O.timestep_norm(x64, pc, pm, pv, gamma, beta, mask if masked else None, None, 1e-5)
    assert rel_err(host(out[0]), y) < TOL[dtype] and np.array_equal(host(out[1]), c)
    assert rel_err(host(out[2]), mu) < 1e-4 and rel_err(host(out[3]), v) < 1e-4
    # without a workspace the entry point refuses rows this long (the one-thread-per-feature kernel would run for
    # milliseconds); the first 128 tokens through that kernel equal the tiled kernels' first 128 (the norm is causal)
    lib = M._lib.load()
    xd = x.contiguous()
    m8 = None if tm is None else tm.to(torch.uint8).contiguous()
    args = [dev(pc, torch.int64), dev(pm), dev(pv), dev(gamma), dev(beta)]

    def serial(Ls):
        xs = xd[:, :Ls].contiguous()
        ms = None if m8 is None else m8[:, :Ls].contiguous()
        ys = torch.empty_like(xs)
        cnt = torch.empty(B, dtype=torch.int64, device=DEV)
        mean = torch.empty(B, H, device=DEV)
        var = torch.empty(B, H, device=DEV)
        cm = torch.empty(B, Ls, H, device=DEV)
        cr = torch.empty(B, Ls, H, device=DEV)
        rc = lib.mega_timestep_norm_fwd(xs.data_ptr(), ys.data_ptr(), M.ops._dtype_code(xs), args[0].data_ptr(),
                                        args[1].data_ptr(), args[2].data_ptr(), args[3].data_ptr(), args[4].data_ptr(),
                                        None if ms is None else ms.data_ptr(), B, Ls, H, 1e-5, cnt.data_ptr(),
                                        mean.data_ptr(), var.data_ptr(), cm.data_ptr(), cr.data_ptr(), None, 0, None)
        torch.cuda.synchronize()
        return rc, ys, cm, cr

    assert serial(L)[0] == -3                                    # MEGA_ERR_WORKSPACE
    rc, ys, cm, cr = serial(128)
    assert rc == 0
    assert rel_err(host(out[0][:, :128]), host(ys)) < (1e-5 if dtype is torch.float32 else 1e-2)
    assert rel_err(host(out[4][:, :128]), host(cm)) < 1e-5 and rel_err(host(out[5][:, :128]), host(cr)) < 1e-5


def test_headline_shape_against_closed_form():
    """B4 x L4096 x D1024, 16 groups, bf16: the textbook cumulative statistics in fp64."""
    rng = np.random.default_rng(1236)
    B, L, H, G = 4, 4096, 1024, 16
    x, x64 = rounded(rng.normal(size=(B, L, H)), torch.bfloat16)
    tn = M.TimestepNorm(H, G).to(DEV).eval()
    with torch.no_grad():
        y = tn(x)
        y2 = tn(x)
    torch.cuda.synchronize()
    assert M.ops.timestep_norm_status() == 0
    assert torch.equal(y, y2)                   # deterministic, workspace left clean
    yc, _, _ = O.timestep_norm_closed_form(x64, None, G)
    assert rel_err(host(y), yc) < TOL[torch.bfloat16]
    # the bf16 rounding of y is the only error source that matters: compare before rounding
    err = np.abs(host(y) - yc)
    assert np.median(err) < 4e-3


def test_errors():
    x = torch.zeros(1, 4, 30, device=DEV)
    z = torch.zeros(1, 4, device=DEV)
    with pytest.raises(RuntimeError, match="divisible"):
        M.ops.group_timestep_norm_fwd(x, torch.zeros(1, dtype=torch.int64, device=DEV), z, z,
                                      torch.ones(30, device=DEV), torch.zeros(30, device=DEV), None, 4, 1e-5)
