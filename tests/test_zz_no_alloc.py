"""mega_group_timestep_norm_fwd_noalloc (tile records in the library's own device array, no
workspace argument, nothing allocated by the call) against mega_group_timestep_norm_fwd on the
same inputs: same kernel, so the results must agree bit for bit.  Two calls in a row, the second on
a smaller input (the array still holds the first call's records), then a shape that does not fit."""
import pytest
import torch

import fairseq_apollo_amd as M
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def _run(entry, x, mask, G, prior, ws):
    lib = M._lib.load()
    B, L, H = x.shape
    pc = torch.full((B,), prior, dtype=torch.int64, device=DEV)
    g = torch.Generator().manual_seed(7)
    pm = (torch.randn(B, G, generator=g) * 0.1).to(DEV)
    pv = (torch.rand(B, G, generator=g) + 0.5).to(DEV)
    gamma = (torch.randn(H, generator=g) * 0.1 + 1).to(DEV)
    beta = (torch.randn(H, generator=g) * 0.1).to(DEV)
    y = torch.empty_like(x)
    count = torch.empty(B, dtype=torch.int64, device=DEV)
    mean = torch.empty(B, G, device=DEV)
    var = torch.empty(B, G, device=DEV)
    gm, cm, cr = (torch.empty(B, L, G, device=DEV) for _ in range(3))
    m8 = None if mask is None else mask.view(torch.uint8)
    stream = torch.cuda.current_stream().cuda_stream
    args = [x.data_ptr(), y.data_ptr(), M.ops._dtype_code(x), pc.data_ptr(), pm.data_ptr(), pv.data_ptr(),
            gamma.data_ptr(), beta.data_ptr(), None if m8 is None else m8.data_ptr(), B, L, H, G, 1e-5,
            count.data_ptr(), mean.data_ptr(), var.data_ptr(), gm.data_ptr(), cm.data_ptr(), cr.data_ptr()]
    if entry == "noalloc":
        rc = lib.mega_group_timestep_norm_fwd_noalloc(*args, stream)
    else:
        rc = lib.mega_group_timestep_norm_fwd(*args, ws.data_ptr(), ws.numel(), stream)
    M._lib.check(rc, entry)
    torch.cuda.synchronize()
    return y, count, mean, var, gm, cm, cr


def _case(B, L, H, G, dtype, masked, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, L, H, generator=g).to(dtype).to(DEV)
    mask = None
    if masked:
        mask = (torch.rand(B, L, generator=g) < 0.2).to(DEV)
    return x, mask


def test_noalloc_matches_workspace_entry_twice_then_rejects_oversize():
    lib = M._lib.load()
    # the status word through which a failed wait is reported: created once per device, outside any capture
    assert lib.mega_lookback_init() == 0
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)
    # first call: the headline activation shape; second call: a smaller, ragged, masked one
    for (B, L, H, G, dtype, masked, seed) in [(4, 4096, 1024, 16, torch.bfloat16, False, 1),
                                             (3, 333, 256, 8, torch.float32, True, 2),
                                             (2, 1000, 512, 16, torch.bfloat16, True, 3)]:
        x, mask = _case(B, L, H, G, dtype, masked, seed)
        got = _run("noalloc", x, mask, G, 3, None)
        ref = _run("workspace", x, mask, G, 3, ws)
        for a, b, name in zip(got, ref, ("y", "count", "mean", "var", "group_mean", "cummean", "cumrstd")):
            assert torch.equal(a, b), f"{name} differs at shape {(B, L, H, G)}"
        assert not torch.isnan(got[0].float()).any()
    # tile and block records beyond the array: 256 + B * (T + ceil(T / 32)) * (2 G + 1) * 8 > 1 MiB, T = ceil(L / TT)
    need = lib.mega_timestep_norm_workspace_bytes(1, 64, 16384, 1024, 16)
    assert need > (1 << 20)
    a = 0x10000
    rc = lib.mega_group_timestep_norm_fwd_noalloc(a, a, 1, a, a + 0x1000, a + 0x2000, a, a, None, 64, 16384, 1024, 16,
                                                  1e-5, a + 0x3000, a + 0x4000, a + 0x5000, None, None, None, None)
    assert rc == -2 and b"fixed scratch" in lib.mega_last_error()
