"""The C-ABI library loads and exports every symbol include/mega_hip.h declares, the ctypes
table covers the same set, and argument checks answer without a GPU."""
import ctypes
import os
import re

import pytest

from conftest import ROOT

import fairseq_apollo_amd as M


def _declared():
    text = open(os.path.join(ROOT, "include", "mega_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mega_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert len(names) >= 15
    lib = ctypes.CDLL(M._lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/mega_hip.h but not exported"
    assert sorted(M._lib.SIGNATURES) == names


def test_argument_checks_need_no_gpu():
    lib = M._lib.load()
    assert lib.mega_abi_version() == 3
    # bad dtype is rejected before anything touches a device
    rc = lib.mega_swiglu_fwd(None, None, None, 7, 16, None)
    assert rc == -1 and b"dtype" in lib.mega_last_error()
    rc = lib.mega_group_timestep_norm_fwd(None, None, 1, None, None, None, None, None, None, 2, 8, 30, 4, 1e-5,
                                          None, None, None, None, None, None, None, 0, None)
    assert rc == -1 and b"multiple" in lib.mega_last_error()
    rc = lib.mega_ema_fwd(None, None, 1, 0, 0, 0, 0, 0, 0, None, None, None, 1, None, None, None, None, 2, 8, 64, 16,
                          0, 0, 1, None, None, 0, None)
    assert rc == -2 and b"ndim" in lib.mega_last_error()
    assert lib.mega_timestep_norm_workspace_bytes(1, 4, 4096, 1024, 16) > 0
    assert lib.mega_ema_fwd_workspace_bytes(4, 1024, 16, 4096, 0, 0) > 0


def test_state_aliasing_rules_answer_without_a_gpu():
    """The decode step and the norms reject a count that overlaps prev_count (several workgroups
    read the old value while one writes the new one); the check runs before anything is launched,
    so made-up addresses are enough."""
    lib = M._lib.load()
    a = 0x10000   # never dereferenced
    step = lambda pc, c: lib.mega_norm_ema_step(a, a, a, 1, pc, a, a, c, a, a, a, a, 1e-5, a, a, a, 1, a, a, a,
                                                4, 64, 4, 16, None)
    assert step(0x20000, 0x20000) == -1 and b"overlap" in lib.mega_last_error()
    assert step(0x20000, 0x20000 + 24) == -1          # partial overlap of the 4 x 8 bytes
    gtsn = lambda pc, pm, pv, c, m, v: lib.mega_group_timestep_norm_fwd(
        a, a, 1, pc, pm, pv, a, a, None, 2, 8, 64, 4, 1e-5, c, m, v, None, None, None, None, 0, None)
    assert gtsn(0x20000, 0x30000, 0x40000, 0x20000, 0x50000, 0x60000) == -1 and b"overlap" in lib.mega_last_error()
    assert gtsn(0x20000, 0x30000, 0x40000, 0x70000, 0x30000, 0x60000) == -1
    assert gtsn(0x20000, 0x30000, 0x40000, 0x70000, 0x50000, 0x40000 + 28) == -1
    ftsn = lib.mega_timestep_norm_fwd(a, a, 1, 0x20000, a, a, a, a, None, 2, 8, 64, 1e-5, 0x20008, a, a, None, None,
                                      None, 0, None)
    assert ftsn == -1 and b"overlap" in lib.mega_last_error()


def test_ops_reject_cpu_tensors():
    import torch
    x = torch.zeros(1, 4, 8)
    with pytest.raises(RuntimeError, match="HIP device"):
        M.ops.swiglu(x, x)
    with pytest.raises(RuntimeError, match="HIP device"):
        M.ops.attention_softmax_fwd(x, 0.0, True)


def test_give_up_status_is_reported_once_by_the_next_call():
    """Host logic of the bounded-wait status: a raised status word makes the next call of an entry point that
    launches a look-back kernel return MEGA_ERR_LAUNCH before anything else is looked at, and clears the
    word; the call after that is judged on its own arguments again.  (On a box without a GPU a plain host
    word stands in for the pinned one the kernels write.)"""
    lib = M._lib.load()
    a = 0x10000   # never dereferenced
    gtsn = lambda: lib.mega_group_timestep_norm_fwd(None, None, 1, None, None, None, None, None, None, 2, 8, 30, 4,
                                                    1e-5, None, None, None, None, None, None, None, 0, None)
    fused = lambda: lib.mega_norm_ema_fwd(a, a, a, 9, 0, 0, 0, a, a, a, a, a, None, 1e-5, a, a, a, a, a, a, 1, a,
                                          None, None, 1, 1024, 64, 1, 16, None, None, 0, None, 0, None)
    assert lib.mega_lookback_status(0) == 0
    try:
        for call, plain_rc in ((gtsn, -1), (fused, -1)):
            lib.mega_test_lookback(0, 0, 1)
            assert lib.mega_lookback_status(0) == 1
            assert call() == -4 and b"gave up" in lib.mega_last_error()
            assert lib.mega_lookback_status(0) == 0          # reported once
            assert call() == plain_rc and b"gave up" not in lib.mega_last_error()
        lib.mega_test_lookback(0, 0, 1)
        assert lib.mega_lookback_status(1) == 1 and lib.mega_lookback_status(0) == 0
        lib.mega_test_lookback(0, 0, 1)
        with pytest.raises(RuntimeError, match="gave up"):
            M.ops.check_lookback("test")
        M.ops.check_lookback("test")                         # cleared
    finally:
        lib.mega_test_lookback(0, 0, 0)
        lib.mega_lookback_status(1)
