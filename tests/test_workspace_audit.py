"""Host-side audit of the address ranges of the backward entry points that partition a workspace
(mega_attention_bwd, mega_gate_qk_bwd, mega_ema_param_grad, mega_(group_)timestep_norm_bwd).

No GPU: under mega_audit_begin() these entry points launch nothing; for every launch they would make they compute the
last byte each operand is addressed at, from the sizes and strides the kernel would receive, and check it against the
registered byte ranges of the call's tensors and workspace (made-up addresses here).  The shapes are the ones the GPU
tests, the sweeps and the training benchmark of configs[4] use, plus ragged ones around the kernels' tile sizes.  The
workspace is registered with exactly `*_workspace_bytes` bytes, so a consumer that addresses one byte more fails."""
import ctypes as C

import pytest

import fairseq_apollo_amd as M

BF16, F16, F32 = 1, 2, 0


class Arena:
    """Made-up, well separated, 4 KiB aligned addresses; every range is registered with the audit."""

    def __init__(self, lib):
        self.lib = lib
        self.next = 0x10000000

    def take(self, nbytes, register=True):
        base = self.next
        self.next += (int(nbytes) + 0xFFFF) // 0x10000 * 0x10000 + 0x10000      # a guard gap after every range
        if register:
            assert self.lib.mega_audit_add(base, int(nbytes)) == 0
        return base


def _finish(lib, rc, min_checks):
    n = C.c_int(0)
    bad = lib.mega_audit_end(C.byref(n))
    assert rc == 0, lib.mega_last_error()
    assert bad == 0, lib.mega_last_error()
    assert n.value >= min_checks, n.value


ATT_SHAPES = [
    # B, L, Nh, H1, H2
    (4, 2048, 4, 128, 1024),      # configs[4]: chunks of the layer's training step
    (2, 4096, 4, 128, 1024),
    (1, 512, 1, 64, 64), (2, 256, 2, 64, 128), (3, 64, 2, 8, 8), (1, 72, 1, 16, 24),
    (2, 100, 3, 32, 40),          # L % 8 != 0: the transposed-copy route
    (1, 37, 1, 8, 16), (2, 1000, 2, 128, 256), (1, 520, 2, 64, 264), (5, 8, 1, 8, 8), (1, 1, 1, 8, 8),
    (1, 16384, 1, 64, 64),
]


@pytest.mark.parametrize("B,L,Nh,H1,H2", ATT_SHAPES)
@pytest.mark.parametrize("causal", [1, 0])
@pytest.mark.parametrize("with_y", [True, False])
@pytest.mark.parametrize("dtype", [BF16, F16])
def test_attention_bwd_stays_inside_its_tensors_and_workspace(B, L, Nh, H1, H2, causal, with_y, dtype):
    lib = M._lib.load()
    es = 2
    lib.mega_audit_begin()
    a = Arena(lib)
    qk, vv, ww = B * L * Nh * H1 * es, B * L * Nh * H2 * es, B * Nh * L * L * es
    dy, q, k, v, w = a.take(vv), a.take(qk), a.take(qk), a.take(vv), a.take(ww)
    y = a.take(vv) if with_y else None
    dq, dk, dv = a.take(qk), a.take(qk), a.take(vv)
    need = lib.mega_attention_bwd_workspace_bytes(dtype, B, L, Nh, H1, H2)
    assert need > 0
    ws = a.take(need)
    rc = lib.mega_attention_bwd(dy, q, k, v, w, y, dq, dk, dv, dtype, B, L, Nh, H1, H2, 0.25, causal, ws, need, None)
    _finish(lib, rc, 12)


def test_audit_catches_a_workspace_that_is_one_byte_short():
    lib = M._lib.load()
    B, L, Nh, H1, H2 = 2, 64, 3, 32, 40
    es = 2
    qk, vv, ww = B * L * Nh * H1 * es, B * L * Nh * H2 * es, B * Nh * L * L * es
    need = lib.mega_attention_bwd_workspace_bytes(BF16, B, L, Nh, H1, H2)
    # the row sums of the softmax backward are the last segment of the workspace (B Nh L floats, padded to 256 bytes):
    # a workspace that ends one byte before their end must be noticed, one that ends exactly there must pass
    rows = B * Nh * L * 4
    end_of_rows = need - (rows + 255) // 256 * 256 + rows
    for registered, expect_bad in ((end_of_rows, False), (end_of_rows - 1, True)):
        lib.mega_audit_begin()
        a = Arena(lib)
        dy, q, k, v, w, y = a.take(vv), a.take(qk), a.take(qk), a.take(vv), a.take(ww), a.take(vv)
        dq, dk, dv = a.take(qk), a.take(qk), a.take(vv)
        ws = a.take(need, register=False)
        assert lib.mega_audit_add(ws, registered) == 0
        rc = lib.mega_attention_bwd(dy, q, k, v, w, y, dq, dk, dv, BF16, B, L, Nh, H1, H2, 1.0, 1, ws, need, None)
        bad = lib.mega_audit_end(None)
        assert rc == 0 and (bad >= 1) == expect_bad, (registered, bad)
    assert b"outside every registered range" in lib.mega_last_error()
    # and a tensor that is too small for its shape
    lib.mega_audit_begin()
    a = Arena(lib)
    dy, q, k, v, w = a.take(vv), a.take(qk - 16), a.take(qk), a.take(vv), a.take(ww)
    dq, dk, dv = a.take(qk), a.take(qk), a.take(vv)
    ws = a.take(need)
    rc = lib.mega_attention_bwd(dy, q, k, v, w, None, dq, dk, dv, BF16, B, L, Nh, H1, H2, 1.0, 1, ws, need, None)
    assert rc == 0 and lib.mega_audit_end(None) >= 1


@pytest.mark.parametrize("T,S,heads", [(8192, 512, 4), (16384, 512, 1), (1, 64, 1), (300, 128, 2), (70000, 256, 4),
                                       (5000, 1024, 8), (33, 8, 1)])
@pytest.mark.parametrize("dtype", [BF16, F32])
def test_gate_qk_bwd(T, S, heads, dtype):
    lib = M._lib.load()
    es = 4 if dtype == F32 else 2
    if S > 2 * 64 * (16 // es):
        pytest.skip("outside the kernel's envelope (the host runs torch operations there)")
    lib.mega_audit_begin()
    a = Arena(lib)
    zs = S + 64                                           # z is a slice of the wider mx_proj output
    dq, dk, dz = a.take(T * S * es), a.take(T * S * es), a.take(T * S * es)
    z = a.take(((T - 1) * zs + S) * es)
    gamma, freqs = a.take(2 * S * 4), a.take(S // heads // 2 * 4)
    dgamma, dbeta = a.take(2 * S * 4), a.take(2 * S * 4)
    need = lib.mega_gate_qk_bwd_workspace_bytes(T, S)
    ws = a.take(need)
    rc = lib.mega_gate_qk_bwd(dq, dk, z, zs, gamma, freqs, dz, dgamma, dbeta, dtype, T, S, heads, 2048, 0, 1e-5, ws,
                              need, None)
    _finish(lib, rc, 7)


@pytest.mark.parametrize("B,D,N,L", [(4, 1024, 16, 4096), (1, 2048, 16, 8192), (2, 100, 7, 333), (3, 8, 1, 5),
                                     (16, 1024, 16, 1024), (1, 24, 32, 64)])
@pytest.mark.parametrize("layout", ["rows", "time_major"])
@pytest.mark.parametrize("reverse", [0, 1])
def test_ema_param_grad(B, D, N, L, layout, reverse):
    lib = M._lib.load()
    if N > 16:
        pytest.skip("sixteen states at a time: the host splits larger layers")
    lib.mega_audit_begin()
    a = Arena(lib)
    es = 2
    dy, x = a.take(B * D * L * es), a.take(B * D * L * es)
    sb, sd, sl = (D * L, L, 1) if layout == "rows" else (L * D, 1, D)
    p, q, g = a.take(D * N * 4), a.take(D * N * 8), a.take(D * N * 8)
    dp, dq, dg, dom = a.take(D * N * 4), a.take(D * N * 8), a.take(D * N * 8), a.take(D * 4)
    need = lib.mega_ema_param_grad_workspace_bytes(B, D, N)
    ws = a.take(need)
    rc = lib.mega_ema_param_grad(dy, x, BF16, sb, sd, sl, sb, sd, sl, p, q, g, None, B, D, N, L, reverse, 0, dp, dq, dg,
                                 dom, ws, need, None)
    _finish(lib, rc, 8)


@pytest.mark.parametrize("B,L,H,G", [(4, 4096, 1024, 16), (1, 8192, 2048, 16), (2, 333, 96, 3), (3, 37, 48, 48),
                                     (1, 1, 32, 2), (2, 1000, 512, 512)])
@pytest.mark.parametrize("dtype", [BF16, F32])
def test_timestep_norm_bwd(B, L, H, G, dtype):
    lib = M._lib.load()
    es = 4 if dtype == F32 else 2
    need = lib.mega_timestep_norm_bwd_workspace_bytes(dtype, B, L, H, G)
    lib.mega_audit_begin()
    a = Arena(lib)
    dy, x, dx = a.take(B * L * H * es), a.take(B * L * H * es), a.take(B * L * H * es)
    pm, cnt = a.take(B * G * 4), a.take(B * 8)
    gm, cm, cr = a.take(B * L * G * 4), a.take(B * L * G * 4), a.take(B * L * G * 4)
    gamma = a.take(H * 4)
    dpm, dpv, dgam, dbet = a.take(B * G * 4), a.take(B * G * 4), a.take(H * 4), a.take(H * 4)
    ws = a.take(need)
    rc = lib.mega_group_timestep_norm_bwd(dy, None, None, x, dtype, pm, cnt, gm, cm, cr, gamma, None, B, L, H, G, dx,
                                          dpm, dpv, dgam, dbet, ws, need, None)
    if rc == -2:
        C.c_int(lib.mega_audit_end(None))
        pytest.skip("outside the envelope of the tiled backward")
    _finish(lib, rc, 8)
