"""Operator surface: the functions fairseq model code reaches through
`fairseq.mega2_extension.ops` (fairseq/csrc/mega2_extension.cc:14-24), with the same names,
argument order and return tuples, plus the fused inference entry points the modules use.

Every function takes torch tensors that live on a HIP device, allocates its outputs with
torch (so they belong to the caller, as torch::empty_like does in the reference), and
enqueues the HIP kernels of libmega_hip.so on torch's current stream.  CPU tensors are
rejected: there is no fallback.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import BF16, F16, F32

_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise RuntimeError(f"unsupported activation dtype {t.dtype} (float32, bfloat16, float16)") from None


def _need_gpu(*ts) -> torch.device:
    dev = None
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("mega HIP ops need tensors on a HIP device; there is no CPU path")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream(dev: torch.device) -> int:
    """Raw handle of torch's current stream on `dev` (the launch stream of every call)."""
    return torch._C._cuda_getCurrentRawStream(dev.index)


class _on_device:
    """`with _on_device(dev):` makes `dev` the current HIP device for the launch; free when it
    already is (the usual case: one process per GPU)."""
    __slots__ = ("idx", "prev")

    def __init__(self, dev: torch.device):
        self.idx = dev.index
        self.prev = -1

    def __enter__(self):
        cur = torch._C._cuda_getDevice()
        if cur != self.idx:
            self.prev = cur
            torch._C._cuda_setDevice(self.idx)

    def __exit__(self, *exc):
        if self.prev >= 0:
            torch._C._cuda_setDevice(self.prev)
        return False


def _f32c(t: torch.Tensor) -> torch.Tensor:
    if t.dtype is torch.float32 and not t.requires_grad and t.is_contiguous():
        return t
    return t.detach().to(torch.float32).contiguous()


def _cplx_as_f32(t: torch.Tensor) -> torch.Tensor:
    """complex [...] -> float32 [..., 2]; real [...] -> [..., 2] with a zero imaginary part."""
    t = t.detach()
    if t.is_complex():
        return torch.view_as_real(t.to(torch.complex64).resolve_conj().contiguous()).contiguous()
    return torch.stack([t.to(torch.float32), torch.zeros_like(t, dtype=torch.float32)], dim=-1).contiguous()


_tsn_ws = {}


def _tsn_workspace(dev: torch.device, nbytes: int, stream: Optional[int] = None) -> torch.Tensor:
    """Zero-filled once, then owned by the TimestepNorm calls (launch epoch + tile records); one per
    (device, stream)."""
    key = (dev.index, _stream(dev) if stream is None else stream)
    ws = _tsn_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 16), dtype=torch.uint8, device=dev)
        _tsn_ws[key] = ws
    return ws


_scratch = {}


def _scratch_buffer(dev: torch.device, nbytes: int, stream: Optional[int] = None) -> torch.Tensor:
    """Grow-only scratch per (device, stream): calls on one stream are ordered, so they can
    share it; its contents never need to survive a call."""
    key = (dev.index, _stream(dev) if stream is None else stream)
    ws = _scratch.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 16), dtype=torch.uint8, device=dev)
        _scratch[key] = ws
    return ws


def timestep_norm_status(dev=None, clear: bool = False) -> int:
    """Error word of the TimestepNorm workspaces of `dev` (non-zero: a tile gave up waiting for
    an earlier tile).  Synchronises; meant for tests and debugging (lookback_status is the view
    that does not synchronise)."""
    bad = 0
    for (idx, _), ws in _tsn_ws.items():
        if dev is None or torch.device(dev).index in (None, idx):
            bad |= int(ws[8:12].view(torch.int32).item())
            if clear:
                ws[8:12].zero_()
    return bad


def lookback_status(clear: bool = False) -> int:
    """Status word of the current device's bounded waits (mega_lookback_status): non-zero once a tile of a
    TimestepNorm or block launch has given up waiting for an earlier tile.  Does not synchronise: a launch that
    is still running may set it later."""
    return int(_lib.load().mega_lookback_status(1 if clear else 0))


def lookback_checked(on: bool) -> None:
    """Checked mode of the bounded waits (mega_lookback_checked): the calls that launch such kernels wait for
    their stream and raise for a give-up of that very call.  Off by default."""
    _lib.load().mega_lookback_checked(1 if on else 0)


def check_lookback(where: str = "") -> None:
    """Raise (and clear the status) if a launch has given up since the last check.  The library does the same
    at the start of the calls that launch such kernels; streaming helpers call this once more when they are
    done, so that a failure in their last chunks does not wait for an unrelated later call."""
    if lookback_status(clear=True):
        raise RuntimeError(f"{where or 'mega'}: a TimestepNorm / moving-average launch gave up waiting for an "
                           "earlier time tile and has written NaN into the outputs and statistics that depended on "
                           "it (workgroups not dispatched in id order, or one workspace used by overlapping launches)")


# --------------------------------------------------------------------------------------
# ops with the reference's names
# --------------------------------------------------------------------------------------


def ema_coeffs_fwd(alpha: torch.Tensor, delta: torch.Tensor, third: torch.Tensor, gamma: torch.Tensor,
                   omega: torch.Tensor, is_complex: bool):
    """The layer's coefficients from its stored parameters in one launch
    (complex_exponential_moving_average.py:79-96 / exponential_moving_average.py:71-80): alpha, delta [K, N, 1];
    third = theta [K, 1, 1] (complex) or beta [K, N, 1] (real); gamma [K, N, 2] or [K, N]; omega [D(, 1)], all of one
    dtype.  -> (p [K, N], q [K, N, 2], gamma [K, N, 2], omega [D]) in fp32, the library's own layout."""
    dev = _need_gpu(alpha, delta, third, gamma, omega)
    lib = _lib.load()
    K, N = alpha.shape[0], alpha.shape[1]
    D = omega.numel()
    ts = [t.detach().contiguous() for t in (alpha, delta, third, gamma, omega)]
    if len({t.dtype for t in ts}) != 1:
        raise RuntimeError("ema_coeffs_fwd: the parameters must share one dtype")
    if ts[1].numel() != K * N or ts[2].numel() != (K if is_complex else K * N) or \
            ts[3].numel() != (2 * K * N if is_complex else K * N):
        raise RuntimeError("ema_coeffs_fwd: parameter shapes do not belong to one layer")
    p = torch.empty(K, N, dtype=torch.float32, device=dev)
    q = torch.empty(K, N, 2, dtype=torch.float32, device=dev)
    g = torch.empty(K, N, 2, dtype=torch.float32, device=dev)
    om = torch.empty(D, dtype=torch.float32, device=dev)
    with _on_device(dev):
        rc = lib.mega_ema_coeffs_fwd(_ptr(ts[0]), _ptr(ts[1]), _ptr(ts[2]), _ptr(ts[3]), _ptr(ts[4]), _dtype_code(ts[0]),
                                     1 if is_complex else 0, K, N, D, _ptr(p), _ptr(q), _ptr(g), _ptr(om), _stream(dev))
    _lib.check(rc, "ema_coeffs_fwd")
    return p, q, g, om


def ema_coeffs_bwd(p_grad: torch.Tensor, q_grad: torch.Tensor, g_grad: torch.Tensor, om_grad: torch.Tensor,
                   alpha: torch.Tensor, delta: torch.Tensor, third: torch.Tensor, gamma_like: torch.Tensor,
                   omega_like: torch.Tensor, is_complex: bool):
    """Backward of ema_coeffs_fwd: gradients of (p [K, N], q, gamma [K, N, 2] as (re, im) pairs -- [K, N] for the real
    layer --, omega [D]) in fp32 -> gradients of (alpha, delta, third, gamma, omega) in the parameters' dtype and
    shapes."""
    dev = _need_gpu(p_grad, q_grad, g_grad, om_grad, alpha, delta, third)
    lib = _lib.load()
    K, N = alpha.shape[0], alpha.shape[1]
    D = omega_like.numel()
    a, d, t = (x.detach().contiguous() for x in (alpha, delta, third))
    gs = [_f32c(x) for x in (p_grad, q_grad, g_grad, om_grad)]
    pair = 2 if is_complex else 1
    if gs[0].numel() != K * N or gs[1].numel() != pair * K * N or gs[2].numel() != pair * K * N or gs[3].numel() != D:
        raise RuntimeError("ema_coeffs_bwd: gradient shapes do not belong to this layer")
    outs = [torch.empty(x.shape, dtype=a.dtype, device=dev) for x in (alpha, delta, third, gamma_like, omega_like)]
    with _on_device(dev):
        rc = lib.mega_ema_coeffs_bwd(_ptr(gs[0]), _ptr(gs[1]), _ptr(gs[2]), _ptr(gs[3]), _ptr(a), _ptr(d), _ptr(t),
                                     _dtype_code(a), 1 if is_complex else 0, K, N, D, _ptr(outs[0]), _ptr(outs[1]),
                                     _ptr(outs[2]), _ptr(outs[3]), _ptr(outs[4]), _stream(dev))
    _lib.check(rc, "ema_coeffs_bwd")
    return tuple(outs)


def norm_params_fwd(weight: torch.Tensor, bias: torch.Tensor, prior_mean: torch.Tensor, prior_logv: torch.Tensor,
                    batch_size: int):
    """What TimestepNorm.forward derives from its parameters on every call (timestep_norm.py:118-131), in one
    launch: -> (weight + 1 [H], bias [H], prior mean [B, G], exp(prior log-variance) [B, G]) in fp32."""
    dev = _need_gpu(weight, bias, prior_mean, prior_logv)
    lib = _lib.load()
    H, G, B = weight.numel(), prior_mean.numel(), int(batch_size)
    w, b, pm, pl = (x.detach().contiguous() for x in (weight, bias, prior_mean, prior_logv))
    if w.dtype != b.dtype or pm.dtype != pl.dtype or b.numel() != H or pl.numel() != G:
        raise RuntimeError("norm_params_fwd: weight / bias and prior_mean / prior_logv must pair up")
    gamma = torch.empty(H, dtype=torch.float32, device=dev)
    beta = torch.empty(H, dtype=torch.float32, device=dev)
    mean = torch.empty(B, G, dtype=torch.float32, device=dev)
    var = torch.empty(B, G, dtype=torch.float32, device=dev)
    with _on_device(dev):
        rc = lib.mega_norm_params_fwd(_ptr(w), _ptr(b), _dtype_code(w), _ptr(pm), _ptr(pl), _dtype_code(pm), H, G, B,
                                      _ptr(gamma), _ptr(beta), _ptr(mean), _ptr(var), _stream(dev))
    _lib.check(rc, "norm_params_fwd")
    return gamma, beta, mean, var


def norm_params_bwd(gamma_grad: torch.Tensor, beta_grad: torch.Tensor, mean_grad: Optional[torch.Tensor],
                    var_grad: Optional[torch.Tensor], weight: torch.Tensor, prior_mean: torch.Tensor,
                    prior_logv: torch.Tensor, batch_size: int, prior_needs_grad: bool):
    """Backward of norm_params_fwd -> (weight_grad, bias_grad, prior_mean_grad, prior_logv_grad) in the
    parameters' dtypes; the prior's are None unless prior_needs_grad."""
    dev = _need_gpu(gamma_grad, beta_grad, weight, prior_logv)
    lib = _lib.load()
    H, G, B = weight.numel(), prior_mean.numel(), int(batch_size)
    gg, gb = _f32c(gamma_grad), _f32c(beta_grad)
    dw = torch.empty(weight.shape, dtype=weight.dtype, device=dev)
    db = torch.empty(weight.shape, dtype=weight.dtype, device=dev)
    dpm = dpl = gm = gv = None
    pl = prior_logv.detach().contiguous()
    if prior_needs_grad:
        gm = torch.zeros(B, G, dtype=torch.float32, device=dev) if mean_grad is None else _f32c(mean_grad)
        gv = torch.zeros(B, G, dtype=torch.float32, device=dev) if var_grad is None else _f32c(var_grad)
        dpm = torch.empty(prior_mean.shape, dtype=prior_mean.dtype, device=dev)
        dpl = torch.empty(prior_mean.shape, dtype=prior_mean.dtype, device=dev)
    with _on_device(dev):
        rc = lib.mega_norm_params_bwd(_ptr(gg), _ptr(gb), _ptr(gm), _ptr(gv), _ptr(pl), _dtype_code(weight),
                                      _dtype_code(pl), H, G, B, _ptr(dw), _ptr(db), _ptr(dpm), _ptr(dpl), _stream(dev))
    _lib.check(rc, "norm_params_bwd")
    return dw, db, dpm, dpl


def ema_parameters_fwd(p: torch.Tensor, log_q: torch.Tensor, gamma: torch.Tensor,
                       h: Optional[torch.Tensor], L: int):
    """-> (w[K,L], b[B,K,L] or None, None).  Reference: ema_parameters_fwd,
    fairseq/csrc/ops/ema_parameters.cc:211-286.  The Vandermonde tensor the reference saves
    for its backward pass is not produced (third value None)."""
    dev = _need_gpu(p, log_q, gamma, h)
    lib = _lib.load()
    K, N = p.shape[0], p.shape[1]
    pf = _f32c(p).reshape(K, N)
    lq = _cplx_as_f32(log_q.reshape(K, N))
    g = _cplx_as_f32(gamma.reshape(K, N))
    w = torch.empty(K, L, dtype=torch.float32, device=dev)
    hb = b = None
    B = 0
    if h is not None:
        B = h.shape[0]
        hb = _cplx_as_f32(h.reshape(B, K, N))
        b = torch.empty(B, K, L, dtype=torch.float32, device=dev)
    with _on_device(dev):
        rc = lib.mega_ema_parameters_fwd(_ptr(pf), _ptr(lq), _ptr(g), _ptr(hb), B, K, N, L, _ptr(w), _ptr(b),
                                         _stream(dev))
    _lib.check(rc, "ema_parameters_fwd")
    return w, b, None


def ema_hidden_fwd(x: torch.Tensor, p: torch.Tensor, log_q: torch.Tensor, h: Optional[torch.Tensor]):
    """-> (h'[B,D,N] complex64, None).  Reference: ema_hidden_fwd,
    fairseq/csrc/ops/ema_hidden.cc:163-194."""
    dev = _need_gpu(x, p, log_q, h)
    lib = _lib.load()
    B, D, L = x.shape
    N = p.shape[1]
    pf = _f32c(p).reshape(D, N)
    lq = _cplx_as_f32(log_q.reshape(D, N))
    hb = None if h is None else _cplx_as_f32(h.reshape(B, D, N))
    out = torch.empty(B, D, N, 2, dtype=torch.float32, device=dev)
    nws = lib.mega_ema_hidden_workspace_bytes(B, D, N, L)
    ws = torch.empty(nws, dtype=torch.uint8, device=dev)
    xd = x.detach()
    with _on_device(dev):
        rc = lib.mega_ema_hidden_fwd(_ptr(xd), _dtype_code(xd), xd.stride(0), xd.stride(1), xd.stride(2), _ptr(pf),
                                     _ptr(lq), _ptr(hb), B, D, N, L, _ptr(out), _ptr(ws), nws, _stream(dev))
    _lib.check(rc, "ema_hidden_fwd")
    return torch.view_as_complex(out), None


def _norm_state(prev_count, prev_mean, prev_var, B, G, dev):
    pc = prev_count
    if not (pc.dtype is torch.int64 and pc.device == dev and pc.is_contiguous()):
        pc = pc.detach().to(device=dev, dtype=torch.int64).contiguous()
    pm = _f32c(prev_mean)
    pv = _f32c(prev_var)
    if pm.numel() != B * G or pv.numel() != B * G or pc.numel() != B:
        raise RuntimeError(f"carried state must hold {B} counts and {B}x{G} means / variances")
    return pc, pm, pv


_ws_bytes_cache = {}


def _mask_u8(mask: Optional[torch.Tensor], B: int, L: int):
    if mask is None:
        return None
    m = mask.detach()
    if m.shape != (B, L):
        raise RuntimeError(f"padding_mask must have shape ({B}, {L}), got {tuple(m.shape)}")
    if m.dtype == torch.bool:
        return m.contiguous().view(torch.uint8)
    return (m != 0).contiguous().view(torch.uint8)


def group_timestep_norm_fwd(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, num_groups: int,
                            eps: float, need_stats: bool = True):
    """-> (y, count[B] int64, mean[B,G], var[B,G], group_mean, cummean, cumrstd) with the last
    three [B,L,G] fp32 (None when need_stats is False; they only serve a backward pass).
    Reference: group_timestep_norm_fwd, fairseq/csrc/ops/timestep_norm.cc:568-636.
    mean / var are carried in fp32 whatever the activation dtype."""
    dev = _need_gpu(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask)
    lib = _lib.load()
    if x.dim() != 3:
        raise RuntimeError("x must be [B, L, H]")
    B, L, H = x.shape
    G = int(num_groups)
    if G <= 0 or H % G != 0:
        raise RuntimeError(f"num_features={H} is not divisible by num_groups={G}")
    xd = x if (x.is_contiguous() and not x.requires_grad) else x.detach().contiguous()
    dt = _dtype_code(xd)
    y = torch.empty_like(xd)
    pc, pm, pv = _norm_state(prev_count, prev_mean, prev_var, B, G, dev)
    count = torch.empty(B, dtype=torch.int64, device=dev)
    mean = torch.empty(B, G, dtype=torch.float32, device=dev)
    var = torch.empty(B, G, dtype=torch.float32, device=dev)
    gm = cm = cr = None
    if need_stats:
        gm = torch.empty(B, L, G, dtype=torch.float32, device=dev)
        cm = torch.empty_like(gm)
        cr = torch.empty_like(gm)
    key = ("tsn", dt, B, L, H, G)
    nws = _ws_bytes_cache.get(key)
    if nws is None:
        nws = _ws_bytes_cache[key] = lib.mega_timestep_norm_workspace_bytes(dt, B, L, H, G)
    stream = _stream(dev)
    ws = _tsn_workspace(dev, nws, stream)
    m8 = _mask_u8(padding_mask, B, L)
    gf, bf = _f32c(gamma), _f32c(beta)
    with _on_device(dev):
        rc = lib.mega_group_timestep_norm_fwd(_ptr(xd), _ptr(y), dt, _ptr(pc), _ptr(pm), _ptr(pv), _ptr(gf), _ptr(bf),
                                              _ptr(m8), B, L, H, G, float(eps), _ptr(count), _ptr(mean), _ptr(var),
                                              _ptr(gm), _ptr(cm), _ptr(cr), _ptr(ws), ws.numel(), stream)
    _lib.check(rc, "group_timestep_norm_fwd")
    return y, count, mean, var, gm, cm, cr


def timestep_norm_fwd(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask, eps: float,
                      need_stats: bool = True):
    """-> (y, count, mean[B,H], var[B,H], cummean, cumrstd).  Reference: timestep_norm_fwd,
    fairseq/csrc/ops/timestep_norm.cc:452-510 (per-feature running statistics)."""
    dev = _need_gpu(x, prev_count, prev_mean, prev_var, gamma, beta, padding_mask)
    lib = _lib.load()
    B, L, H = x.shape
    xd = x.detach().contiguous()
    dt = _dtype_code(xd)
    y = torch.empty_like(xd)
    pc, pm, pv = _norm_state(prev_count, prev_mean, prev_var, B, H, dev)
    count = torch.empty(B, dtype=torch.int64, device=dev)
    mean = torch.empty(B, H, dtype=torch.float32, device=dev)
    var = torch.empty(B, H, dtype=torch.float32, device=dev)
    cm = cr = None
    if need_stats:
        cm = torch.empty(B, L, H, dtype=torch.float32, device=dev)
        cr = torch.empty_like(cm)
    m8 = _mask_u8(padding_mask, B, L)
    gf, bf = _f32c(gamma), _f32c(beta)
    key = ("tsn_feat", dt, B, L, H)
    nws = _ws_bytes_cache.get(key)
    if nws is None:
        nws = _ws_bytes_cache[key] = lib.mega_timestep_norm_workspace_bytes(dt, B, L, H, H)
    stream = _stream(dev)
    ws = _scratch_buffer(dev, nws, stream) if nws else None      # tile states of the time-parallel kernels
    with _on_device(dev):
        rc = lib.mega_timestep_norm_fwd(_ptr(xd), _ptr(y), dt, _ptr(pc), _ptr(pm), _ptr(pv), _ptr(gf), _ptr(bf),
                                        _ptr(m8), B, L, H, float(eps), _ptr(count), _ptr(mean), _ptr(var), _ptr(cm),
                                        _ptr(cr), _ptr(ws), ws.numel() if ws is not None else 0, stream)
    _lib.check(rc, "timestep_norm_fwd")
    return y, count, mean, var, cm, cr


def _tsn_bwd(name, y_grad, mean_grad, var_grad, x, prev_mean, count, group_mean, cummean, cumrstd, gamma,
             padding_mask, G: int):
    dev = _need_gpu(y_grad, mean_grad, var_grad, x, prev_mean, count, group_mean, cummean, cumrstd, gamma,
                    padding_mask)
    lib = _lib.load()
    if x.dim() != 3 or y_grad.shape != x.shape:
        raise RuntimeError(f"{name}: x and y_grad must be [B, L, H] of the same shape")
    B, L, H = x.shape
    if G <= 0 or H % G != 0:
        raise RuntimeError(f"num_features={H} is not divisible by num_groups={G}")
    xd = x.detach().contiguous()
    dyd = y_grad.detach().to(xd.dtype).contiguous()
    dt = _dtype_code(xd)
    for nm, t in (("cummean", cummean), ("cumrstd", cumrstd)) + ((("group_mean", group_mean),) if group_mean is not None else ()):
        if t.shape != (B, L, G) or t.dtype is not torch.float32:
            raise RuntimeError(f"{name}: {nm} must be the forward's [B, L, G] float32 output")
    f32 = lambda t: None if t is None else _f32c(t).reshape(B, G)
    mg, vg, pm = f32(mean_grad), f32(var_grad), f32(prev_mean)
    cnt = count.detach().to(torch.int64).contiguous()
    if cnt.numel() != B:
        raise RuntimeError(f"{name}: count must be [B]")
    dx = torch.empty_like(xd)
    dpm = torch.empty(B, G, dtype=torch.float32, device=dev)
    dpv = torch.empty(B, G, dtype=torch.float32, device=dev)
    dg = torch.empty(H, dtype=torch.float32, device=dev)
    db = torch.empty(H, dtype=torch.float32, device=dev)
    nws = lib.mega_timestep_norm_bwd_workspace_bytes(dt, B, L, H, G)
    stream = _stream(dev)
    ws = _scratch_buffer(dev, nws, stream)
    m8 = _mask_u8(padding_mask, B, L)
    gm = None if group_mean is None else group_mean.contiguous()
    with _on_device(dev):
        rc = lib.mega_group_timestep_norm_bwd(_ptr(dyd), _ptr(mg), _ptr(vg), _ptr(xd), dt, _ptr(pm), _ptr(cnt),
                                              _ptr(gm), _ptr(cummean.contiguous()), _ptr(cumrstd.contiguous()),
                                              _ptr(_f32c(gamma)), _ptr(m8), B, L, H, G, _ptr(dx), _ptr(dpm),
                                              _ptr(dpv), _ptr(dg), _ptr(db), _ptr(ws), ws.numel(), stream)
    _lib.check(rc, name)
    return dx, dpm, dpv, dg, db


def group_timestep_norm_bwd(y_grad, mean_grad, var_grad, x, prev_mean, count, group_mean, cummean, cumrstd, gamma,
                            padding_mask, num_groups: int):
    """-> (x_grad, prev_mean_grad[B,G], prev_var_grad[B,G], gamma_grad[H], beta_grad[H]); the state
    and parameter gradients are fp32.  Reference: group_timestep_norm_bwd,
    fairseq/csrc/ops/timestep_norm.cc:638-708 (recurrences at :318-450).  mean_grad / var_grad may
    be None (zeros)."""
    return _tsn_bwd("group_timestep_norm_bwd", y_grad, mean_grad, var_grad, x, prev_mean, count, group_mean, cummean,
                    cumrstd, gamma, padding_mask, int(num_groups))


def timestep_norm_bwd(y_grad, mean_grad, var_grad, x, prev_mean, count, cummean, cumrstd, gamma, padding_mask):
    """Per-feature form of group_timestep_norm_bwd.  Reference: timestep_norm_bwd,
    fairseq/csrc/ops/timestep_norm.cc:512-566 (recurrences at :104-217)."""
    return _tsn_bwd("timestep_norm_bwd", y_grad, mean_grad, var_grad, x, prev_mean, count, None, cummean, cumrstd,
                    gamma, padding_mask, x.shape[-1])


def group_sequence_norm_fwd(x, gamma, beta, padding_mask, num_groups: int, eps: float, length_last: bool = False):
    """-> (y, count[B] int64, mean[B,G], rstd[B,G]).  x: [B, L, H], or [B, H, L] with length_last.
    Reference: group_sequence_norm_fwd, fairseq/csrc/ops/sequence_norm.cc:953-1010."""
    dev = _need_gpu(x, gamma, beta, padding_mask)
    lib = _lib.load()
    if x.dim() != 3:
        raise RuntimeError("x must be [B, L, H] (or [B, H, L] with length_last)")
    B = x.shape[0]
    H, L = (x.shape[1], x.shape[2]) if length_last else (x.shape[2], x.shape[1])
    G = int(num_groups)
    if G <= 0 or H % G != 0:
        raise RuntimeError(f"num_features={H} is not divisible by num_groups={G}")
    xd = x.detach().contiguous()
    dt = _dtype_code(xd)
    y = torch.empty_like(xd)
    count = torch.empty(B, dtype=torch.int64, device=dev)
    mean = torch.empty(B, G, dtype=torch.float32, device=dev)
    rstd = torch.empty(B, G, dtype=torch.float32, device=dev)
    stream = _stream(dev)
    ws = _scratch_buffer(dev, lib.mega_sequence_norm_workspace_bytes(dt, B, L, H, G, 1 if length_last else 0), stream)
    m8 = _mask_u8(padding_mask, B, L)
    with _on_device(dev):
        rc = lib.mega_group_sequence_norm_fwd(_ptr(xd), _ptr(y), dt, _ptr(_f32c(gamma)), _ptr(_f32c(beta)), _ptr(m8),
                                              B, L, H, G, float(eps), 1 if length_last else 0, _ptr(count),
                                              _ptr(mean), _ptr(rstd), _ptr(ws), ws.numel(), stream)
    _lib.check(rc, "group_sequence_norm_fwd")
    return y, count, mean, rstd


def sequence_norm_fwd(x, gamma, beta, padding_mask, eps: float, length_last: bool = False):
    """Per-feature form: -> (y, count[B], mean[B,H], rstd[B,H]).  Reference: sequence_norm_fwd,
    fairseq/csrc/ops/sequence_norm.cc:844-900."""
    H = x.shape[1] if length_last else x.shape[2]
    return group_sequence_norm_fwd(x, gamma, beta, padding_mask, H, eps, length_last)


def group_sequence_norm_bwd(y_grad, x, count, mean, rstd, gamma, padding_mask, num_groups: int,
                            length_last: bool = False):
    """-> (x_grad, gamma_grad[H], beta_grad[H]) (parameter gradients in fp32).  Reference:
    group_sequence_norm_bwd, fairseq/csrc/ops/sequence_norm.cc:1012-1063.  The kernels work on
    [B, H, L]; a [B, L, H] call goes through transposed copies."""
    dev = _need_gpu(y_grad, x, count, mean, rstd, gamma, padding_mask)
    lib = _lib.load()
    if x.dim() != 3 or y_grad.shape != x.shape:
        raise RuntimeError("x and y_grad must have the same 3-D shape")
    if not length_last:
        dx, dg, db = group_sequence_norm_bwd(y_grad.transpose(1, 2), x.transpose(1, 2), count, mean, rstd, gamma,
                                             padding_mask, num_groups, True)
        return dx.transpose(1, 2).contiguous(), dg, db
    B, H, L = x.shape
    G = int(num_groups)
    if G <= 0 or H % G != 0:
        raise RuntimeError(f"num_features={H} is not divisible by num_groups={G}")
    xd = x.detach().contiguous()
    gd = y_grad.detach().to(xd.dtype).contiguous()
    dx = torch.empty_like(xd)
    dg = torch.empty(H, dtype=torch.float32, device=dev)
    db = torch.empty(H, dtype=torch.float32, device=dev)
    stream = _stream(dev)
    ws = _scratch_buffer(dev, lib.mega_sequence_norm_bwd_workspace_bytes(B, H, G), stream)
    m8 = _mask_u8(padding_mask, B, L)
    cnt = count.detach().to(torch.int64).contiguous()
    with _on_device(dev):
        rc = lib.mega_group_sequence_norm_bwd(_ptr(gd), _ptr(xd), _dtype_code(xd), _ptr(cnt),
                                              _ptr(_f32c(mean).reshape(B, G)), _ptr(_f32c(rstd).reshape(B, G)),
                                              _ptr(_f32c(gamma)), _ptr(m8), B, L, H, G, _ptr(dx), _ptr(dg), _ptr(db),
                                              _ptr(ws), ws.numel(), stream)
    _lib.check(rc, "group_sequence_norm_bwd")
    return dx, dg, db


def sequence_norm_bwd(y_grad, x, count, mean, rstd, gamma, padding_mask, length_last: bool = False):
    """Per-feature form.  Reference: sequence_norm_bwd, fairseq/csrc/ops/sequence_norm.cc:902-951."""
    H = x.shape[1] if length_last else x.shape[2]
    return group_sequence_norm_bwd(y_grad, x, count, mean, rstd, gamma, padding_mask, H, length_last)


def _dropkey_seed(dropout: float, seed: Optional[int]) -> int:
    """The 64-bit seed that names a DropKey mask: the caller's, or one drawn from torch's CPU
    generator (so torch.manual_seed makes a run repeatable, as it does for the reference's Philox
    offsets, fairseq/csrc/ops/attention_softmax_kernel.cu:44-55)."""
    if not 0.0 <= dropout <= 1.0:
        raise RuntimeError("dropout must lie in [0, 1]")
    if dropout == 0.0:
        return 0
    if seed is None:
        seed = int(torch.randint(0, 2 ** 62, (1,), dtype=torch.int64).item())
    return seed & (2 ** 64 - 1)


def attention_softmax_fwd(x: torch.Tensor, dropout: float, use_causal_mask: bool,
                          seed: Optional[int] = None) -> torch.Tensor:
    """Reference: attention_softmax_fwd, fairseq/csrc/ops/attention_softmax.cc:6-18.  `dropout` is
    DropKey (scores set to -inf with that probability before the softmax); `seed` names the mask."""
    seed = _dropkey_seed(dropout, seed)
    dev = _need_gpu(x)
    lib = _lib.load()
    if x.dim() < 2:
        raise RuntimeError("x must have at least 2 dimensions")
    xd = x.detach().contiguous()
    outer, inner = xd.shape[-2], xd.shape[-1]
    batch = xd.numel() // max(outer * inner, 1)
    y = torch.empty_like(xd)
    with _on_device(dev):
        rc = lib.mega_attention_softmax_fwd(_ptr(xd), _ptr(y), _dtype_code(xd), batch, outer, inner,
                                            1 if use_causal_mask else 0, float(dropout), seed, _stream(dev))
    _lib.check(rc, "attention_softmax_fwd")
    return y


def attention_fwd(q, k, v, scale: float, dropout: float, use_causal_mask: bool, need_weights: bool = False,
                  seed: Optional[int] = None, weights_only: bool = False):
    """-> (y[B,L,Nh,H2], w[B,Nh,L,L] or None).  Reference: attention_fwd,
    fairseq/csrc/ops/attention_kernel.cu:40-131; the L x L weights are only written on request.
    `dropout` is DropKey on the scaled scores, `seed` names the mask (shared with
    attention_softmax_fwd on the [B,Nh,L,L] scores).  `weights_only`: -> (None, w), the second product is not
    formed (what a backward that did not keep the weights asks for; matrix-core shapes only)."""
    need_weights = need_weights or weights_only
    seed = _dropkey_seed(dropout, seed)
    dev = _need_gpu(q, k, v)
    lib = _lib.load()
    if q.dim() != 4 or k.shape != q.shape or v.shape[:3] != q.shape[:3]:
        raise RuntimeError("attention_fwd: q, k must be [B,L,N,H1] and v [B,L,N,H2]")
    qd, kd, vd = (t.detach().contiguous() for t in (q, k, v))
    if not (qd.dtype == kd.dtype == vd.dtype):
        raise RuntimeError("attention_fwd: q, k, v must share one dtype")
    B, L, Nh, H1 = qd.shape
    H2 = vd.shape[3]
    y = None if weights_only else torch.empty(B, L, Nh, H2, dtype=qd.dtype, device=dev)
    w = torch.empty(B, Nh, L, L, dtype=qd.dtype, device=dev) if need_weights else None
    nws = lib.mega_attention_workspace_bytes(_dtype_code(qd), B, L, Nh, H1, H2)
    if not nws and L >= 64 and qd.numel():
        # outside the matrix-core kernels (fp32, head sizes that are not multiples of 8): the two products as batched
        # library GEMMs around this library's softmax, which is what the reference does for every shape
        # (attention_kernel.cu:40-131); the library's own fallback is a kernel of one thread per score.  The scores
        # are rounded to the activation type before the softmax, as the reference's are.
        s = torch.einsum('bqnh,bknh->bnqk', qd, kd)
        if float(scale) != 1.0:
            s.mul_(float(scale))
        wts = attention_softmax_fwd(s, dropout, use_causal_mask, seed)
        del s
        y = None if weights_only else torch.einsum('bnqk,bknh->bqnh', wts, vd).contiguous()
        return y, (wts if need_weights else None)
    ws = _scratch_buffer(dev, nws) if nws else None
    with _on_device(dev):
        rc = lib.mega_attention_fwd(_ptr(qd), _ptr(kd), _ptr(vd), _ptr(y), _ptr(w), _dtype_code(qd), B, L, Nh, H1, H2,
                                    float(scale), 1 if use_causal_mask else 0, float(dropout), seed, _ptr(ws),
                                    ws.numel() if nws else 0, _stream(dev))
    _lib.check(rc, "attention_fwd")
    return y, w


def attention_softmax_bwd(y_grad: torch.Tensor, y: torch.Tensor, use_causal_mask: bool, scale: float = 1.0,
                          inplace: bool = False) -> torch.Tensor:
    """x_grad = scale * y * (y_grad - sum(y * y_grad, -1)).  Reference: attention_softmax_bwd,
    fairseq/csrc/ops/attention_softmax.cc:20-26 (scale = 1); `inplace` overwrites y_grad, as the
    reference's attention backward does with its weight gradient."""
    dev = _need_gpu(y_grad, y)
    lib = _lib.load()
    if y_grad.shape != y.shape or y.dim() < 2:
        raise RuntimeError("attention_softmax_bwd: y_grad and y must have the same shape (>= 2 dimensions)")
    yd = y.detach().contiguous()
    gd = y_grad.detach().to(yd.dtype).contiguous()
    outer, inner = yd.shape[-2], yd.shape[-1]
    batch = yd.numel() // max(outer * inner, 1)
    dx = gd if inplace else torch.empty_like(yd)
    with _on_device(dev):
        rc = lib.mega_attention_softmax_bwd(_ptr(gd), _ptr(yd), _ptr(dx), _dtype_code(yd), batch, outer, inner,
                                            1 if use_causal_mask else 0, float(scale), _stream(dev))
    _lib.check(rc, "attention_softmax_bwd")
    return dx


def attention_keeps_no_weights(q, k, v, dropout: float) -> bool:
    """True when a training forward of these operands can leave the L x L weights unsaved: no DropKey, and a shape
    whose weights the matrix-core path can form again in the backward."""
    if dropout > 0.0 or q.dim() != 4 or q.dtype == torch.float32 or not q.is_cuda:
        return False
    B, L, Nh, H1 = q.shape
    H2 = v.shape[3]
    lib = _lib.load()
    dt = _dtype_code(q)
    return bool(lib.mega_attention_workspace_bytes(dt, B, L, Nh, H1, H2)) and \
        bool(lib.mega_attention_bwd_workspace_bytes(dt, B, L, Nh, H1, H2))


def attention_bwd(y_grad, q, k, v, w, scale: float, use_causal_mask: bool, y=None):
    """-> (q_grad, k_grad, v_grad).  Reference: attention_bwd, fairseq/csrc/ops/attention_kernel.cu:133-255:
    four batched products around the softmax backward; w [B, Nh, L, L] are the forward's weights.
    16-bit activations with head sizes that are multiples of 8 run through the library's own matrix-core
    products (mega_attention_bwd: head-strided operands read in place, the causal half of every product
    skipped); fp32 and odd head sizes through four batched library GEMMs around mega_attention_softmax_bwd.
    `y` (not in the reference's signature): the forward's output; with it the softmax backward's row sums are
    y_grad . y and the L x L weight gradient never reaches memory.  It must be the output the forward produced
    from this very `w` (y = w v); a `y` from anywhere else gives a wrong score gradient without any check --
    pass None when in doubt."""
    dev = _need_gpu(y_grad, q, k, v, w)
    if q.dim() != 4 or w is None or w.dim() != 4:
        raise RuntimeError("attention_bwd: q, k, v must be [B,L,N,H] and w [B,N,L,L]")
    qd, kd, vd, wd = (t.detach().contiguous() for t in (q, k, v, w))
    g = y_grad.detach().to(qd.dtype).contiguous()
    B, L, Nh, H1 = qd.shape
    H2 = vd.shape[3]
    if kd.shape != qd.shape or vd.shape[:3] != qd.shape[:3] or g.shape != vd.shape or wd.shape != (B, Nh, L, L):
        raise RuntimeError("attention_bwd: q, k [B,L,N,H1], v and y_grad [B,L,N,H2], w [B,N,L,L] expected")
    if not (qd.dtype == kd.dtype == vd.dtype == wd.dtype):
        raise RuntimeError("attention_bwd: q, k, v, w must share one dtype")
    lib = _lib.load()
    nws = lib.mega_attention_bwd_workspace_bytes(_dtype_code(qd), B, L, Nh, H1, H2) if qd.numel() else 0
    if nws:
        yd = None
        if y is not None and y.shape == vd.shape and y.dtype == vd.dtype:
            yd = y.detach().contiguous()
        q_grad, k_grad, v_grad = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
        ws = _scratch_buffer(dev, nws)
        with _on_device(dev):
            rc = lib.mega_attention_bwd(_ptr(g), _ptr(qd), _ptr(kd), _ptr(vd), _ptr(wd), _ptr(yd), _ptr(q_grad), _ptr(k_grad),
                                        _ptr(v_grad), _dtype_code(qd), B, L, Nh, H1, H2, float(scale),
                                        1 if use_causal_mask else 0, _ptr(ws), ws.numel(), _stream(dev))
        _lib.check(rc, "attention_bwd")
        return q_grad, k_grad, v_grad
    v_grad = torch.einsum('bnqk,bqnh->bknh', wd, g)
    w_grad = torch.einsum('bqnh,bknh->bnqk', g, vd).contiguous()
    s_grad = attention_softmax_bwd(w_grad, wd, use_causal_mask, scale=float(scale), inplace=True)
    k_grad = torch.einsum('bnqk,bqnh->bknh', s_grad, qd)
    q_grad = torch.einsum('bnqk,bknh->bqnh', s_grad, kd)
    return q_grad, k_grad, v_grad


# --------------------------------------------------------------------------------------
# fused inference entry points used by the modules
# --------------------------------------------------------------------------------------


def transpose_2d(x: torch.Tensor, reverse_rows: bool = False, reverse_cols: bool = False) -> torch.Tensor:
    """x: [B, R, C] contiguous (2- or 4-byte elements) -> contiguous [B, C, R] (mega_transpose_2d); reverse_rows /
    reverse_cols read x with its rows / columns in reverse order (x.flip(1) / x.flip(2) first)."""
    dev = _need_gpu(x)
    lib = _lib.load()
    if x.dim() != 3 or not x.is_contiguous() or x.element_size() not in (2, 4):
        raise RuntimeError("transpose_2d: a contiguous [B, R, C] tensor of 2- or 4-byte elements expected")
    B, R, Cc = x.shape
    out = torch.empty(B, Cc, R, dtype=x.dtype, device=dev)
    with _on_device(dev):
        rc = lib.mega_transpose_2d(_ptr(x), _ptr(out), x.element_size(), B, R, Cc, 1 if reverse_rows else 0,
                                   1 if reverse_cols else 0, _stream(dev))
    _lib.check(rc, "transpose_2d")
    return out


class PreparedEMA:
    """Coefficients of one moving-average layer converted once to the layout the library
    takes (fp32, complex as (re, im) pairs); calling it runs the fused layer forward.
    Modules in eval mode keep one of these next to their cached coefficients."""

    def __init__(self, p: torch.Tensor, q: torch.Tensor, gamma: torch.Tensor, omega: torch.Tensor,
                 bidirectional: bool = False, truncation: Optional[int] = None, shift: bool = True):
        self.dev = _need_gpu(p, q, gamma, omega)
        self.K, self.N = p.shape[0], p.shape[1]
        self.D = self.K // 2 if bidirectional else self.K
        if omega.numel() != self.D:
            raise RuntimeError(f"coefficient rows {self.K} do not match kernel_dim for embed_dim {omega.numel()}")
        self.is_complex = bool(q.is_complex() or gamma.is_complex())
        self.p = _f32c(p).reshape(self.K, self.N)
        self.q = _cplx_as_f32(q.reshape(self.K, self.N))
        self.gamma = _cplx_as_f32(gamma.reshape(self.K, self.N))
        self.omega = _f32c(omega).reshape(self.D)
        self.bidirectional = bool(bidirectional)
        self.trunc = 0 if truncation is None or truncation < 1 else int(truncation)
        self.shift = bool(shift)
        # kernel generation once per set of coefficients (operand images of the matrix-core path)
        self.image = None
        lib = _lib.load()
        nimg = lib.mega_ema_image_bytes(self.D, self.N, 1 if self.bidirectional else 0)
        if nimg > 0:
            self.image = torch.empty(nimg, dtype=torch.uint8, device=self.dev)
            with _on_device(self.dev):
                rc = lib.mega_ema_prepare(_ptr(self.p), _ptr(self.q), _ptr(self.gamma), 1 if self.is_complex else 0,
                                          _ptr(self.omega), self.D, self.N, 1 if self.bidirectional else 0,
                                          1 if self.shift else 0, _ptr(self.image), nimg, _stream(self.dev))
            _lib.check(rc, "ema_prepare")

    def __call__(self, x: torch.Tensor, padding_mask: Optional[torch.Tensor] = None,
                 h: Optional[torch.Tensor] = None, want_state: bool = False,
                 out: Optional[torch.Tensor] = None, out_layout: str = "rows"
                 ) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
        """x: [B, D, L] with any strides.  The result is a contiguous [B, D, L] tensor (rows in time, what
        the reference's convolution returns, fused_ops/fftconv.py:45-61) unless `out` is given or
        out_layout == "input" asks for x's own strides."""
        dev = self.dev
        _need_gpu(x, padding_mask, h)
        lib = _lib.load()
        if x.dim() != 3:
            raise RuntimeError("x must be [B, D, L]")
        B, D, L = x.shape
        if D != self.D:
            raise RuntimeError(f"coefficient rows {self.K} do not match kernel_dim {2 * D if self.bidirectional else D}")
        xd = x.detach()
        dt = _dtype_code(xd)
        if 0 in xd.stride() and xd.numel() > 0:
            xd = xd.contiguous()
        if (out is None and xd.dtype in (torch.float32, torch.float16) and B > 0 and 64 <= L <= 16384 and self.N <= 16
                and not self.trunc and xd.stride() == (L * D, 1, D)
                and not ((want_state or h is not None) and L % 1024)):
            # fp32 / fp16 activations that lie time-major in memory: the matrix-core kernels for these types take rows
            # in time ([B, D, L]); a tiled transposition each way costs less than the vector-ALU path for this
            # layout (4 x 1024 x 4096 in fp32: 343 us there, 45 us on rows)
            y, hc = self(transpose_2d(xd.transpose(1, 2)), padding_mask, h, want_state)
            if out_layout == "input":
                y = transpose_2d(y).transpose(1, 2)
            return y, hc
        if out is not None:
            y = out
            if y.shape != xd.shape or y.dtype != xd.dtype:
                raise RuntimeError("out must match x in shape and dtype")
        elif out_layout == "input" and _dense(xd):
            y = torch.empty_strided(xd.shape, xd.stride(), dtype=xd.dtype, device=dev)
        elif out_layout in ("rows", "input"):
            y = torch.empty(xd.shape, dtype=xd.dtype, device=dev)
        else:
            raise RuntimeError(f"out_layout must be 'rows' or 'input', got {out_layout!r}")
        m8 = _mask_u8(padding_mask, B, L)
        N = self.N
        hin = None if h is None else _cplx_as_f32(h.reshape(B, D, N))
        hout = torch.empty(B, D, N, 2, dtype=torch.float32, device=dev) if (want_state or h is not None) else None
        key = ("ema", B, D, N, L, self.bidirectional, self.trunc)
        nws = _ws_bytes_cache.get(key)
        if nws is None:
            nws = _ws_bytes_cache[key] = lib.mega_ema_fwd_workspace_bytes(B, D, N, L, 1 if self.bidirectional else 0,
                                                                         self.trunc)
        stream = _stream(dev)
        ws = _scratch_buffer(dev, nws, stream)
        with _on_device(dev):
            rc = lib.mega_ema_fwd(_ptr(xd), _ptr(y), dt, xd.stride(0), xd.stride(1), xd.stride(2), y.stride(0),
                                  y.stride(1), y.stride(2), _ptr(self.p), _ptr(self.q), _ptr(self.gamma),
                                  1 if self.is_complex else 0, _ptr(self.omega), _ptr(m8), _ptr(hin), _ptr(hout),
                                  B, D, N, L, 1 if self.bidirectional else 0, self.trunc, 1 if self.shift else 0,
                                  _ptr(self.image), _ptr(ws), ws.numel(), stream)
        _lib.check(rc, "ema_fwd")
        hc = None
        if hout is not None:
            hc = torch.view_as_complex(hout) if self.is_complex else hout[..., 0]
        return y, hc


    def norm_forward(self, x: torch.Tensor, prev_count, prev_mean, prev_var, norm_gamma, norm_beta,
                     num_groups: int, eps: float, padding_mask: Optional[torch.Tensor] = None,
                     h: Optional[torch.Tensor] = None, want_state: bool = False, out_layout: str = "rows",
                     want_stats: bool = False):
        """TimestepNorm followed by this layer in one call (moving_average_gated_attention.py:304-315:
        x = norm(x); mx = move(x^T)).  x: [B, L, D].  -> (xn [B, L, D], y, count, mean, var, h_out); y is a
        contiguous [B, D, L] tensor (out_layout "rows", what the reference's convolution returns) or a
        [B, D, L] view of [B, L, D] memory (out_layout "input").  Covered shapes run as one kernel, the
        rest as the two operators one after the other (mega_norm_ema_fwd).  want_stats (a training
        forward): two more results, cummean and cumrstd [B, L, G], what the norm's backward pass reads
        (timestep_norm.py:35-43)."""
        dev = self.dev
        _need_gpu(x, prev_count, prev_mean, prev_var, norm_gamma, norm_beta, padding_mask, h)
        if self.bidirectional or self.trunc:
            raise RuntimeError("norm_forward: one-sided layers without kernel truncation only")
        lib = _lib.load()
        if x.dim() != 3 or x.shape[2] != self.D:
            raise RuntimeError(f"x must be [B, L, {self.D}]")
        B, L, D = x.shape
        G = int(num_groups)
        if G <= 0 or D % G != 0:
            raise RuntimeError(f"num_features={D} is not divisible by num_groups={G}")
        xd = x if (x.is_contiguous() and not x.requires_grad) else x.detach().contiguous()
        dt = _dtype_code(xd)
        if out_layout not in ("rows", "input"):
            raise RuntimeError(f"out_layout must be 'rows' or 'input', got {out_layout!r}")
        if xd.dtype is not torch.bfloat16 and 64 <= L <= 16384 and self.N <= 16 and B > 0 \
                and not ((want_state or h is not None) and L % 1024):
            # fp32 / fp16: the two operators, the second through PreparedEMA.__call__, which takes the normalised
            # activations (time-major in memory) onto the rows kernels; inside the library's own two-operator
            # route the moving average would read them in place on its vector-ALU path
            if want_stats:
                xn, count, mean, var, _, cm, cr = group_timestep_norm_fwd(xd, prev_count, prev_mean, prev_var, norm_gamma,
                                                                          norm_beta, padding_mask, G, eps)
            else:
                xn, count, mean, var = group_timestep_norm_fwd(xd, prev_count, prev_mean, prev_var, norm_gamma,
                                                               norm_beta, padding_mask, G, eps, need_stats=False)[:4]
            y, hc = self(xn.transpose(1, 2), padding_mask, h, want_state, out_layout=out_layout)
            return (xn, y, count, mean, var, hc, cm, cr) if want_stats else (xn, y, count, mean, var, hc)
        xn = torch.empty_like(xd)
        if out_layout == "rows":
            y = torch.empty(B, D, L, dtype=xd.dtype, device=dev)
        elif out_layout == "input":
            y = torch.empty(B, L, D, dtype=xd.dtype, device=dev).transpose(1, 2)
        else:
            raise RuntimeError(f"out_layout must be 'rows' or 'input', got {out_layout!r}")
        pc, pm, pv = _norm_state(prev_count, prev_mean, prev_var, B, G, dev)
        count = torch.empty(B, dtype=torch.int64, device=dev)
        mean = torch.empty(B, G, dtype=torch.float32, device=dev)
        var = torch.empty(B, G, dtype=torch.float32, device=dev)
        N = self.N
        hin = None if h is None else _cplx_as_f32(h.reshape(B, D, N))
        hout = torch.empty(B, D, N, 2, dtype=torch.float32, device=dev) if (want_state or h is not None) else None
        key = ("norm_ema", B, L, D, G, N)
        sizes = _ws_bytes_cache.get(key)
        if sizes is None:
            sizes = _ws_bytes_cache[key] = (lib.mega_norm_ema_fwd_workspace_bytes(B, L, D, G, N),
                                            lib.mega_norm_ema_fwd_scratch_bytes(B, L, D, G, N))
        stream = _stream(dev)
        ws = _tsn_workspace(dev, sizes[0], stream)
        sc = _scratch_buffer(dev, sizes[1], stream)
        m8 = _mask_u8(padding_mask, B, L)
        gf, bf = _f32c(norm_gamma), _f32c(norm_beta)
        cm = cr = None
        if want_stats:
            cm = torch.empty(B, L, G, dtype=torch.float32, device=dev)
            cr = torch.empty(B, L, G, dtype=torch.float32, device=dev)
        with _on_device(dev):
            rc = lib.mega_norm_ema_fwd_train(_ptr(xd), _ptr(xn), _ptr(y), dt, y.stride(0), y.stride(1), y.stride(2),
                                             _ptr(pc), _ptr(pm), _ptr(pv), _ptr(gf), _ptr(bf), _ptr(m8), float(eps),
                                             _ptr(count), _ptr(mean), _ptr(var), _ptr(cm), _ptr(cr), _ptr(self.p),
                                             _ptr(self.q), _ptr(self.gamma), 1 if self.is_complex else 0,
                                             _ptr(self.omega), _ptr(hin), _ptr(hout), B, L, D, G, N, _ptr(self.image),
                                             _ptr(ws), ws.numel(), _ptr(sc), sc.numel(), stream)
        _lib.check(rc, "norm_ema_fwd")
        hc = None
        if hout is not None:
            hc = torch.view_as_complex(hout) if self.is_complex else hout[..., 0]
        if want_stats:
            return xn, y, count, mean, var, hc, cm, cr
        return xn, y, count, mean, var, hc

    def adjoint(self, y_grad: torch.Tensor, padding_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Gradient of the layer output with respect to its input x:
        dx[t] = (1 - mask[t]) sum_s k(s - t) dy[s] + omega dy[t], the same layer (one- or two-sided)
        run backwards in time.  A channel-contiguous y_grad ([B, L, D] memory) is read in place with
        negated token strides; rows in time are flipped through a copy.  The result has y_grad's
        layout."""
        if self.trunc:
            raise NotImplementedError("adjoint: layers without kernel truncation only")
        dev = self.dev
        _need_gpu(y_grad, padding_mask)
        lib = _lib.load()
        B, D, L = y_grad.shape
        if D != self.D:
            raise RuntimeError("y_grad must be [B, D, L] of this layer")
        g = y_grad.detach()
        if L == 0 or B == 0:
            return torch.empty_like(g)
        if (g.dtype in (torch.float32, torch.float16) and 64 <= L <= 16384 and self.N <= 16
                and g.stride() == (L * D, 1, D)):
            # fp32 / fp16 gradients that lie time-major in memory: onto rows in time and back through the tiled
            # transposition, which also reverses the time axis each way (as __call__ does for the forward)
            out, _ = self(transpose_2d(g.transpose(1, 2), reverse_rows=True))
            dx = transpose_2d(out, reverse_cols=True).transpose(1, 2)
        elif g.stride(1) != 1 or not _dense(g):
            # time is the fast axis (or the layout is irregular): flip, run forwards, flip back
            out, _ = self(g.flip(-1))
            dx = out.flip(-1)
        else:
            dx = torch.empty_strided(g.shape, g.stride(), dtype=g.dtype, device=dev)
            es = g.element_size()
            bi = 1 if self.bidirectional else 0
            key = ("ema", B, D, self.N, L, self.bidirectional, 0)
            nws = _ws_bytes_cache.get(key)
            if nws is None:
                nws = _ws_bytes_cache[key] = lib.mega_ema_fwd_workspace_bytes(B, D, self.N, L, bi, 0)
            stream = _stream(dev)
            ws = _scratch_buffer(dev, nws, stream)
            sl = g.stride(2)
            with _on_device(dev):
                rc = lib.mega_ema_fwd(g.data_ptr() + (L - 1) * sl * es, dx.data_ptr() + (L - 1) * sl * es,
                                      _dtype_code(g), g.stride(0), g.stride(1), -sl, dx.stride(0), dx.stride(1), -sl,
                                      _ptr(self.p), _ptr(self.q), _ptr(self.gamma), 1 if self.is_complex else 0,
                                      _ptr(self.omega), None, None, None, B, D, self.N, L, bi, 0,
                                      1 if self.shift else 0, _ptr(self.image), _ptr(ws), ws.numel(), stream)
            _lib.check(rc, "ema_fwd (adjoint)")
        if padding_mask is not None:
            dx = torch.where(padding_mask.to(torch.bool).unsqueeze(1), self.omega.to(g.dtype).view(1, D, 1) * g, dx)
        return dx


def ema_forward(x: torch.Tensor, p: torch.Tensor, q: torch.Tensor, gamma: torch.Tensor, omega: torch.Tensor,
                padding_mask: Optional[torch.Tensor] = None, h: Optional[torch.Tensor] = None,
                want_state: bool = False, bidirectional: bool = False, truncation: Optional[int] = None,
                shift: bool = True, out_layout: str = "rows") -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Whole moving-average layer in one call (BaseMovingLayer.forward,
    fairseq/modules/base_moving_average.py:120-172).

    x: [B, D, L] (any strides; a transposed view of a [B, L, D] tensor is read in place);
    p: [K, N]; q, gamma: [K, N] real or complex; omega: [D]; h: [B, D, N] carried state.
    Returns (y, h') with y a contiguous [B, D, L] tensor (out_layout="input": x's strides) and h'
    complex64 (or None).
    """
    _need_gpu(x)
    return PreparedEMA(p, q, gamma, omega, bidirectional, truncation, shift)(x, padding_mask, h, want_state,
                                                                            out_layout=out_layout)


def _dense(t: torch.Tensor) -> bool:
    """True when the tensor's strides describe a permutation of a contiguous block."""
    if t.numel() == 0:
        return False
    pairs = sorted(((s, n) for s, n in zip(t.stride(), t.shape) if n > 1), reverse=True)
    expect = 1
    for s, n in reversed(pairs):
        if s != expect:
            return False
        expect *= n
    return True


def ema_step(x_t: torch.Tensor, p, q, gamma, omega, h: Optional[torch.Tensor]):
    """One decode step: x_t [B, D] -> (y_t [B, D], h' [B, D, N]).
    BaseMovingLayer.one_step, fairseq/modules/base_moving_average.py:105-118, plus omega x."""
    dev = _need_gpu(x_t, p, q, gamma, omega, h)
    lib = _lib.load()
    B, D = x_t.shape
    N = p.shape[1]
    is_complex = q.is_complex() or gamma.is_complex()
    xd = x_t.detach().contiguous()
    y = torch.empty_like(xd)
    pf = _f32c(p).reshape(D, N)
    qf = _cplx_as_f32(q.reshape(D, N))
    gf = _cplx_as_f32(gamma.reshape(D, N))
    of = _f32c(omega).reshape(D)
    hin = None if h is None else _cplx_as_f32(h.reshape(B, D, N))
    hout = torch.empty(B, D, N, 2, dtype=torch.float32, device=dev)
    with _on_device(dev):
        rc = lib.mega_ema_step(_ptr(xd), _ptr(y), _dtype_code(xd), _ptr(pf), _ptr(qf), _ptr(gf),
                               1 if is_complex else 0, _ptr(of), _ptr(hin), _ptr(hout), B, D, N, _stream(dev))
    _lib.check(rc, "ema_step")
    return y, (torch.view_as_complex(hout) if is_complex else hout[..., 0])


class DecodeStep:
    """Streaming decode of the norm -> moving-average pair: one launch per token.  Holds the
    converted coefficients and the carried state (norm count / mean / var, EMA h) on the device
    and updates them in place."""

    def __init__(self, norm_weight, norm_bias, num_groups: int, eps: float, p, q, gamma, omega, batch_size: int,
                 prior_count: int = 0):
        self.dev = _need_gpu(norm_weight, norm_bias, p, q, gamma, omega)
        self.D, self.N = p.shape[0], p.shape[1]
        self.G, self.eps, self.B = int(num_groups), float(eps), int(batch_size)
        self.is_complex = bool(q.is_complex() or gamma.is_complex())
        self.nw = (_f32c(norm_weight) + 1.0).contiguous()
        self.nb = _f32c(norm_bias)
        self.p = _f32c(p).reshape(self.D, self.N)
        self.q = _cplx_as_f32(q.reshape(self.D, self.N))
        self.gamma = _cplx_as_f32(gamma.reshape(self.D, self.N))
        self.omega = _f32c(omega).reshape(self.D)
        # two count buffers used in turn: every (stream, group) workgroup of a launch reads the old
        # count while one workgroup per stream writes the new one, so the two must not share memory
        self.count = torch.full((self.B,), prior_count, dtype=torch.int64, device=self.dev)
        self._count_next = torch.empty_like(self.count)
        self.mean = torch.zeros(self.B, self.G, dtype=torch.float32, device=self.dev)
        self.var = torch.ones(self.B, self.G, dtype=torch.float32, device=self.dev)
        self.h = torch.zeros(self.B, self.D, self.N, 2, dtype=torch.float32, device=self.dev)

    def __call__(self, x_t: torch.Tensor):
        """x_t: [B, D] -> (xn_t, y_t), both [B, D]."""
        lib = _lib.load()
        xd = x_t.detach().contiguous()
        xn = torch.empty_like(xd)
        y = torch.empty_like(xd)
        with _on_device(self.dev):
            rc = lib.mega_norm_ema_step(_ptr(xd), _ptr(xn), _ptr(y), _dtype_code(xd), _ptr(self.count), _ptr(self.mean),
                                        _ptr(self.var), _ptr(self._count_next), _ptr(self.mean), _ptr(self.var), _ptr(self.nw),
                                        _ptr(self.nb), self.eps, _ptr(self.p), _ptr(self.q), _ptr(self.gamma),
                                        1 if self.is_complex else 0, _ptr(self.omega), _ptr(self.h), _ptr(self.h),
                                        self.B, self.D, self.G, self.N, _stream(self.dev))
        _lib.check(rc, "norm_ema_step")
        self.count, self._count_next = self._count_next, self.count
        return xn, y

    def steps(self, x: torch.Tensor):
        """x: [B, K, D], K consecutive tokens of every stream -> (xn, y), both [B, K, D]: the same as K calls,
        in one launch (the state is read and written once).  Coefficient shapes the multi-token kernel does not
        cover take K single steps."""
        lib = _lib.load()
        if x.dim() != 3 or x.shape[0] != self.B or x.shape[2] != self.D:
            raise RuntimeError(f"x must be [{self.B}, K, {self.D}]")
        K = x.shape[1]
        np_ = self.N // 4
        if not (self.is_complex and self.N % 4 == 0 and self.N <= 32 and np_ & (np_ - 1) == 0):
            outs = [self(x[:, k]) for k in range(K)]
            if not outs:
                return torch.empty_like(x), torch.empty_like(x)
            return torch.stack([o[0] for o in outs], 1), torch.stack([o[1] for o in outs], 1)
        xd = x.detach().contiguous()
        xn = torch.empty_like(xd)
        y = torch.empty_like(xd)
        if K == 0:
            return xn, y
        with _on_device(self.dev):
            rc = lib.mega_norm_ema_steps(_ptr(xd), _ptr(xn), _ptr(y), _dtype_code(xd), K, _ptr(self.count),
                                         _ptr(self.mean), _ptr(self.var), _ptr(self._count_next), _ptr(self.mean),
                                         _ptr(self.var), _ptr(self.nw), _ptr(self.nb), self.eps, _ptr(self.p), _ptr(self.q),
                                         _ptr(self.gamma), 1, _ptr(self.omega), _ptr(self.h), _ptr(self.h), self.B, self.D,
                                         self.G, self.N, _stream(self.dev))
        _lib.check(rc, "norm_ema_steps")
        self.count, self._count_next = self._count_next, self.count
        return xn, y

    @property
    def state(self) -> torch.Tensor:
        return torch.view_as_complex(self.h) if self.is_complex else self.h[..., 0]


class _CausalConvFunc(torch.autograd.Function):
    """fairseq/modules/fused_ops/fftconv.py:11-41 (FFTConvFunc) with the kernel in the time domain."""

    @staticmethod
    def forward(ctx, x, k):
        ctx.save_for_backward(x, k)
        return _long_conv(x, k, False, True)

    @staticmethod
    def backward(ctx, y_grad):
        x, k = ctx.saved_tensors
        x_grad, k_grad = fftconv_bwd(y_grad, x, k)
        return x_grad, k_grad.to(k.dtype)


def fftconv(x: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """Causal long convolution with an explicit kernel k[D, Lk] (fftconv,
    fairseq/modules/fused_ops/fftconv.py:11-27); evaluated in the time domain.  Differentiable."""
    if torch.is_grad_enabled() and (x.requires_grad or k.requires_grad):
        return _CausalConvFunc.apply(x, k)
    return _long_conv(x, k, False, True)


class _EMAParametersFunc(torch.autograd.Function):
    """fairseq/modules/fused_ops/ema_parameters.py:11-35 (EMAParametersFunc): kernel and carried-state bias
    from the coefficients, differentiable in p, q, gamma and h."""

    @staticmethod
    def forward(ctx, p, q, gamma, h, length):
        log_q = q.detach().log()
        w, b, _ = ema_parameters_fwd(p, log_q, gamma, h, length)
        ctx.save_for_backward(p, log_q, gamma, h)
        return w, b

    @staticmethod
    def backward(ctx, w_grad, b_grad):
        p, log_q, gamma, h = ctx.saved_tensors
        if h is None:
            b_grad = None
        elif b_grad is None:
            b_grad = torch.zeros(h.shape[0], p.shape[0], w_grad.shape[-1], dtype=torch.float32, device=w_grad.device)
        p_grad, q_grad, gamma_grad, h_grad = ema_parameters_bwd(w_grad, b_grad, p, log_q, gamma, h)
        return (_like_input(p_grad, p), _like_input(q_grad, log_q, p.shape), _like_input(gamma_grad, gamma),
                None if h is None else _like_input(h_grad, h), None)


class _EMAHiddenFunc(torch.autograd.Function):
    """fairseq/modules/fused_ops/ema_hidden.py:8-30 (EMAHiddenFunc): the state after the last token,
    differentiable in x, p, q and h."""

    @staticmethod
    def forward(ctx, x, p, q, h):
        log_q = q.detach().log()
        y, _ = ema_hidden_fwd(x, p, log_q, h)
        ctx.save_for_backward(x, p, log_q, h)
        return y if log_q.is_complex() else y.real.contiguous()

    @staticmethod
    def backward(ctx, y_grad):
        x, p, log_q, h = ctx.saved_tensors
        x_grad, p_grad, q_grad, h_grad = ema_hidden_bwd(y_grad, x, p, log_q, h)
        return (x_grad.to(x.dtype), _like_input(p_grad, p), _like_input(q_grad, log_q, p.shape),
                None if h is None else _like_input(h_grad, h))


def _like_input(g: torch.Tensor, t: torch.Tensor, shape=None) -> torch.Tensor:
    """A gradient in the type (real or complex) and shape of the input it belongs to."""
    if not t.is_complex() and g.is_complex():
        g = g.real
    g = g.to(torch.complex64 if t.is_complex() else t.dtype)
    return g.reshape(t.shape if shape is None else shape).contiguous()


def ema_parameters(p: torch.Tensor, q: torch.Tensor, gamma: torch.Tensor, h: Optional[torch.Tensor], length: int):
    """-> (k [K, length] fp32, b [B, K, length] fp32 or None): k[l] = Re sum_n p gamma q^l and the carried
    state's contribution b[l] = Re sum_n gamma q^(l+1) h, differentiable (ema_parameters,
    fairseq/modules/fused_ops/ema_parameters.py:11-35).  p, q: [K, N]; gamma: [K, N]; h: [B, K, N] or None."""
    return _EMAParametersFunc.apply(p, q, gamma, h, length)


def ema_hidden(x: torch.Tensor, p: torch.Tensor, q: torch.Tensor, h: Optional[torch.Tensor]) -> torch.Tensor:
    """-> h' [B, D, N] = q^L h + sum_j p q^(L-1-j) x[j], differentiable (ema_hidden,
    fairseq/modules/fused_ops/ema_hidden.py:8-30); real for real coefficients."""
    return _EMAHiddenFunc.apply(x, p, q, h)


def _rfft_len(L: int) -> int:
    """Length of the real transform the reference's convolution uses: 2 * pow2ceil(L)
    (fused_ops/fftconv.py:17-18, 47)."""
    N = L if (L & (L - 1)) == 0 else (1 << L.bit_length())
    return 2 * N


def rfft(x: torch.Tensor, flip: bool = False) -> torch.Tensor:
    """Reference: rfft, fairseq/csrc/ops/fftconv.cc:6-8 (ops/fftconv_kernel.cu:23-44, 169-212): the
    unnormalised real transform of length 2 * pow2ceil(L) over the last axis, of the time-reversed
    signal when `flip` -> [..., pow2ceil(L) + 1] complex64.  The kernels of this library work in the
    time domain; the operator exists for callers written against the reference's extension and runs
    the library transform."""
    _need_gpu(x)
    xf = x.detach().float()
    return torch.fft.rfft(xf.flip(-1) if flip else xf, n=_rfft_len(x.size(-1)))


def _from_spectrum(t_f: torch.Tensor, L: int, what: str) -> torch.Tensor:
    n = _rfft_len(L)
    if not t_f.is_complex() or t_f.size(-1) != n // 2 + 1:
        raise RuntimeError(f"{what} must be a complex spectrum with {n // 2 + 1} bins for L = {L}")
    return torch.fft.irfft(t_f, n=n)[..., :L]


def fftconv_fwd(x: torch.Tensor, k_f: torch.Tensor):
    """-> (y [B,H,L] of x's dtype, x_f [B,H,pow2ceil(L)+1] complex64).  Reference: fftconv_fwd,
    fairseq/csrc/ops/fftconv.cc:10-13 (ops/fftconv_kernel.cu:46-78, 214-269): the causal convolution
    with the kernel given as its spectrum k_f = rfft(k).  The first L taps are taken back out of the
    spectrum and the convolution runs in the time domain; x_f is produced because the reference's
    autograd function saves it.  No L <= 8192 limit."""
    _need_gpu(x, k_f)
    if x.dim() != 3:
        raise RuntimeError("fftconv_fwd: x must be [B, H, L]")
    L = x.size(-1)
    k = _from_spectrum(k_f, L, "k_f").float().contiguous()
    return _long_conv(x, k, False, True), rfft(x, False)


def fftconv_bwd(y_grad: torch.Tensor, x: torch.Tensor, k: torch.Tensor, k_dtype: Optional[torch.dtype] = None):
    """-> (x_grad [B,D,L], k_grad [D,Lk]) of y = fftconv(x, k): the two correlations of
    fused_ops/fftconv.py:66-88 (x_grad[t] = sum_l k[l] dy[t+l], k_grad[l] = sum_{b,t} dy[t] x[t-l]) as
    causal convolutions of the time-reversed gradient, through the same explicit-kernel op (a
    correctness path, O(L Lk) per row; the modules use ema_backward, which forms neither k nor k_grad).
    Two call forms: (y_grad, x, k) in the time domain (k_grad in fp32), and the reference's
    fftconv_bwd(y_grad, x_f, k_f, k_dtype) (fairseq/csrc/ops/fftconv.cc:15-20) with the spectra its
    forward saved, k_grad [D, L] in k_dtype."""
    _need_gpu(y_grad, x, k)
    if x.is_complex() or k.is_complex():
        L = y_grad.size(-1)
        xt = _from_spectrum(x, L, "x_f").to(y_grad.dtype)
        kt = _from_spectrum(k, L, "k_f").float().contiguous()
        x_grad, k_grad = fftconv_bwd(y_grad, xt, kt)
        return x_grad, k_grad.to(k_dtype if k_dtype is not None else torch.float32)
    B, D, L = x.shape
    Lk = k.shape[1]
    r = y_grad.detach().to(x.dtype).flip(-1).contiguous()              # r[t] = dy[L-1-t]
    x_grad = _long_conv(r, k, False, True).flip(-1)
    k_grad = torch.zeros(D, L, dtype=torch.float32, device=x.device)
    xf = x.detach().float()
    for b in range(B):
        # y[t] = sum_j x_b[j] r_b[t-j] = sum_j x_b[j] dy_b[L-1-t+j]  ->  k_grad[l] += y[L-1-l]
        k_grad += _long_conv(r[b:b + 1].float(), xf[b], False, True)[0].flip(-1)
    return x_grad, k_grad[:, :Lk].contiguous()


def bidirectional_fftconv(x: torch.Tensor, k: torch.Tensor, shift: bool = True) -> torch.Tensor:
    """bidirectional_fftconv, fairseq/modules/fused_ops/fftconv.py:85-100; k is [2D, Lk]:
    y[t] = sum_l k1[l] x[t-l] + sum_l k2[l] x[t+l+1] (shift) or x[t+l] (no shift).  Under autograd the two
    halves run as two causal convolutions, the second one over reversed time (the reference's is plain
    torch.fft and differentiable the same way)."""
    if torch.is_grad_enabled() and (x.requires_grad or k.requires_grad):
        D = x.size(1)
        fwd = fftconv(x, k[:D])
        back = fftconv(x.flip(-1), k[D:]).flip(-1)
        if shift:
            back = torch.nn.functional.pad(back[..., 1:], (0, 1))
        return fwd + back
    return _long_conv(x, k, True, shift)


def _long_conv(x, k, bidirectional, shift):
    dev = _need_gpu(x, k)
    lib = _lib.load()
    B, D, L = x.shape
    xd = x.detach().contiguous()
    kf = _f32c(k)
    if kf.shape[0] != (2 * D if bidirectional else D):
        raise RuntimeError("kernel rows do not match the channel count")
    Lk = kf.shape[1]
    y = torch.empty_like(xd)
    with _on_device(dev):
        rc = lib.mega_long_conv_fwd(_ptr(xd), _ptr(y), _dtype_code(xd), _ptr(kf), B, D, L, Lk,
                                    1 if bidirectional else 0, 1 if shift else 0, _stream(dev))
    _lib.check(rc, "long_conv_fwd")
    return y


def swiglu(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """silu(a) * b, elementwise."""
    dev = _need_gpu(a, b)
    lib = _lib.load()
    if a.shape != b.shape or a.dtype != b.dtype:
        raise RuntimeError("swiglu: a and b must have the same shape and dtype")
    ad, bd = a.detach().contiguous(), b.detach().contiguous()
    y = torch.empty_like(ad)
    with _on_device(dev):
        rc = lib.mega_swiglu_fwd(_ptr(ad), _ptr(bd), _ptr(y), _dtype_code(ad), ad.numel(), _stream(dev))
    _lib.check(rc, "swiglu_fwd")
    return y


def silu(x: torch.Tensor, inplace: bool = False) -> torch.Tensor:
    """x / (1 + exp(-x)), elementwise (F.silu; moving_average_gated_attention.py:303-316,
    normalized_feedforward_network.py:82); `inplace` overwrites a contiguous x."""
    dev = _need_gpu(x)
    lib = _lib.load()
    xd = x.detach()
    if not xd.is_contiguous():
        xd, inplace = xd.contiguous(), True
    y = xd if inplace else torch.empty_like(xd)
    with _on_device(dev):
        rc = lib.mega_silu_fwd(_ptr(xd), _ptr(y), _dtype_code(xd), xd.numel(), _stream(dev))
    _lib.check(rc, "silu_fwd")
    return y


def silu_bwd(y_grad: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """Backward of silu: y_grad * silu'(x)."""
    dev = _need_gpu(y_grad, x)
    lib = _lib.load()
    xd = x.detach().contiguous()
    g = y_grad.detach().to(xd.dtype).contiguous()
    dx = torch.empty_like(xd)
    with _on_device(dev):
        rc = lib.mega_silu_bwd(_ptr(g), _ptr(xd), _ptr(dx), _dtype_code(xd), xd.numel(), _stream(dev))
    _lib.check(rc, "silu_bwd")
    return dx


def colsum(x: torch.Tensor, out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Sum of a [..., W] tensor over everything but its last axis (a projection's bias gradient), slabs of rows
    added in a fixed order; rows that are not whole 16-byte pieces go through torch."""
    dev = _need_gpu(x)
    lib = _lib.load()
    W = x.shape[-1]
    out_dtype = x.dtype if out_dtype is None else out_dtype
    xr, rs = _rows(x)
    T = _ntok(x)
    if T == 0 or (W * xr.element_size()) % 16 or (rs * xr.element_size()) % 16 or xr.data_ptr() % 16:
        return x.detach().reshape(-1, W).sum(0, dtype=torch.float32).to(out_dtype)
    out = torch.empty(W, dtype=out_dtype, device=dev)
    stream = _stream(dev)
    ws = _scratch_buffer(dev, lib.mega_colsum_workspace_bytes(T, W), stream)
    with _on_device(dev):
        rc = lib.mega_colsum(_ptr(xr), rs, _dtype_code(xr), T, W, _ptr(out), _DT[out_dtype], _ptr(ws), ws.numel(), stream)
    _lib.check(rc, "colsum")
    return out


# ------------------------------------------------------------------------------------------------
# per-token glue of the gated-attention layer (rows of a wider projection output are passed in
# place: every input carries its own row stride)
# ------------------------------------------------------------------------------------------------
def _rows(t: torch.Tensor):
    """(tensor whose data_ptr is the first row, row stride in elements) of a [..., W] tensor whose
    leading axes walk memory uniformly; anything else is made contiguous first."""
    t = t.detach()
    ok = t.stride(-1) == 1 or t.shape[-1] == 1
    for i in range(t.dim() - 2):
        ok = ok and (t.shape[i] == 1 or t.stride(i) == t.stride(i + 1) * t.shape[i + 1])
    if not ok:
        t = t.contiguous()
    if t.dim() == 1:
        return t, t.shape[-1]
    return t, t.stride(-2) if t.shape[-2] > 1 else max(t.stride(-2), t.shape[-1])


def _grad_slot(out: Optional[torch.Tensor], like: torch.Tensor):
    """(tensor to write a gradient of `like`'s shape into, its row stride): `out` when the caller hands over a
    row-strided slice of a wider buffer (last axis contiguous, rows uniformly spaced, 16-byte aligned rows),
    else a new contiguous tensor."""
    if out is not None:
        ok = out.shape == like.shape and out.dtype == like.dtype and out.device == like.device and out.dim() >= 2
        ok = ok and (out.stride(-1) == 1) and (out.stride(-2) * out.element_size()) % 16 == 0 and out.data_ptr() % 16 == 0
        for i in range(out.dim() - 2):
            ok = ok and (out.shape[i] == 1 or out.stride(i) == out.stride(i + 1) * out.shape[i + 1])
        if ok:
            return out, out.stride(-2)
    t = torch.empty(like.shape, dtype=like.dtype, device=like.device)
    return t, like.shape[-1]


def _ntok(t: torch.Tensor) -> int:
    return t.numel() // t.shape[-1] if t.shape[-1] else 0


def rms_norm_fwd(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x * rsqrt(mean(x^2, -1) + eps) * weight (fairseq/modules/norm_layer/layer_norm.py:51-59)."""
    dev = _need_gpu(x)
    lib = _lib.load()
    xr, xs = _rows(x)
    w = None if weight is None else _f32c(weight)
    if w is not None and w.numel() != x.shape[-1]:
        raise RuntimeError("rms_norm_fwd: weight must hold one value per feature")
    y = torch.empty(x.shape, dtype=x.dtype, device=dev)
    with _on_device(dev):
        rc = lib.mega_rms_norm_fwd(_ptr(xr), xs, _ptr(w), _ptr(y), _dtype_code(xr), _ntok(x), x.shape[-1], float(eps),
                                   _stream(dev))
    _lib.check(rc, "rms_norm_fwd")
    return y


def gate_qk_fwd(z: torch.Tensor, gamma: torch.Tensor, beta: torch.Tensor, freqs: torch.Tensor, num_heads: int,
                chunk: int, pos0: int = 0, eps: float = 1e-5):
    """q, k = rotary(normalize(z) * gamma[i] + beta[i]), i = 0, 1
    (moving_average_gated_attention.py:324-328, relative_positional_bias.py:86-97 with qidx = 0).
    z: [..., S]; gamma, beta: [2, S] (gamma is the multiplier, "+ 1" included); freqs: [S/heads/2];
    the position of a token is pos0 + its index modulo `chunk` along the flattened leading axes."""
    dev = _need_gpu(z)
    lib = _lib.load()
    S = z.shape[-1]
    zr, zs = _rows(z)
    if zs % 2 or zr.data_ptr() % (2 * zr.element_size()):
        zr, zs = z.detach().contiguous(), S        # the kernel moves feature pairs: rows must start on an even element
    g, b, f = _f32c(gamma), _f32c(beta), _f32c(freqs)
    if g.shape != (2, S) or b.shape != (2, S) or num_heads < 1 or S % num_heads or f.numel() * 2 * num_heads != S:
        raise RuntimeError("gate_qk_fwd: gamma, beta must be [2, S] and freqs [S / heads / 2]")
    q = torch.empty(z.shape, dtype=z.dtype, device=dev)
    k = torch.empty(z.shape, dtype=z.dtype, device=dev)
    with _on_device(dev):
        rc = lib.mega_gate_qk_fwd(_ptr(zr), zs, _ptr(g), _ptr(b), _ptr(f), _ptr(q), _ptr(k), _dtype_code(zr), _ntok(z),
                                  S, num_heads, int(chunk), int(pos0), float(eps), _stream(dev))
    _lib.check(rc, "gate_qk_fwd")
    return q, k


def gate_qk_bwd(q_grad: torch.Tensor, k_grad: torch.Tensor, z: torch.Tensor, gamma: torch.Tensor, freqs: torch.Tensor,
                num_heads: int, chunk: int, pos0: int = 0, eps: float = 1e-5,
                z_grad_out: Optional[torch.Tensor] = None):
    """Backward of gate_qk_fwd: -> (z_grad [..., S] in z's dtype, gamma_grad [2, S] fp32, beta_grad [2, S] fp32).
    z_grad_out: a row-strided slice of a wider gradient buffer to write z_grad into (returned as z_grad).
    The autograd graph it replaces is normalize -> affine -> rotary
    (moving_average_gated_attention.py:324-328, relative_positional_bias.py:86-97)."""
    dev = _need_gpu(q_grad, k_grad, z)
    lib = _lib.load()
    S = z.shape[-1]
    zr, zs = _rows(z)
    if (zs * zr.element_size()) % 16 or zr.data_ptr() % 16:
        zr, zs = z.detach().contiguous(), S        # the kernel reads whole 16-byte vectors
    g, f = _f32c(gamma), _f32c(freqs)
    if g.shape != (2, S) or num_heads < 1 or S % num_heads or f.numel() * 2 * num_heads != S:
        raise RuntimeError("gate_qk_bwd: gamma must be [2, S] and freqs [S / heads / 2]")
    if q_grad.shape != z.shape or k_grad.shape != z.shape:
        raise RuntimeError("gate_qk_bwd: q_grad, k_grad must have z's shape")
    dq = q_grad.detach().to(z.dtype).contiguous()
    dk = k_grad.detach().to(z.dtype).contiguous()
    dz, dzs = _grad_slot(z_grad_out, z)
    dgamma = torch.empty(2, S, dtype=torch.float32, device=dev)
    dbeta = torch.empty(2, S, dtype=torch.float32, device=dev)
    T = _ntok(z)
    nws = lib.mega_gate_qk_bwd_workspace_bytes(T, S)
    with _on_device(dev):
        stream = _stream(dev)
        ws = _scratch_buffer(dev, nws, stream)
        rc = lib.mega_gate_qk_bwd_strided(_ptr(dq), _ptr(dk), _ptr(zr), zs, _ptr(g), _ptr(f), _ptr(dz), dzs,
                                          _ptr(dgamma), _ptr(dbeta), _dtype_code(zr), T, S, num_heads, int(chunk),
                                          int(pos0), float(eps), _ptr(ws), ws.numel(), stream)
    _lib.check(rc, "gate_qk_bwd")
    return dz, dgamma, dbeta


def gate_mul_fwd(a: torch.Tensor, r: torch.Tensor) -> torch.Tensor:
    """a * silu(r) (moving_average_gated_attention.py:330, 407)."""
    dev = _need_gpu(a, r)
    lib = _lib.load()
    if a.shape != r.shape or a.dtype != r.dtype:
        raise RuntimeError("gate_mul_fwd: a and r must have the same shape and dtype")
    ar, as_ = _rows(a)
    rr, rs = _rows(r)
    y = torch.empty(a.shape, dtype=a.dtype, device=dev)
    with _on_device(dev):
        rc = lib.mega_gate_mul_fwd(_ptr(ar), as_, _ptr(rr), rs, _ptr(y), _dtype_code(ar), _ntok(a), a.shape[-1],
                                   _stream(dev))
    _lib.check(rc, "gate_mul_fwd")
    return y


def gate_out_fwd(residual: torch.Tensor, u: torch.Tensor, hx: torch.Tensor, hp: torch.Tensor) -> torch.Tensor:
    """residual + sigmoid(u) * (silu(hx + hp) - residual)
    (moving_average_gated_attention.py:322, 409, 412)."""
    dev = _need_gpu(residual, u, hx, hp)
    lib = _lib.load()
    if not (residual.shape == u.shape == hx.shape == hp.shape) or len({residual.dtype, u.dtype, hx.dtype, hp.dtype}) != 1:
        raise RuntimeError("gate_out_fwd: all four operands must have the same shape and dtype")
    r0, rs = _rows(residual)
    u0, us = _rows(u)
    x0, xs = _rows(hx)
    p0, ps = _rows(hp)
    y = torch.empty(residual.shape, dtype=residual.dtype, device=dev)
    with _on_device(dev):
        rc = lib.mega_gate_out_fwd(_ptr(r0), rs, _ptr(u0), us, _ptr(x0), xs, _ptr(p0), ps, _ptr(y), _dtype_code(r0),
                                   _ntok(residual), residual.shape[-1], _stream(dev))
    _lib.check(rc, "gate_out_fwd")
    return y


def ema_backward(y_grad: torch.Tensor, x: torch.Tensor, p: torch.Tensor, q: torch.Tensor, gamma: torch.Tensor,
                 omega: torch.Tensor, padding_mask: Optional[torch.Tensor] = None,
                 layer: Optional[PreparedEMA] = None):
    """Backward of ema_forward (one- or two-sided, no carried state, no truncation):
    -> (x_grad, p_grad [K,N], q_grad [K,N], gamma_grad [K,N], omega_grad [D]); q_grad / gamma_grad are
    complex for the complex layer, in torch's convention for a real loss (dL = Re(conj(grad) dz)).
    It replaces fftconv_bwd + ema_parameters_bwd of the reference
    (fairseq/modules/fused_ops/fftconv.py:32-41, fused_ops/ema_parameters.py:23-33,
    csrc/ops/ema_parameters.cc:80-97) without forming the kernel or its gradient."""
    dev = _need_gpu(y_grad, x, p, q, gamma, omega, padding_mask)
    lib = _lib.load()
    if x.dim() != 3 or y_grad.shape != x.shape:
        raise RuntimeError("x and y_grad must be [B, D, L] of the same shape")
    B, D, L = x.shape
    if layer is None:
        layer = PreparedEMA(p, q, gamma, omega, bidirectional=p.shape[0] == 2 * D)
    N = layer.N
    xd = x.detach()
    g = y_grad.detach().to(xd.dtype)
    if 0 in g.stride() and g.numel() > 0:
        g = g.contiguous()
    dx = layer.adjoint(g, padding_mask)
    K = layer.K                                           # D, or 2 D for a two-sided layer
    dp = torch.empty(K, N, dtype=torch.float32, device=dev)
    dq = torch.empty(K, N, 2, dtype=torch.float32, device=dev)
    dg = torch.empty(K, N, 2, dtype=torch.float32, device=dev)
    dom = torch.empty(D, dtype=torch.float32, device=dev)
    m8 = _mask_u8(padding_mask, B, L)
    stream = _stream(dev)
    # first D rows: the causal half; second D rows (two-sided layers): the same sums over the tokens
    # walked backwards, lags starting at 1 when the layer shifts its backward kernel
    halves = [(0, 0, 0)] + ([(D, 1, 1 if layer.shift else 0)] if layer.bidirectional else [])
    # the sums of one state do not involve the others: more than 16 states go through the kernel 16 at a time
    NS = 16
    scratch_om = dom if (not layer.bidirectional and N <= NS) else torch.empty_like(dom)
    with _on_device(dev):
        for off, rev, lag in halves:
            for n0 in range(0, N, NS):
                n1 = min(N, n0 + NS)
                whole = n0 == 0 and n1 == N
                pp = layer.p[off:off + D] if whole else layer.p[off:off + D, n0:n1].contiguous()
                qq = layer.q[off:off + D] if whole else layer.q[off:off + D, n0:n1].contiguous()
                gg = layer.gamma[off:off + D] if whole else layer.gamma[off:off + D, n0:n1].contiguous()
                if whole:
                    tp, tq, tg = dp[off:], dq[off:], dg[off:]
                else:
                    tp = torch.empty(D, n1 - n0, dtype=torch.float32, device=dev)
                    tq = torch.empty(D, n1 - n0, 2, dtype=torch.float32, device=dev)
                    tg = torch.empty(D, n1 - n0, 2, dtype=torch.float32, device=dev)
                ws = _scratch_buffer(dev, lib.mega_ema_param_grad_workspace_bytes(B, D, n1 - n0), stream)
                rc = lib.mega_ema_param_grad(_ptr(g), _ptr(xd), _dtype_code(xd), g.stride(0), g.stride(1), g.stride(2),
                                             xd.stride(0), xd.stride(1), xd.stride(2), _ptr(pp), _ptr(qq), _ptr(gg),
                                             _ptr(m8), B, D, n1 - n0, L, rev, lag, _ptr(tp), _ptr(tq), _ptr(tg),
                                             _ptr(dom if (off == 0 and n0 == 0) else scratch_om), _ptr(ws), ws.numel(),
                                             stream)
                _lib.check(rc, "ema_param_grad")
                if not whole:
                    dp[off:off + D, n0:n1] = tp
                    dq[off:off + D, n0:n1] = tq
                    dg[off:off + D, n0:n1] = tg
    if layer.is_complex:
        return dx, dp, torch.view_as_complex(dq), torch.view_as_complex(dg), dom
    return dx, dp, dq[..., 0], dg[..., 0], dom


def gate_mul_bwd(y_grad: torch.Tensor, a: torch.Tensor, r: torch.Tensor, r_grad_out: Optional[torch.Tensor] = None):
    """Backward of gate_mul_fwd: -> (a_grad, r_grad); r_grad_out: a row-strided slice to write r_grad into."""
    dev = _need_gpu(y_grad, a, r)
    lib = _lib.load()
    ar, as_ = _rows(a)
    rr, rs = _rows(r)
    g = y_grad.detach().to(a.dtype).contiguous()
    da = torch.empty(a.shape, dtype=a.dtype, device=dev)
    dr, drs = _grad_slot(r_grad_out, a)
    with _on_device(dev):
        rc = lib.mega_gate_mul_bwd_strided(_ptr(g), _ptr(ar), as_, _ptr(rr), rs, _ptr(da), _ptr(dr), drs,
                                           _dtype_code(ar), _ntok(a), a.shape[-1], _stream(dev))
    _lib.check(rc, "gate_mul_bwd")
    return da, dr


def gate_out_bwd(y_grad: torch.Tensor, residual: torch.Tensor, u: torch.Tensor, hx: torch.Tensor, hp: torch.Tensor,
                 u_grad_out: Optional[torch.Tensor] = None, h_grad_out: Optional[torch.Tensor] = None):
    """Backward of gate_out_fwd: -> (residual_grad, u_grad, h_grad); h_grad is the gradient of hx and of hp.
    u_grad_out, h_grad_out: row-strided slices to write those two into."""
    dev = _need_gpu(y_grad, residual, u, hx, hp)
    lib = _lib.load()
    r0, rs = _rows(residual)
    u0, us = _rows(u)
    x0, xs = _rows(hx)
    p0, ps = _rows(hp)
    g = y_grad.detach().to(residual.dtype).contiguous()
    dres = torch.empty(residual.shape, dtype=residual.dtype, device=dev)
    du, dus = _grad_slot(u_grad_out, residual)
    dh, dhs = _grad_slot(h_grad_out, residual)
    with _on_device(dev):
        rc = lib.mega_gate_out_bwd_strided(_ptr(g), _ptr(r0), rs, _ptr(u0), us, _ptr(x0), xs, _ptr(p0), ps, _ptr(dres),
                                           _ptr(du), dus, _ptr(dh), dhs, _dtype_code(r0), _ntok(residual),
                                           residual.shape[-1], _stream(dev))
    _lib.check(rc, "gate_out_bwd")
    return dres, du, dh


def swiglu_bwd(y_grad: torch.Tensor, a: torch.Tensor, b: torch.Tensor):
    """Backward of swiglu: -> (a_grad, b_grad)."""
    dev = _need_gpu(y_grad, a, b)
    lib = _lib.load()
    ad, bd = a.detach().contiguous(), b.detach().contiguous()
    g = y_grad.detach().to(ad.dtype).contiguous()
    da, db = torch.empty_like(ad), torch.empty_like(ad)
    with _on_device(dev):
        rc = lib.mega_swiglu_bwd(_ptr(g), _ptr(ad), _ptr(bd), _ptr(da), _ptr(db), _dtype_code(ad), ad.numel(),
                                 _stream(dev))
    _lib.check(rc, "swiglu_bwd")
    return da, db


def ema_parameters_bwd(w_grad: torch.Tensor, b_grad: Optional[torch.Tensor], p: torch.Tensor, log_q: torch.Tensor,
                       gamma: torch.Tensor, h: Optional[torch.Tensor], v: Optional[torch.Tensor] = None):
    """-> (p_grad [D,N], q_grad [D,N] complex, gamma_grad [D,N] complex, h_grad [B,D,N] complex or None):
    the gradients of ema_parameters_fwd's kernel w [D, L] (and bias b [B, D, L]) outputs.
    Reference: ema_parameters_bwd, fairseq/csrc/ops/ema_parameters.cc:80-186 (`v`, the Vandermonde
    matrix its CUDA path keeps, is not needed).  The power sums sum_l g[l] q^l and sum_l g[l] l q^(l-1)
    come from the parameter-sum kernel of the fused backward: fed a unit impulse as x, its state
    is q^t, so the "kernel gradient" it sees is g itself."""
    dev = _need_gpu(w_grad, b_grad, p, log_q, gamma, h)
    D, N = p.shape
    L = w_grad.shape[-1]
    q = torch.exp(log_q.detach().to(torch.complex64)).reshape(D, N)
    pf = _f32c(p).reshape(D, N)
    gc = gamma.detach().to(torch.complex64).reshape(D, N)
    one = torch.ones(D, N, dtype=torch.float32, device=dev)
    zero = torch.zeros(D, dtype=torch.float32, device=dev)

    def power_sums(g: torch.Tensor):
        """g [R, D, L] -> (S2, S1) [R, D, N] complex: sum_l g q^l, sum_l g l q^(l-1) per row."""
        R = g.shape[0]
        imp = torch.zeros(1, D, L, dtype=torch.float32, device=dev)
        imp[:, :, 0] = 1.0
        s2, s1 = [], []
        for r in range(R):                      # the kernel adds rows up; here every row is wanted by itself
            _, _, dq, dg, _ = ema_backward(g[r:r + 1].float(), imp, one, q, one.to(torch.complex64), zero)
            s2.append(torch.conj(dg))           # with p = gamma = 1: dgamma = conj(S2), dq = conj(S1)
            s1.append(torch.conj(dq))
        return torch.stack(s2), torch.stack(s1)

    S2, S1 = power_sums(w_grad.detach().reshape(1, D, L))
    S2, S1 = S2[0], S1[0]
    p_grad = (S2 * gc).real
    q_grad = torch.conj(S1 * pf * gc)
    gamma_grad = torch.conj(S2 * pf)
    h_grad = None
    if b_grad is not None:
        if h is None:
            raise RuntimeError("ema_parameters_bwd: b_grad needs the carried state h")
        hc = h.detach().to(torch.complex64).reshape(-1, D, N)
        T2, T1 = power_sums(b_grad.detach().reshape(-1, D, L))
        # the bias uses q^(l+1): sum_l g q^(l+1) = q T2, sum_l g (l+1) q^l = T2 + q T1   (ema_parameters.cc:100-116)
        sum2 = q * T2
        sum1 = T2 + q * T1
        q_grad = q_grad + torch.conj(sum1 * gc * hc).sum(0)
        gamma_grad = gamma_grad + torch.conj(sum2 * hc).sum(0)
        h_grad = torch.conj(sum2 * gc)
    return p_grad, q_grad, gamma_grad, h_grad


def ema_hidden_bwd(y_grad: torch.Tensor, x: torch.Tensor, p: torch.Tensor, log_q: torch.Tensor,
                   h: Optional[torch.Tensor], v: Optional[torch.Tensor] = None):
    """-> (x_grad [B,D,L], p_grad [D,N], q_grad [D,N] complex, h_grad [B,D,N] complex or None): the
    gradients of ema_hidden_fwd, h' = q^L h + sum_j p q^(L-1-j) x[j].
    Reference: ema_hidden_bwd, fairseq/csrc/ops/ema_hidden.cc:66-159.  Built from two existing
    kernels: x_grad is the layer's kernel with conj(y_grad) in the place of gamma, read backwards
    (kernel generation); the power sums sum_j x[j] q^(L-1-j) and sum_j x[j] (L-1-j) q^(L-2-j) are the
    state and its q-derivative at the last token, which the parameter-sum kernel returns when its
    "y_grad" is a unit impulse there."""
    dev = _need_gpu(y_grad, x, p, log_q, h)
    B, D, L = x.shape
    N = p.shape[1]
    lq = log_q.detach().to(torch.complex64).reshape(D, N)
    q = torch.exp(lq)
    pf = _f32c(p).reshape(D, N)
    dyc = torch.conj(y_grad.detach().to(torch.complex64).reshape(B, D, N))
    one = torch.ones(D, N, dtype=torch.float32, device=dev)
    zero = torch.zeros(D, dtype=torch.float32, device=dev)
    imp = torch.zeros(1, D, L, dtype=torch.float32, device=dev)
    imp[:, :, L - 1] = 1.0
    xg = torch.empty(B, D, L, dtype=x.dtype, device=dev)
    p_grad = torch.zeros(D, N, dtype=torch.float32, device=dev)
    sum2 = torch.zeros(D, N, dtype=torch.complex64, device=dev)
    xf = x.detach().float()
    for b in range(B):
        w, _, _ = ema_parameters_fwd(pf, lq, dyc[b], None, L)          # Re sum_n p q^l conj(dy): lag l = L-1-j
        xg[b] = w.flip(-1).to(x.dtype)
        _, _, dq1, dg1, _ = ema_backward(imp, xf[b:b + 1], one, q, one.to(torch.complex64), zero)
        s_end, g_end = torch.conj(dg1), torch.conj(dq1)                # with p = gamma = 1
        p_grad += (dyc[b] * s_end).real
        sum2 += dyc[b] * pf * g_end
    q_grad = torch.conj(sum2)
    h_grad = None
    if h is not None:
        hc = h.detach().to(torch.complex64).reshape(B, D, N)
        qL1 = torch.exp(lq * (L - 1))
        q_grad = q_grad + torch.conj((dyc * hc).sum(0) * qL1 * L)
        h_grad = torch.conj(dyc * qL1 * q)
    return xg, p_grad, q_grad, h_grad
