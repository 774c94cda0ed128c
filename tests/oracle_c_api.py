"""ctypes wrappers around the plain-C oracle (oracle/libmega_oracle.so): numpy in, numpy out.
Shared by the tests, __graft_entry__.smoke() and the cpu_baseline leg of bench.py."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_PATH = os.path.join(ROOT, "oracle", "libmega_oracle.so")
_lib = None


def lib():
    global _lib
    if _lib is None:
        src = os.path.join(ROOT, "oracle", "mega_oracle.c")
        if not os.path.exists(_PATH) or os.path.getmtime(_PATH) < os.path.getmtime(src):
            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "oracle"])
        _lib = C.CDLL(_PATH)
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _cplx2(a, dt):
    a = np.asarray(a)
    out = np.empty(a.shape + (2,), dt)
    out[..., 0] = a.real
    out[..., 1] = a.imag
    return np.ascontiguousarray(out)


def ema_kernel(p, q, gamma, L, dt=np.float64):
    K, N = p.shape
    sfx = "f64" if dt == np.float64 else "f32"
    w = np.empty((K, L), dt)
    lq = _cplx2(np.log(np.asarray(q).astype(np.complex128)), dt)
    g = _cplx2(gamma, dt)
    pp = np.ascontiguousarray(p, dt)
    getattr(lib(), "ora_ema_kernel_" + sfx)(_p(pp), _p(lq), _p(g), C.c_int64(K), C.c_int64(N), C.c_int64(L), _p(w))
    return w


def ema_bias(q, gamma, h, L, dt=np.float64):
    B, K, N = h.shape
    sfx = "f64" if dt == np.float64 else "f32"
    b = np.empty((B, K, L), dt)
    lq = _cplx2(np.log(np.asarray(q).astype(np.complex128)), dt)
    getattr(lib(), "ora_ema_bias_" + sfx)(_p(lq), _p(_cplx2(gamma, dt)), _p(_cplx2(h, dt)), C.c_int64(B),
                                          C.c_int64(K), C.c_int64(N), C.c_int64(L), _p(b))
    return b


def ema_hidden(x, p, q, h=None, dt=np.float64):
    B, D, L = x.shape
    N = p.shape[1]
    sfx = "f64" if dt == np.float64 else "f32"
    y = np.empty((B, D, N, 2), dt)
    lq = _cplx2(np.log(np.asarray(q).astype(np.complex128)), dt)
    hh = None if h is None else _cplx2(h, dt)
    getattr(lib(), "ora_ema_hidden_" + sfx)(_p(np.ascontiguousarray(x, dt)), _p(np.ascontiguousarray(p, dt)), _p(lq),
                                            _p(hh), C.c_int64(B), C.c_int64(D), C.c_int64(N), C.c_int64(L), _p(y))
    return y[..., 0] + 1j * y[..., 1]


def causal_conv_direct(x, k):
    B, D, L = x.shape
    Lk = k.shape[1]
    y = np.empty((B, D, L), np.float64)
    lib().ora_causal_conv_direct_f64(_p(np.ascontiguousarray(x, np.float64)), _p(np.ascontiguousarray(k, np.float64)),
                                     C.c_int64(B), C.c_int64(D), C.c_int64(L), C.c_int64(Lk), _p(y))
    return y


def timestep_norm(x, prev_count, prev_mean, prev_var, gamma, beta, mask=None, num_groups=None, eps=1e-5,
                  dt=np.float64):
    B, L, H = x.shape
    sfx = "f64" if dt == np.float64 else "f32"
    G = H if num_groups is None else num_groups
    xx = np.ascontiguousarray(x, dt)
    y = np.empty_like(xx)
    count = np.empty(B, np.int64)
    mean = np.empty((B, G), dt)
    var = np.empty((B, G), dt)
    pc = np.ascontiguousarray(prev_count, np.int64)
    pm = np.ascontiguousarray(prev_mean, dt).reshape(B, G)
    pv = np.ascontiguousarray(prev_var, dt).reshape(B, G)
    gm = np.ascontiguousarray(gamma, dt)
    bt = np.ascontiguousarray(beta, dt)
    mk = None if mask is None else np.ascontiguousarray(mask, np.uint8)
    if num_groups is None:
        getattr(lib(), "ora_timestep_norm_" + sfx)(_p(xx), _p(pc), _p(pm), _p(pv), _p(gm), _p(bt), _p(mk),
                                                   C.c_int64(B), C.c_int64(L), C.c_int64(H), C.c_double(eps), _p(y),
                                                   _p(count), _p(mean), _p(var))
    else:
        scratch = np.empty(2 * B * L * G, dt)
        getattr(lib(), "ora_group_timestep_norm_" + sfx)(_p(xx), _p(pc), _p(pm), _p(pv), _p(gm), _p(bt), _p(mk),
                                                         C.c_int64(B), C.c_int64(L), C.c_int64(H), C.c_int64(G),
                                                         C.c_double(eps), _p(y), _p(count), _p(mean), _p(var),
                                                         _p(scratch))
    return y, count, mean, var


def attention_softmax(x, causal):
    x = np.ascontiguousarray(x, np.float64)
    outer, inner = x.shape[-2], x.shape[-1]
    batch = x.size // (outer * inner)
    y = np.empty_like(x)
    lib().ora_attention_softmax_f64(_p(x), C.c_int64(batch), C.c_int64(outer), C.c_int64(inner),
                                    C.c_int(1 if causal else 0), _p(y))
    return y
