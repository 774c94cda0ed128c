"""ctypes binding of libmega_hip.so (the C ABI declared in include/mega_hip.h).

The library is the product: there is no CPU or PyTorch fallback.  If it has not been
built, loading raises with the build command; if a call is rejected, the reason the
library recorded is raised as RuntimeError (the reference raises RuntimeError from
TORCH_CHECK in the same situations).
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmega_hip.so")

F32, BF16, F16 = 0, 1, 2

_p = C.c_void_p
_i64 = C.c_int64
_int = C.c_int
_sz = C.c_size_t

# name -> (restype, argtypes); must list every symbol of include/mega_hip.h
SIGNATURES = {
    "mega_last_error": (C.c_char_p, []),
    "mega_abi_version": (_int, []),
    "mega_lookback_init": (_int, []),
    "mega_lookback_status": (_int, [_int]),
    "mega_lookback_checked": (None, [_int]),
    "mega_test_lookback": (None, [C.c_uint, _int, _int]),
    "mega_test_timestep_norm_bwd_onepass": (None, [_int]),
    "mega_audit_begin": (None, []),
    "mega_audit_add": (_int, [_p, _sz]),
    "mega_audit_end": (_int, [C.POINTER(_int)]),
    "mega_ema_parameters_fwd": (_int, [_p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _p, _p]),
    "mega_ema_hidden_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64]),
    "mega_ema_hidden_fwd": (_int, [_p, _int, _i64, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _p, _sz, _p]),
    "mega_ema_fwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _int, _i64]),
    "mega_ema_fwd": (_int, [_p, _p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _int, _p, _p, _p, _p,
                            _i64, _i64, _i64, _i64, _int, _i64, _int, _p, _p, _sz, _p]),
    "mega_ema_image_bytes": (_sz, [_i64, _i64, _int]),
    "mega_ema_prepare": (_int, [_p, _p, _p, _int, _p, _i64, _i64, _int, _int, _p, _sz, _p]),
    "mega_ema_step": (_int, [_p, _p, _int, _p, _p, _p, _int, _p, _p, _p, _i64, _i64, _i64, _p]),
    "mega_norm_ema_step": (_int, [_p, _p, _p, _int, _p, _p, _p, _p, _p, _p, _p, _p, C.c_double, _p, _p, _p, _int, _p, _p,
                                  _p, _i64, _i64, _i64, _i64, _p]),
    "mega_norm_ema_steps": (_int, [_p, _p, _p, _int, _i64, _p, _p, _p, _p, _p, _p, _p, _p, C.c_double, _p, _p, _p, _int,
                                   _p, _p, _p, _i64, _i64, _i64, _i64, _p]),
    "mega_norm_ema_fwd_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64]),
    "mega_norm_ema_fwd_scratch_bytes": (_sz, [_i64, _i64, _i64, _i64, _i64]),
    "mega_norm_ema_fwd": (_int, [_p, _p, _p, _int, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p, C.c_double, _p, _p, _p,
                                 _p, _p, _p, _int, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _sz, _p, _sz, _p]),
    "mega_norm_ema_fwd_train": (_int, [_p, _p, _p, _int, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p, C.c_double, _p, _p,
                                       _p, _p, _p, _p, _p, _p, _int, _p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p, _p,
                                       _sz, _p, _sz, _p]),
    "mega_ema_param_grad_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "mega_ema_param_grad": (_int, [_p, _p, _int, _i64, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p, _i64, _i64, _i64,
                                   _i64, _int, _int, _p, _p, _p, _p, _p, _sz, _p]),
    "mega_long_conv_fwd": (_int, [_p, _p, _int, _p, _i64, _i64, _i64, _i64, _int, _int, _p]),
    "mega_timestep_norm_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64]),
    "mega_group_timestep_norm_fwd": (_int, [_p, _p, _int, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, C.c_double,
                                            _p, _p, _p, _p, _p, _p, _p, _sz, _p]),
    "mega_group_timestep_norm_fwd_noalloc": (_int, [_p, _p, _int, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64,
                                                    C.c_double, _p, _p, _p, _p, _p, _p, _p]),
    "mega_timestep_norm_fwd": (_int, [_p, _p, _int, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, C.c_double,
                                      _p, _p, _p, _p, _p, _p, _sz, _p]),
    "mega_timestep_norm_bwd_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64]),
    "mega_group_timestep_norm_bwd": (_int, [_p, _p, _p, _p, _int, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64,
                                            _p, _p, _p, _p, _p, _p, _sz, _p]),
    "mega_timestep_norm_bwd": (_int, [_p, _p, _p, _p, _int, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64,
                                      _p, _p, _p, _p, _p, _p, _sz, _p]),
    "mega_sequence_norm_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64, _int]),
    "mega_group_sequence_norm_fwd": (_int, [_p, _p, _int, _p, _p, _p, _i64, _i64, _i64, _i64, C.c_double, _int,
                                            _p, _p, _p, _p, _sz, _p]),
    "mega_sequence_norm_fwd": (_int, [_p, _p, _int, _p, _p, _p, _i64, _i64, _i64, C.c_double, _int,
                                      _p, _p, _p, _p, _sz, _p]),
    "mega_sequence_norm_bwd_workspace_bytes": (_sz, [_i64, _i64, _i64]),
    "mega_group_sequence_norm_bwd": (_int, [_p, _p, _int, _p, _p, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _p, _p,
                                            _p, _sz, _p]),
    "mega_attention_softmax_fwd": (_int, [_p, _p, _int, _i64, _i64, _i64, _int, C.c_float, C.c_uint64, _p]),
    "mega_attention_bwd_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64, _i64]),
    "mega_attention_bwd": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, C.c_float, _int,
                                  _p, _sz, _p]),
    "mega_attention_softmax_bwd": (_int, [_p, _p, _p, _int, _i64, _i64, _i64, _int, C.c_float, _p]),
    "mega_attention_workspace_bytes": (_sz, [_int, _i64, _i64, _i64, _i64, _i64]),
    "mega_attention_fwd": (_int, [_p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, C.c_float, _int, C.c_float,
                                  C.c_uint64, _p, _sz, _p]),
    "mega_swiglu_fwd": (_int, [_p, _p, _p, _int, _i64, _p]),
    "mega_silu_fwd": (_int, [_p, _p, _int, _i64, _p]),
    "mega_rms_norm_fwd": (_int, [_p, _i64, _p, _p, _int, _i64, _i64, C.c_double, _p]),
    "mega_gate_qk_fwd": (_int, [_p, _i64, _p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, C.c_double, _p]),
    "mega_gate_qk_bwd_workspace_bytes": (_sz, [_i64, _i64]),
    "mega_gate_qk_bwd": (_int, [_p, _p, _p, _i64, _p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _i64, _i64, C.c_double,
                                _p, _sz, _p]),
    "mega_gate_mul_fwd": (_int, [_p, _i64, _p, _i64, _p, _int, _i64, _i64, _p]),
    "mega_gate_out_fwd": (_int, [_p, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _int, _i64, _i64, _p]),
    "mega_gate_mul_bwd": (_int, [_p, _p, _i64, _p, _i64, _p, _p, _int, _i64, _i64, _p]),
    "mega_gate_out_bwd": (_int, [_p, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _p, _p, _int, _i64, _i64, _p]),
    "mega_swiglu_bwd": (_int, [_p, _p, _p, _p, _p, _int, _i64, _p]),
    "mega_silu_bwd": (_int, [_p, _p, _p, _int, _i64, _p]),
    "mega_colsum_workspace_bytes": (_sz, [_i64, _i64]),
    "mega_colsum": (_int, [_p, _i64, _int, _i64, _i64, _p, _int, _p, _sz, _p]),
    "mega_transpose_2d": (_int, [_p, _p, _int, _i64, _i64, _i64, _int, _int, _p]),
    "mega_ema_coeffs_fwd": (_int, [_p, _p, _p, _p, _p, _int, _int, _i64, _i64, _i64, _p, _p, _p, _p, _p]),
    "mega_ema_coeffs_bwd": (_int, [_p, _p, _p, _p, _p, _p, _p, _int, _int, _i64, _i64, _i64, _p, _p, _p, _p, _p, _p]),
    "mega_norm_params_fwd": (_int, [_p, _p, _int, _p, _p, _int, _i64, _i64, _i64, _p, _p, _p, _p, _p]),
    "mega_norm_params_bwd": (_int, [_p, _p, _p, _p, _p, _int, _int, _i64, _i64, _i64, _p, _p, _p, _p, _p]),
    "mega_gate_qk_bwd_strided": (_int, [_p, _p, _p, _i64, _p, _p, _p, _i64, _p, _p, _int, _i64, _i64, _i64, _i64, _i64,
                                        C.c_double, _p, _sz, _p]),
    "mega_gate_mul_bwd_strided": (_int, [_p, _p, _i64, _p, _i64, _p, _p, _i64, _int, _i64, _i64, _p]),
    "mega_gate_out_bwd_strided": (_int, [_p, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _p, _i64, _p, _i64, _int, _i64,
                                         _i64, _p]),
}

_lib = None


def load() -> C.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python fairseq-apollo_amd/build.py` "
            "(hipcc --offload-arch=gfx950).  There is no fallback path."
        )
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().mega_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what}: {msg} (code {rc})")
