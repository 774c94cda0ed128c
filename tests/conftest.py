import ctypes
import importlib.util
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def rel_err(a, b, eps=1.0):
    """max |a - b| / max(|b|, eps * rms(b)) elementwise-maximised: the error measure of all
    parity tests (eps = 1 keeps near-zero reference entries from dominating)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    rms = float(np.sqrt(np.mean(b * b))) if b.size else 0.0
    den = np.maximum(np.abs(b), eps * rms + 1e-300)
    return float(np.max(np.abs(a - b) / den)) if b.size else 0.0


@pytest.fixture(scope="session")
def oracle_c():
    """The plain-C oracle (oracle/libmega_oracle.so), built on demand with gcc."""
    path = os.path.join(ROOT, "oracle", "libmega_oracle.so")
    src = os.path.join(ROOT, "oracle", "mega_oracle.c")
    if not os.path.exists(path) or os.path.getmtime(path) < os.path.getmtime(src):
        import subprocess
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "oracle"])
    return ctypes.CDLL(path)


@pytest.fixture(scope="session")
def ref_cpu():
    """The reference's own CPU translation units, compiled in place by `make -C oracle ref`
    into oracle/_ref (git-ignored).  Tests that need it are skipped where it was not built."""
    path = os.path.join(ROOT, "oracle", "_ref", "mega2_ref_cpu.so")
    if not os.path.exists(path):
        pytest.skip("oracle/_ref not built (needs the reference tree: make -C oracle ref)")
    import torch  # noqa: F401  (the extension links against libtorch)
    old = sys.getdlopenflags()
    # the CUDA entry points the translation units dispatch to stay unresolved: bind lazily
    sys.setdlopenflags(os.RTLD_LAZY | os.RTLD_GLOBAL)
    try:
        spec = importlib.util.spec_from_file_location("mega2_ref_cpu", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
    finally:
        sys.setdlopenflags(old)
    return mod


def mega_init_real(rng, K, N):
    """Mega initialisation of the real EMA (exponential_moving_average.py:56-69)."""
    alpha = rng.normal(0, 0.2, (K, N, 1))
    delta = rng.normal(0, 0.2, (K, N, 1))
    beta = rng.normal(0, 0.02, (K, N, 1)) + np.where(np.arange(N) % 2 == 0, 1.0, -1.0).reshape(1, N, 1)
    gamma = rng.normal(0, 1.0, (K, N))
    return alpha, delta, beta, gamma


def mega_init_complex(rng, K, N, theta_uniform=True):
    """Complex EMA parameters; theta ~ U(0, pi) expressed through the module's
    parametrisation sigmoid(theta_param) 2 pi = theta."""
    alpha = rng.normal(0, 0.2, (K, N, 1))
    delta = rng.normal(0, 0.2, (K, N, 1))
    th = rng.uniform(0.02, np.pi - 0.02, (K, 1, 1))
    frac = th / (2 * np.pi)
    theta = np.log(frac / (1 - frac))
    gamma = np.zeros((K, N, 2))
    gamma[..., 0] = rng.normal(0, 1.0, (K, N))
    return alpha, delta, theta, gamma
