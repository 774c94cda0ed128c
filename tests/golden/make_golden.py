"""Writes tests/golden/ref_cpu_vectors.npz: inputs and outputs of the reference's own CPU
operators for this path, produced by oracle/_ref (fairseq/csrc/ops/timestep_norm.cc,
ema_parameters.cc, ema_hidden.cc, sequence_norm.cc compiled in place by `make -C oracle ref`).

    python tests/golden/make_golden.py

The file holds data only (seeded inputs, the reference's outputs); it lets the parity tests
run where neither the reference tree nor oracle/_ref exist.
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))


def load_ref():
    path = os.path.join(ROOT, "oracle", "_ref", "mega2_ref_cpu.so")
    old = sys.getdlopenflags()
    sys.setdlopenflags(os.RTLD_LAZY | os.RTLD_GLOBAL)
    try:
        spec = importlib.util.spec_from_file_location("mega2_ref_cpu", path)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
    finally:
        sys.setdlopenflags(old)
    return mod


def main():
    from conftest import mega_init_complex
    from oracle import mega_oracle as O

    ref = load_ref()
    out = {}
    t = torch.from_numpy

    # group TimestepNorm: ragged padding, carried statistics, non-trivial affine
    rng = np.random.default_rng(20240)
    for tag, (B, L, H, G, masked) in {"gtsn_a": (3, 37, 48, 4, True), "gtsn_b": (2, 130, 64, 16, False),
                                      "gtsn_c": (1, 1, 32, 2, False)}.items():
        x = rng.normal(size=(B, L, H)).astype(np.float32) * 1.7 + 0.3
        mask = (rng.random((B, L)) < 0.25) if masked else None
        pc = rng.integers(0, 6, B).astype(np.int64)
        pm = (rng.normal(size=(B, G)) * 0.2).astype(np.float32)
        pv = (rng.random((B, G)) + 0.5).astype(np.float32)
        pm[pc == 0] = 0.0
        pv[pc == 0] = 1.0
        gamma = (rng.normal(size=H) + 1).astype(np.float32)
        beta = rng.normal(size=H).astype(np.float32)
        y, c, mu, v = ref.group_timestep_norm_fwd(t(x), t(pc), t(pm), t(pv), t(gamma), t(beta),
                                                  None if mask is None else t(mask), G, 1e-5)[:4]
        out.update({f"{tag}.x": x, f"{tag}.prev_count": pc, f"{tag}.prev_mean": pm, f"{tag}.prev_var": pv,
                    f"{tag}.gamma": gamma, f"{tag}.beta": beta, f"{tag}.groups": np.int64(G),
                    f"{tag}.y": y.numpy(), f"{tag}.count": c.numpy(), f"{tag}.mean": mu.numpy(),
                    f"{tag}.var": v.numpy()})
        if mask is not None:
            out[f"{tag}.mask"] = mask

    # per-feature TimestepNorm
    B, L, H = 2, 41, 24
    x = rng.normal(size=(B, L, H)).astype(np.float32)
    mask = rng.random((B, L)) < 0.2
    pc = np.array([0, 3], np.int64)
    pm = np.zeros((B, H), np.float32)
    pv = np.ones((B, H), np.float32)
    pm[1] = rng.normal(size=H) * 0.1
    pv[1] = rng.random(H) + 0.5
    gamma = (rng.normal(size=H) + 1).astype(np.float32)
    beta = rng.normal(size=H).astype(np.float32)
    y, c, mu, v = ref.timestep_norm_fwd(t(x), t(pc), t(pm), t(pv), t(gamma), t(beta), t(mask), 1e-5)[:4]
    out.update({"tsn.x": x, "tsn.mask": mask, "tsn.prev_count": pc, "tsn.prev_mean": pm, "tsn.prev_var": pv,
                "tsn.gamma": gamma, "tsn.beta": beta, "tsn.y": y.numpy(), "tsn.count": c.numpy(),
                "tsn.mean": mu.numpy(), "tsn.var": v.numpy()})

    # kernel generation (with and without a carried state) and the hidden-state update
    K, N, L, B = 6, 16, 96, 2
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    p = p.astype(np.float32)
    q = q.astype(np.complex64)
    g = g.astype(np.complex64)
    h = (rng.normal(size=(B, K, N)) + 1j * rng.normal(size=(B, K, N))).astype(np.complex64)
    log_q = t(q).log()
    w, b, _ = ref.ema_parameters_fwd(t(p), log_q, t(g), t(h), L)
    x = rng.normal(size=(B, K, L)).astype(np.float32)
    hy, _ = ref.ema_hidden_fwd(t(x), t(p), log_q, t(h))
    hy0, _ = ref.ema_hidden_fwd(t(x), t(p), log_q, None)
    out.update({"ema.p": p, "ema.q": q, "ema.log_q": log_q.numpy(), "ema.gamma": g, "ema.h": h, "ema.x": x,
                "ema.length": np.int64(L), "ema.kernel": w.numpy(), "ema.bias": b.numpy(),
                "ema.hidden": hy.numpy(), "ema.hidden_zero_start": hy0.numpy()})

    # backward operators (own generator, so the arrays above keep their values).  TimestepNorm
    # cases have padding at the end of the rows only: behind an interior masked token the
    # reference's CPU forward stores a cumulative mean that includes the masked token
    # (timestep_norm.cc:291-296), and its backward then differentiates a different function.
    rng = np.random.default_rng(20241)
    for tag, (B, L, H, G, pad) in {"gtsn_bwd_a": (2, 45, 48, 4, True), "gtsn_bwd_b": (3, 70, 64, 16, False),
                                   "tsn_bwd": (2, 33, 24, None, True)}.items():
        GG = H if G is None else G
        x = (rng.normal(size=(B, L, H)) * 1.4 + 0.2).astype(np.float32)
        mask = None
        if pad:
            mask = np.zeros((B, L), bool)
            for b in range(B):
                mask[b, L - int(rng.integers(1, 9)):] = True
        pc = rng.integers(1, 6, B).astype(np.int64)
        pm = (rng.normal(size=(B, GG)) * 0.2).astype(np.float32)
        pv = (rng.random((B, GG)) + 0.5).astype(np.float32)
        gamma = (rng.normal(size=H) * 0.3 + 1).astype(np.float32)
        beta = rng.normal(size=H).astype(np.float32)
        dy = rng.normal(size=(B, L, H)).astype(np.float32)
        dm = rng.normal(size=(B, GG)).astype(np.float32)
        dv = rng.normal(size=(B, GG)).astype(np.float32)
        tm = None if mask is None else t(mask)
        if G is None:
            y, c, mu, v, cm, cr = ref.timestep_norm_fwd(t(x), t(pc), t(pm), t(pv), t(gamma), t(beta), tm, 1e-5)
            gr = ref.timestep_norm_bwd(t(dy), t(dm), t(dv), t(x), t(pm), c, cm, cr, t(gamma), tm)
        else:
            y, c, mu, v, gm, cm, cr = ref.group_timestep_norm_fwd(t(x), t(pc), t(pm), t(pv), t(gamma), t(beta), tm, G,
                                                                  1e-5)
            gr = ref.group_timestep_norm_bwd(t(dy), t(dm), t(dv), t(x), t(pm), c, gm, cm, cr, t(gamma), tm, G)
        out.update({f"{tag}.x": x, f"{tag}.prev_count": pc, f"{tag}.prev_mean": pm, f"{tag}.prev_var": pv,
                    f"{tag}.gamma": gamma, f"{tag}.beta": beta, f"{tag}.groups": np.int64(0 if G is None else G),
                    f"{tag}.y_grad": dy, f"{tag}.mean_grad": dm, f"{tag}.var_grad": dv,
                    f"{tag}.x_grad": gr[0].numpy(), f"{tag}.prev_mean_grad": gr[1].numpy(),
                    f"{tag}.prev_var_grad": gr[2].numpy(), f"{tag}.gamma_grad": gr[3].numpy(),
                    f"{tag}.beta_grad": gr[4].numpy()})
        if mask is not None:
            out[f"{tag}.mask"] = mask

    # kernel gradient -> coefficient gradients
    K, N, L = 5, 16, 80
    p, q, g = O.ema_coeffs_complex(*mega_init_complex(rng, K, N))
    p, q, g = p.astype(np.float32), q.astype(np.complex64), g.astype(np.complex64)
    dk = rng.normal(size=(K, L)).astype(np.float32)
    log_q = t(q).log()
    w, _, vander = ref.ema_parameters_fwd(t(p), log_q, t(g), None, L)
    dp, dq, dg, _ = ref.ema_parameters_bwd(t(dk), None, t(p), log_q, t(g), None, vander)
    out.update({"ema_bwd.p": p, "ema_bwd.q": q, "ema_bwd.gamma": g, "ema_bwd.kernel_grad": dk,
                "ema_bwd.p_grad": dp.numpy(), "ema_bwd.q_grad": dq.numpy(), "ema_bwd.gamma_grad": dg.numpy()})
    # the same with a carried state: the bias gradient adds to dq, dgamma and gives dh
    hb = (rng.normal(size=(2, K, N)) + 1j * rng.normal(size=(2, K, N))).astype(np.complex64)
    db = rng.normal(size=(2, K, L)).astype(np.float32)
    _, _, vander = ref.ema_parameters_fwd(t(p), log_q, t(g), t(hb), L)
    dp2, dq2, dg2, dh2 = ref.ema_parameters_bwd(t(dk), t(db), t(p), log_q, t(g), t(hb), vander)
    out.update({"ema_bwd.h": hb, "ema_bwd.bias_grad": db, "ema_bwd.p_grad_b": dp2.numpy(), "ema_bwd.q_grad_b": dq2.numpy(),
                "ema_bwd.gamma_grad_b": dg2.numpy(), "ema_bwd.h_grad_b": dh2.numpy()})

    # hidden-state update backward (with a carried state)
    B2, L2 = 2, 40
    xh = rng.normal(size=(B2, K, L2)).astype(np.float32)
    hh = (rng.normal(size=(B2, K, N)) + 1j * rng.normal(size=(B2, K, N))).astype(np.complex64)
    dhy = (rng.normal(size=(B2, K, N)) + 1j * rng.normal(size=(B2, K, N))).astype(np.complex64)
    _, vh = ref.ema_hidden_fwd(t(xh), t(p), log_q, t(hh))
    gx, gp, gq, gh = ref.ema_hidden_bwd(t(dhy), t(xh), t(p), log_q, t(hh), vh)
    out.update({"hid_bwd.x": xh, "hid_bwd.h": hh, "hid_bwd.y_grad": dhy, "hid_bwd.p": p, "hid_bwd.q": q,
                "hid_bwd.x_grad": gx.numpy(), "hid_bwd.p_grad": gp.numpy(), "hid_bwd.q_grad": gq.numpy(),
                "hid_bwd.h_grad": gh.numpy()})

    # SequenceNorm: both layouts, group and per-feature, ragged padding
    rng = np.random.default_rng(20242)
    for tag, (B, L, H, G, last, masked) in {"gsn_a": (3, 37, 48, 4, False, True), "gsn_b": (2, 130, 64, 16, True, True),
                                           "gsn_c": (2, 50, 32, 2, True, False), "sn_a": (2, 41, 24, None, True, True),
                                           "sn_b": (2, 33, 20, None, False, False)}.items():
        x = (rng.normal(size=(B, H, L) if last else (B, L, H)) * 1.6 + 0.4).astype(np.float32)
        mask = (rng.random((B, L)) < 0.25) if masked else None
        gamma = (rng.normal(size=H) * 0.3 + 1).astype(np.float32)
        beta = rng.normal(size=H).astype(np.float32)
        tm = None if mask is None else t(mask)
        if G is None:
            y, c, mu, r = ref.sequence_norm_fwd(t(x), t(gamma), t(beta), tm, 1e-5, last)
        else:
            y, c, mu, r = ref.group_sequence_norm_fwd(t(x), t(gamma), t(beta), tm, G, 1e-5, last)
        out.update({f"{tag}.x": x, f"{tag}.gamma": gamma, f"{tag}.beta": beta, f"{tag}.groups": np.int64(0 if G is None else G),
                    f"{tag}.length_last": np.int64(1 if last else 0), f"{tag}.y": y.numpy(), f"{tag}.count": c.numpy(),
                    f"{tag}.mean": mu.numpy(), f"{tag}.rstd": r.numpy()})
        if mask is not None:
            out[f"{tag}.mask"] = mask

    # SequenceNorm backward
    rng = np.random.default_rng(20243)
    for tag, (B, L, H, G, last, masked) in {"gsn_bwd_a": (2, 45, 48, 4, True, True), "gsn_bwd_b": (3, 40, 32, 8, False, True),
                                           "sn_bwd": (2, 33, 24, None, True, False)}.items():
        x = (rng.normal(size=(B, H, L) if last else (B, L, H)) * 1.3 + 0.3).astype(np.float32)
        dy = rng.normal(size=x.shape).astype(np.float32)
        mask = (rng.random((B, L)) < 0.25) if masked else None
        gamma = (rng.normal(size=H) * 0.3 + 1).astype(np.float32)
        beta = rng.normal(size=H).astype(np.float32)
        tm = None if mask is None else t(mask)
        if G is None:
            y, c, mu, r = ref.sequence_norm_fwd(t(x), t(gamma), t(beta), tm, 1e-5, last)
            gr = ref.sequence_norm_bwd(t(dy), t(x), c, mu, r, t(gamma), tm, last)
        else:
            y, c, mu, r = ref.group_sequence_norm_fwd(t(x), t(gamma), t(beta), tm, G, 1e-5, last)
            gr = ref.group_sequence_norm_bwd(t(dy), t(x), c, mu, r, t(gamma), tm, G, last)
        out.update({f"{tag}.x": x, f"{tag}.y_grad": dy, f"{tag}.gamma": gamma, f"{tag}.beta": beta,
                    f"{tag}.groups": np.int64(0 if G is None else G), f"{tag}.length_last": np.int64(1 if last else 0),
                    f"{tag}.x_grad": gr[0].numpy(), f"{tag}.gamma_grad": gr[1].numpy(), f"{tag}.beta_grad": gr[2].numpy()})
        if mask is not None:
            out[f"{tag}.mask"] = mask

    dst = os.path.join(HERE, "ref_cpu_vectors.npz")
    np.savez_compressed(dst, **out)
    print(dst, os.path.getsize(dst), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
