"""Writes tests/golden/position_vectors.npz: inputs and outputs of the reference's two positional modules,
RotaryEmbedding and SimpleRelativePositionalBias (fairseq/modules/relative_positional_bias.py:13-94).

    python tests/golden/make_position_golden.py

That file imports nothing but torch, so it is loaded here by path (no `import fairseq`), in the container
that holds the reference tree.  The closed forms and invariants the oracle tests use (norm kept, position 0
unchanged, scores depend on the position difference) do not fix the frequency convention of the rotation or
the index arithmetic of the pad / tile / view construction of the bias matrix; these vectors do.  The output
file holds data only (seeded inputs, the reference's outputs).
"""
import importlib.util
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/fairseq/modules/relative_positional_bias.py"


def main():
    spec = importlib.util.spec_from_file_location("ref_relative_positional_bias", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    out = {}
    gen = torch.Generator().manual_seed(4242)
    # rotary: [B, C, S] as the layer passes it (positions restart with every chunk); a query offset as in
    # incremental decoding (one query at the end of the cached keys); a non-default base
    for tag, (B, C, S, base, qidx) in {"rot_a": (3, 7, 8, None, 0), "rot_b": (2, 16, 64, None, 0),
                                      "rot_c": (2, 9, 6, 500.0, 0), "rot_d": (2, 5, 8, None, 4)}.items():
        m = mod.RotaryEmbedding(S, 32, base)
        xk = torch.randn(B, C, S, generator=gen, dtype=torch.float64)
        xq = torch.randn(B, 1 if qidx else C, S, generator=gen, dtype=torch.float64)
        q, k = m(xq, xk, qidx=qidx)
        out.update({f"{tag}.xq": xq.numpy(), f"{tag}.xk": xk.numpy(), f"{tag}.q": q.double().numpy(),
                    f"{tag}.k": k.double().numpy(), f"{tag}.base": np.float64(10000.0 if base is None else base),
                    f"{tag}.qidx": np.int64(qidx), f"{tag}.freqs": m.freqs.double().numpy()})
    # learned bias per relative offset: the [C, C] matrix the attention adds to q k^T
    for tag, (mp, C) in {"bias_a": (16, 5), "bias_b": (16, 16), "bias_c": (9, 1), "bias_d": (33, 12)}.items():
        m = mod.SimpleRelativePositionalBias(mp)
        with torch.no_grad():
            m.rel_pos_bias.copy_(torch.randn(2 * mp - 1, generator=gen))
        out.update({f"{tag}.param": m.rel_pos_bias.detach().double().numpy(), f"{tag}.C": np.int64(C),
                    f"{tag}.matrix": m(C).detach().double().numpy()})
    path = os.path.join(HERE, "position_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, len(out), "arrays")


if __name__ == "__main__":
    main()
