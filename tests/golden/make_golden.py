"""Writes tests/golden/moda_small.npz.

The reference ships no vectors for this path, so the fixture is produced by the
oracle's literal fp64 row loops (form (i), the transcription of
moda_v14.py:1900-1991, moda_v16.py:2487-2582, fda_v12.py:1143-1196) with
gradients from fp64 autograd of the dense form, on seeded inputs that
``oracle.make_inputs`` regenerates.  Stored as fp32.  Run from the repo root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", ".."))
import oracle  # noqa: E402

CASES = {  # mode: (B, T, H, D, L, G, seed, chunk_tokens)
    "causal": (1, 48, 2, 64, 4, 2, 100, 0),
    "noncausal": (1, 37, 2, 64, 3, 1, 101, 0),
    "chunk_visible": (1, 40, 2, 64, 3, 2, 102, 4),
    "depth_only": (1, 33, 2, 64, 5, 2, 103, 0),
}


def main():
    out = {}
    for mode, (B, T, H, D, L, G, seed, cb) in CASES.items():
        inp = oracle.make_inputs(B, T, H, D, L, G, seed=seed, dtype=torch.float32, std=0.5,
                                 depth_only=(mode == "depth_only"))
        o, lse = oracle.moda_rows(inp["q"], inp["k"], inp["v"], inp["kd"], inp["vd"], D ** -0.5, G, mode, cb,
                                  dtype=torch.float64)
        r = oracle.moda_dense_fwd_bwd(inp, D ** -0.5, G, mode, cb, dtype=torch.float64)
        assert torch.allclose(o, r["o"], atol=1e-12) and torch.allclose(lse, r["lse"], atol=1e-12)
        out[f"{mode}_meta"] = np.array([B, T, H, D, L, G, seed], dtype=np.int64)
        out[f"{mode}_o"] = o.numpy().astype(np.float32)
        out[f"{mode}_lse"] = lse.numpy().astype(np.float32)
        for n in ("dq", "dk", "dv", "dkd", "dvd"):
            if r[n] is not None:
                out[f"{mode}_{n}"] = r[n].numpy().astype(np.float32)
    path = os.path.join(os.path.dirname(__file__), "moda_small.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
