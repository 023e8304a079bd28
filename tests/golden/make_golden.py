"""Writes tests/golden/castle_small.npz: seeded inputs and the oracle's outputs for them.

The reference holds no numeric fixtures for this path (its tests are property checks on
unseeded inputs), and the oracle is pinned by closed forms and brute force in
tests/test_oracle_core.py, so these vectors come from the oracle (fp64, stored as fp32).
They freeze the expected numbers: a later change of the oracle or of the kernels that moves
any of them fails tests/test_golden.py.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import castle_oracle as O  # noqa: E402

CASES = {"a": (1, 2, 24, 16), "b": (1, 1, 70, 32), "c": (1, 1, 72, 64)}   # B, H, L, d


def main():
    blob = {}
    for name, (B, H, L, d) in CASES.items():
        g = torch.Generator().manual_seed(1234 + L)
        ops = [torch.randn(B, H, L, d, generator=g).float() * 0.7 for _ in range(6)]   # qc kc vc qu ku vu
        dout = torch.randn(B, H, L, d, generator=g).float()
        s = d ** -0.5
        ops64 = [t.double() for t in ops]
        out, U = O.parallel_core(*ops64, s, want_U=True)
        grads = O.closed_form_grads(*ops64, s, dout.double())
        # last position as a cached step on top of the first L-1
        head = [t[..., : L - 1, :] for t in ops64]
        _, U_head = O.parallel_core(*head, s, want_U=True)
        step_out, cache = O.decode_core((U_head, head[3], head[1], head[2]), *[t[..., L - 1:, :] for t in ops64], s)
        for key, val in zip(("qc", "kc", "vc", "qu", "ku", "vu"), ops):
            blob[f"{name}_{key}"] = val.numpy()
        blob[f"{name}_dout"] = dout.numpy()
        blob[f"{name}_out"] = out.float().numpy()
        blob[f"{name}_U"] = U.float().numpy()
        blob[f"{name}_U_head"] = U_head.float().numpy()
        blob[f"{name}_step_out"] = step_out.float().numpy()
        for key, val in zip(("dqc", "dkc", "dvc", "dqu", "dku", "dvu"), grads):
            blob[f"{name}_{key}"] = val.float().numpy()
    np.savez_compressed(os.path.join(HERE, "castle_small.npz"), **blob)
    print("wrote", os.path.join(HERE, "castle_small.npz"))


if __name__ == "__main__":
    main()
