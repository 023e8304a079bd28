"""Golden vectors (tests/golden/castle_small.npz, written by tests/golden/make_golden.py).

CPU: the oracle must reproduce them.  GPU: the HIP path, called through the C ABI, must
match them: fp32 within atol 1e-3 for outputs (north-star tolerance) and 2e-2 for
gradients (the reference's own bound, tests/test_lookahead.py:135,143)."""
import os

import numpy as np
import pytest
import torch

from oracle import castle_oracle as O

PATH = os.path.join(os.path.dirname(__file__), "golden", "castle_small.npz")
CASES = ("a", "b", "c")
OPS = ("qc", "kc", "vc", "qu", "ku", "vu")
GRADS = ("dqc", "dkc", "dvc", "dqu", "dku", "dvu")


def load(case):
    z = np.load(PATH)
    return {k[len(case) + 1:]: torch.from_numpy(z[k]) for k in z.files if k.startswith(case + "_")}


@pytest.mark.parametrize("case", CASES)
def test_oracle_reproduces_golden(case):
    v = load(case)
    ops = [v[k].double() for k in OPS]
    s = ops[0].shape[-1] ** -0.5
    out, U = O.parallel_core(*ops, s, want_U=True)
    assert torch.allclose(out.float(), v["out"], atol=1e-6) and torch.allclose(U.float(), v["U"], atol=1e-5)
    for g, name in zip(O.closed_form_grads(*ops, s, v["dout"].double()), GRADS):
        assert torch.allclose(g.float(), v[name], atol=1e-6), name
    L = ops[0].shape[-2]
    head = [t[..., : L - 1, :] for t in ops]
    step, cache = O.decode_core((v["U_head"].double(), head[3], head[1], head[2]), *[t[..., L - 1:, :] for t in ops], s)
    assert torch.allclose(step.float(), v["step_out"], atol=1e-6)
    assert torch.allclose(step.float(), v["out"][..., L - 1:, :], atol=1e-6)       # decode == parallel
    assert torch.allclose(cache.U.float(), v["U"], atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES)
def test_hip_matches_golden_fp32(case):
    from lookahead_keys_attention_amd import ops as H

    v = load(case)
    dev = torch.device("cuda:0")
    leaves = [v[k].to(dev).requires_grad_() for k in OPS]
    s = leaves[0].shape[-1] ** -0.5
    out, U = H.castle_attention_hip(*leaves, s, True)
    out.backward(v["dout"].to(dev))
    assert (out.detach().cpu() - v["out"]).abs().max() <= 1e-3
    assert (U.cpu() - v["U"]).abs().max() <= 1e-3
    for leaf, name in zip(leaves, GRADS):
        assert (leaf.grad.cpu() - v[name]).abs().max() <= 2e-2, name
    # last position as a cached step over capacity buffers
    B, Hh, L, d = v["qc"].shape
    bufs = [torch.zeros(B, Hh, L + 2, d, device=dev) for _ in range(4)]
    for buf, src in zip(bufs, (v["U_head"], v["qu"][..., : L - 1, :], v["kc"][..., : L - 1, :], v["vc"][..., : L - 1, :])):
        buf[:, :, : L - 1] = src.to(dev)
    tok = [v[k][..., L - 1:, :].to(dev) for k in OPS]
    step = torch.empty(B, Hh, 1, d, device=dev)
    H.castle_decode_step_hip(*bufs, L - 1, *tok, s, step, H.decode_workspace(B, Hh, d, dev))
    assert (step.cpu() - v["step_out"]).abs().max() <= 1e-3
    assert (bufs[0][:, :, :L].cpu() - v["U"]).abs().max() <= 1e-3
