"""Pins oracle/castle_oracle.py without importing the reference.

Each check is chosen so that a plausible transcription mistake fails it:
brute force from the definition (mask off-by-one, wrong index order), the vu=0
case against torch's own causal SDPA (softmax / scale / causal mask), the qu=0
closed form (lookahead sum limits and the 1/2 gate), structural invariants, and
the reference's own property: parallel == cached sequential (tests/test_lookahead.py:10-64
of the reference, atol 1e-6 in fp32).
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import castle_oracle as O


def rand_heads(L, d, lead=(), seed=0, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(*lead, L, d, generator=g, dtype=dtype) for _ in range(6)]


@pytest.mark.parametrize("L,d,seed", [(1, 4, 0), (2, 4, 1), (7, 3, 2), (12, 8, 3)])
def test_parallel_matches_bruteforce_definition(L, d, seed):
    qc, kc, vc, qu, ku, vu = rand_heads(L, d, seed=seed)
    scale = d ** -0.5
    out, U = O.parallel_core(qc, kc, vc, qu, ku, vu, scale, want_U=True)
    out_bf, U_bf = O.bruteforce_core(qc, kc, vc, qu, ku, vu, scale)
    assert torch.allclose(out, out_bf, atol=1e-12)
    assert torch.allclose(U, U_bf, atol=1e-12)


def test_zero_lookahead_values_reduce_to_causal_sdpa():
    qc, kc, vc, qu, ku, vu = rand_heads(33, 16, lead=(2, 3), seed=4)
    out = O.parallel_core(qc, kc, vc, qu, ku, torch.zeros_like(vu), 16 ** -0.5)
    ref = F.scaled_dot_product_attention(qc, kc, vc, is_causal=True)
    assert torch.allclose(out, ref, atol=1e-12)


def test_zero_lookahead_queries_closed_form():
    # qu = 0 -> A = 1/2 above the diagonal -> U^i_k = (c_i - c_k)/2 with c = cumsum(vu)
    L, d = 29, 8
    qc, kc, vc, qu, ku, vu = rand_heads(L, d, seed=5)
    s = d ** -0.5
    out, U = O.parallel_core(qc, kc, vc, torch.zeros_like(qu), ku, vu, s, want_U=True)
    c = vu.cumsum(0)
    assert torch.allclose(U, 0.5 * (c[-1][None] - c), atol=1e-12)
    Su = 0.5 * torch.einsum("id,ikd->ik", qc * s, c[:, None, :] - c[None, :, :])
    S = (qc * s) @ kc.t() - F.silu(Su)
    S = S.masked_fill(torch.ones(L, L, dtype=torch.bool).triu(1), -float("inf"))
    assert torch.allclose(out, S.softmax(-1) @ vc, atol=1e-12)


def test_structural_invariants():
    qc, kc, vc, qu, ku, vu = rand_heads(17, 8, seed=6)
    s = 8 ** -0.5
    S, Su, A, T = O.parallel_scores(qc, kc, qu, ku, vu, s)
    assert torch.all(torch.diagonal(Su) == 0)            # no lookahead source in (i, i]
    assert torch.all(A.tril(0) == 0) and torch.all(T.triu(1) == 0)
    out, U = O.parallel_core(qc, kc, vc, qu, ku, vu, s, want_U=True)
    assert torch.all(U[-1] == 0)                          # last position has no lookahead
    assert torch.allclose(out[0], vc[0], atol=1e-14)      # single visible key
    # causality of the core: a change in the future leaves the past untouched
    qc2, vu2 = qc.clone(), vu.clone()
    qc2[10:] += 1.0
    vu2[10:] -= 2.0
    out2 = O.parallel_core(qc2, kc, vc, qu, ku, vu2, s)
    assert torch.allclose(out[:10], out2[:10], atol=1e-13)


@pytest.mark.parametrize("split", [0, 1, 5])
def test_decode_equals_parallel(split):
    L, d = 11, 8
    ops = rand_heads(L, d, lead=(2, 2), seed=7)
    qc, kc, vc, qu, ku, vu = ops
    s = d ** -0.5
    full, U_full = O.parallel_core(qc, kc, vc, qu, ku, vu, s, want_U=True)
    cache, outs = None, []
    if split:
        head = [t[..., :split, :] for t in ops]
        o, U = O.parallel_core(*head, s, want_U=True)
        outs.append(o)
        cache = O.OracleCache(U, head[3], head[1], head[2])
    for t in range(split, L):
        tok = [x[..., t:t + 1, :] for x in ops]
        o, cache = O.decode_core(cache, *tok, s)
        outs.append(o)
    assert torch.allclose(torch.cat(outs, dim=-2), full, atol=1e-12)
    assert torch.allclose(cache.U, U_full, atol=1e-12)
    assert torch.equal(cache.qu_cache, qu) and torch.equal(cache.kc_cache, kc)


def test_decode_first_token_closed_form():
    qc, kc, vc, qu, ku, vu = rand_heads(1, 8, lead=(2,), seed=8)
    out, cache = O.decode_core(None, qc, kc, vc, qu, ku, vu, 8 ** -0.5)
    assert torch.allclose(out, vc) and torch.all(cache.U == 0) and cache.U.shape[-2] == 1


@pytest.mark.parametrize("L,d", [(9, 4), (24, 8)])
def test_closed_form_grads_match_autograd(L, d):
    ops = [t.requires_grad_() for t in rand_heads(L, d, lead=(2,), seed=9)]
    s = d ** -0.5
    g = torch.randn(2, L, d, generator=torch.Generator().manual_seed(10), dtype=torch.float64)
    out = O.parallel_core(*ops, s)
    auto = torch.autograd.grad(out, ops, g)
    hand = O.closed_form_grads(*[t.detach() for t in ops], s, g)
    for a, h in zip(auto, hand):
        assert torch.allclose(a, h, atol=1e-11)


def test_closed_form_grads_sdpa_special_case():
    L, d = 16, 8
    qc, kc, vc, qu, ku, _ = rand_heads(L, d, lead=(1, 2), seed=11)
    g = torch.randn(1, 2, L, d, generator=torch.Generator().manual_seed(12), dtype=torch.float64)
    leaves = [t.clone().requires_grad_() for t in (qc, kc, vc)]
    ref = torch.autograd.grad(F.scaled_dot_product_attention(*leaves, is_causal=True), leaves, g)
    hand = O.closed_form_grads(qc, kc, vc, qu, ku, torch.zeros_like(qc), d ** -0.5, g)
    for r, h in zip(ref, hand[:3]):
        assert torch.allclose(r, h, atol=1e-11)


@pytest.mark.parametrize("L,d,nb", [(8, 4, 4), (24, 8, 8), (32, 16, 32), (64, 8, 16)])
def test_blockwise_state_form_equals_dense(L, d, nb):
    qc, kc, vc, qu, ku, vu = rand_heads(L, d, seed=13)
    s = d ** -0.5
    g = torch.randn(L, d, generator=torch.Generator().manual_seed(14), dtype=torch.float64)
    out, U = O.parallel_core(qc, kc, vc, qu, ku, vu, s, want_U=True)
    fw = O.blockwise_forward(qc, kc, vc, qu, ku, vu, s, nb)
    assert torch.allclose(fw["out"], out, atol=1e-11) and torch.allclose(fw["U"], U, atol=1e-11)
    bw = O.blockwise_backward(qc, kc, vc, qu, ku, vu, s, nb, g)
    dense = O.closed_form_grads(qc, kc, vc, qu, ku, vu, s, g)
    for a, b in zip(bw["grads"], dense):
        assert torch.allclose(a, b, atol=1e-10)
    # the full-length checker (no reverse-state snapshots kept) is the same computation
    out_h, U_h, grads_h = O.blockwise_head(qc, kc, vc, qu, ku, vu, s, nb, g)
    assert torch.allclose(out_h, out, atol=1e-11) and torch.allclose(U_h, U, atol=1e-11)
    for a, b in zip(grads_h, dense):
        assert torch.allclose(a, b, atol=1e-10)


# ---- module level: the reference's own CPU test properties ------------------
@pytest.mark.parametrize("prenorm", [False, True])
def test_module_parallel_equals_cached_sequential(prenorm):
    # shapes of the reference test (B2 L16 dim32 d16 H2 split8), atol 1e-6 fp32
    dim, d, H, L, split = 32, 16, 2, 16, 8
    p = O.default_init(dim, H, d, seed=0, prenorm=prenorm)
    x = torch.randn(2, L, dim, generator=torch.Generator().manual_seed(1))
    y0, cache = O.module_forward(x[:, :split], p, H, return_next_cache=True)
    ys = [y0]
    for t in range(split, L):
        y, cache = O.module_forward(x[:, t:t + 1], p, H, cache=cache, return_next_cache=True)
        ys.append(y)
    full = O.module_forward(x, p, H)
    assert torch.allclose(torch.cat(ys, 1), full, atol=1e-6)
    assert cache.U.shape == (2, H, L, d)


@pytest.mark.parametrize("prenorm", [False, True])
def test_module_causality(prenorm):
    dim, d, H, L = 64, 32, 2, 32
    p = O.default_init(dim, H, d, seed=2, prenorm=prenorm)
    x = torch.randn(2, L, dim, generator=torch.Generator().manual_seed(3))
    assert torch.allclose(O.module_forward(x, p, H)[:, :L // 2], O.module_forward(x[:, :L // 2], p, H), atol=1e-6)


def test_module_rejects_multi_token_with_cache():
    p = O.default_init(32, 2, 16, seed=0)
    x = torch.randn(1, 4, 32)
    _, cache = O.module_forward(x, p, 2, return_next_cache=True)
    with pytest.raises(AssertionError):
        O.module_forward(x, p, 2, cache=cache)


def test_readme_config_parallel_vs_sequential_fp32():
    # benchmark configuration 1: Castle(512, 8, 64), x (2,128,512) fp32, atol 1e-3
    p = O.default_init(512, 8, 64, seed=0)
    x = torch.randn(2, 128, 512, generator=torch.Generator().manual_seed(0))
    full = O.module_forward(x, p, 8)
    cache, ys = None, []
    for t in range(128):
        y, cache = O.module_forward(x[:, t:t + 1], p, 8, cache=cache)
        ys.append(y)
    assert torch.allclose(torch.cat(ys, 1), full, atol=1e-3)


def test_rope_closed_form_properties():
    """The oracle's rotary embedding against what the mathematics fixes (no formula retyped):
    identity at position 0; norm preserving; additive in the position; the dot product of two
    rotated rows depends on the position difference only; pair i at position p turns by exactly
    p * 10000^(-2i/d) radians (checked through the angle of a unit vector)."""
    g = torch.Generator().manual_seed(9)
    d, n = 16, 7
    x = torch.randn(2, n, d, generator=g, dtype=torch.float64)
    y = torch.randn(2, n, d, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 5, 9, 30, 1000])
    r = O.rope(x, pos)
    assert torch.equal(r[:, 0], x[:, 0])
    assert torch.allclose(r.norm(dim=-1), x.norm(dim=-1), atol=1e-12)
    assert torch.allclose(O.rope(O.rope(x, pos), pos + 3), O.rope(x, 2 * pos + 3), atol=1e-9)
    assert torch.allclose(O.rope(O.rope(x, pos), -pos), x, atol=1e-9)
    dots = (O.rope(x, pos + 4) * O.rope(y, pos + 1)).sum(-1)
    assert torch.allclose(dots, (O.rope(x, pos + 103) * O.rope(y, pos + 100)).sum(-1), atol=1e-8)
    e = torch.zeros(1, 1, d, dtype=torch.float64)
    e[..., 0::2] = 1.0                                   # every pair is the unit vector (1, 0)
    turned = O.rope(e, torch.tensor([3]))
    angle = torch.atan2(turned[0, 0, 1::2], turned[0, 0, 0::2])
    want = torch.tensor([math.remainder(3.0 * 10000.0 ** (-2.0 * i / d), 2 * math.pi) for i in range(d // 2)], dtype=torch.float64)
    assert torch.allclose(angle, want, atol=1e-12)
    # interleaved pairs: only elements 2i and 2i+1 mix
    one = torch.zeros(1, 1, d, dtype=torch.float64)
    one[..., 4] = 1.0
    out = O.rope(one, torch.tensor([2]))
    assert (out[0, 0].abs() > 1e-9).nonzero().flatten().tolist() == [4, 5]


def test_dense_module_rotation_equals_oracle_rope():
    from lookahead_keys_attention_amd.castle import rotate_half_pairs

    x = torch.randn(2, 3, 40, 32, generator=torch.Generator().manual_seed(4))
    pos = torch.arange(5, 45)
    assert torch.allclose(rotate_half_pairs(x, pos).double(), O.rope(x.double(), pos), atol=1e-4)
