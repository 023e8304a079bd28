"""Host side of the drop-in: constructor, state_dict layout, cache type, error behaviour and
the dense (use_triton=False) formulation, all on CPU.  Mirrors the reference's CPU tests
(tests/test_lookahead.py:10-64, 145-182 of the reference)."""
import pytest
import torch

from lookahead_keys_attention_amd import Castle, Cache
from oracle import castle_oracle as O


def test_state_dict_layout_and_attributes():
    m = Castle(32, heads=2, dim_head=16, use_triton=False, prenorm=True)
    sd = m.state_dict()
    assert set(sd) == {"norm.weight", "to_all_qkv.weight", "combine_heads.weight"}
    assert sd["to_all_qkv.weight"].shape == (6 * 2 * 16, 32) and sd["combine_heads.weight"].shape == (32, 32)
    assert (m.dim, m.heads, m.dim_head, m.use_triton) == (32, 2, 16, False)
    assert m.scale == 16 ** -0.5
    assert Cache._fields == ("U", "qu_cache", "kc_cache", "vc_cache")


def test_default_init_matches_reference_construction_order():
    torch.manual_seed(7)
    m = Castle(64, heads=2, dim_head=32, use_triton=False)
    p = O.default_init(64, 2, 32, seed=7)
    assert torch.equal(m.to_all_qkv.weight, p["to_all_qkv.weight"])
    assert torch.equal(m.combine_heads.weight, p["combine_heads.weight"])


@pytest.mark.parametrize("prenorm", [False, True])
def test_dense_module_equals_oracle(prenorm):
    torch.manual_seed(0)
    m = Castle(32, heads=2, dim_head=16, use_triton=False, prenorm=prenorm)
    p = {k: v.detach() for k, v in m.state_dict().items()}
    x = torch.randn(2, 16, 32)
    y, cache = m(x, return_next_cache=True)
    yo, co = O.module_forward(x, p, 2, return_next_cache=True)
    assert torch.allclose(y, yo, atol=1e-6) and torch.allclose(cache.U, co.U, atol=1e-6)
    assert isinstance(cache, Cache) and cache.qu_cache.shape == (2, 2, 16, 16)
    xt = torch.randn(2, 1, 32)
    yt, c2 = m(xt, cache=cache)            # return_next_cache defaults to True for one token
    yto, c2o = O.module_forward(xt, p, 2, cache=co)
    assert torch.allclose(yt, yto, atol=1e-6) and torch.allclose(c2.U, c2o.U, atol=1e-6)
    assert c2.kc_cache.shape[-2] == 17


@pytest.mark.parametrize("prenorm", [False, True])
@pytest.mark.parametrize("rotary", [False, True])
def test_dense_parallel_equals_sequential(prenorm, rotary):
    torch.manual_seed(1)
    m = Castle(32, heads=2, dim_head=16, use_triton=False, prenorm=prenorm, rotary_emb=rotary).eval()
    x = torch.randn(2, 16, 32)
    with torch.no_grad():
        y0, cache = m(x[:, :8], return_next_cache=True)
        ys = [y0]
        for t in range(8, 16):
            y, cache = m(x[:, t:t + 1], cache=cache, return_next_cache=True)
            ys.append(y)
        assert torch.allclose(torch.cat(ys, 1), m(x), atol=1e-5)


@pytest.mark.parametrize("rotary", [False, True])
def test_dense_causality(rotary):
    torch.manual_seed(2)
    m = Castle(64, heads=2, dim_head=32, use_triton=False, rotary_emb=rotary).eval()
    x = torch.randn(2, 32, 64)
    with torch.no_grad():
        assert torch.allclose(m(x)[:, :16], m(x[:, :16]), atol=1e-6)


def test_error_behaviour():
    m = Castle(32, heads=2, dim_head=16, use_triton=False)
    x = torch.randn(1, 4, 32)
    _, cache = m(x, return_next_cache=True)
    with pytest.raises(AssertionError):          # lookahead_keys_attention.py:117
        m(x, cache=cache)
    native = Castle(32, heads=2, dim_head=16, use_triton=True)   # the library is built in this tree
    with pytest.raises(RuntimeError, match="GPU"):
        native(x)                                                # CPU tensor on the native path: loud failure
    assert native.use_triton is True


def test_plain_tuple_cache_is_accepted_on_dense_path():
    torch.manual_seed(3)
    m = Castle(32, heads=2, dim_head=16, use_triton=False).eval()
    x = torch.randn(1, 5, 32)
    with torch.no_grad():
        _, cache = m(x[:, :4], return_next_cache=True)
        y1, _ = m(x[:, 4:], cache=tuple(cache))
        y2, _ = m(x[:, 4:], cache=cache)
    assert torch.equal(y1, y2)


def test_rotary_state_dict_entry_matches_the_reference_module():
    # the reference holds RotaryEmbedding(dim=dim_head) as `rotary_emb` (lookahead_keys_attention.py:71-73),
    # whose only state entry is the frozen frequency vector theta^(-2i/d)
    m = Castle(32, heads=2, dim_head=16, use_triton=False, rotary_emb=True)
    sd = m.state_dict()
    assert set(sd) == {"to_all_qkv.weight", "combine_heads.weight", "rotary_emb.freqs"}
    expect = 1.0 / (10000.0 ** (torch.arange(0, 16, 2).float() / 16))
    assert torch.allclose(sd["rotary_emb.freqs"], expect, rtol=1e-6, atol=0)
    assert not m.rotary_emb.freqs.requires_grad
    other = Castle(32, heads=2, dim_head=16, use_triton=False, rotary_emb=True)
    other.load_state_dict(sd, strict=True)
    assert "rotary_emb.freqs" not in Castle(32, heads=2, dim_head=16, use_triton=False).state_dict()


def test_auto_selected_kernels_fall_back_to_dense_on_cpu_tensors(monkeypatch):
    # use_triton=None resolves like the reference (lookahead_keys_attention.py:58) and a CPU tensor
    # then takes the dense path (lookahead_keys_attention.py:120); only an explicit True insists
    monkeypatch.setattr(torch.cuda, "is_available", lambda: True)
    torch.manual_seed(4)
    auto = Castle(32, heads=2, dim_head=16)
    assert auto.use_triton is True
    dense = Castle(32, heads=2, dim_head=16, use_triton=False)
    dense.load_state_dict(auto.state_dict())
    x = torch.randn(1, 6, 32)
    with torch.no_grad():
        assert torch.equal(auto(x), dense(x))
    from lookahead_keys_attention_amd import _native
    monkeypatch.setattr(_native, "is_built", lambda: False)
    assert Castle(32, heads=2, dim_head=16).use_triton is False      # no library: not selected
    with pytest.raises(AssertionError):
        Castle(32, heads=2, dim_head=16, use_triton=True)


def test_single_token_call_is_differentiable_when_grad_is_needed():
    # lookahead_keys_attention.py:166-203 is plain differentiable PyTorch; a module whose native step
    # is inference-only must not return an output cut off from its parameters
    torch.manual_seed(5)
    m = Castle(32, heads=2, dim_head=16, use_triton=False)
    x = torch.randn(1, 3, 32)
    with torch.no_grad():
        _, cache = m(x[:, :2], return_next_cache=True)
    y, _ = m(x[:, 2:], cache=cache)
    y.sum().backward()
    assert m.to_all_qkv.weight.grad is not None and m.to_all_qkv.weight.grad.abs().sum() > 0
