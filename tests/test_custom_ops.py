"""The operators are registered with torch.library (torch.ops.castle_hip.*): schemas, fake (meta)
implementations and autograd formulas are exercised here without a GPU, through FakeTensorMode
(shape / stride / dtype propagation forward and backward); opcheck on real tensors is a GPU test."""
import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

from lookahead_keys_attention_amd import Castle, ops


def test_operators_are_registered_with_schemas():
    for name in ("attention", "attention_bwd", "attention_packed", "attention_packed_bwd"):
        assert hasattr(torch.ops.castle_hip, name)
    schema = str(torch.ops.castle_hip.attention.default._schema)
    assert "Tensor q" in schema and "float scale" in schema and "bool want_U" in schema
    # whether the forward keeps its state snapshots is an argument, not a global read inside the operator:
    # the fake and the real implementation cannot disagree about the size of the `state` output
    assert "bool keep_state" in schema and "bool keep_state" in str(torch.ops.castle_hip.attention_packed.default._schema)
    assert "!" not in schema and "!" not in str(torch.ops.castle_hip.attention_packed.default._schema)   # functional


def test_fake_tensor_forward_and_backward_of_the_six_operand_operator():
    # fake tensors on the CPU device: the autograd engine needs a live device of the tensors' type for
    # the backward sweep, and there is no GPU in this process; the fake implementations never look at it
    with FakeTensorMode():
        six = [torch.empty(2, 3, 100, 64, dtype=torch.bfloat16, requires_grad=True) for _ in range(6)]
        out, U = ops.castle_attention_hip(*six, 0.125, True)
        assert out.shape == (2, 3, 100, 64) and out.stride() == (100 * 3 * 64, 64, 3 * 64, 1) and out.dtype == torch.bfloat16
        assert U.shape == (2, 3, 100, 64) and out.requires_grad and not U.requires_grad
        out.sum().backward()
        assert all(t.grad is not None and t.grad.shape == t.shape for t in six)
        assert ops.castle_attention_hip(*six, 0.125).shape == (2, 3, 100, 64)
        with pytest.raises(ValueError):
            ops.castle_attention_hip(*[torch.empty(1, 1, 8, 48) for _ in range(6)], 0.1)   # head dim
        proj = torch.empty(2, 100, 6 * 3 * 64, dtype=torch.bfloat16, requires_grad=True)
        merged, U = ops.castle_attention_packed(proj, 3, 0.125, True, 150)
        assert merged.shape == (2, 100, 3 * 64) and U.shape == (2, 3, 100, 64) and U._base.shape == (2, 3, 150, 64)
        merged.sum().backward()
        assert proj.grad.shape == proj.shape
        # the state output follows the argument, in the fake implementation as in the real one
        for keep in (True, False):
            _, _, _, state = torch.ops.castle_hip.attention_packed(proj.detach(), 3, 0.125, False, 0, 0, keep)
            assert (state.numel() > 0) == keep


def test_fake_tensor_trace_of_the_module():
    """Castle.forward traces without a GPU: projection -> registered operator -> output projection,
    forward and backward, for the parallel pass with and without the cache."""
    with FakeTensorMode(), torch.device("cuda"):
        m = Castle(64, heads=2, dim_head=32, use_triton=True, prenorm=True)
        x = torch.empty(2, 40, 64, device="cuda", requires_grad=True)
        y = m(x)
        assert y.shape == (2, 40, 64) and y.requires_grad
        if torch.cuda.is_available():   # the backward sweep needs a live device of the tensors' type
            y.sum().backward()
            assert x.grad.shape == x.shape and m.to_all_qkv.weight.grad.shape == m.to_all_qkv.weight.shape
        y2, cache = m(x, return_next_cache=True)
        assert cache.U.shape == (2, 2, 40, 32) and cache.kc_cache.shape == (2, 2, 40, 32)


@pytest.mark.gpu
def test_opcheck_on_the_gpu():
    g = torch.Generator().manual_seed(0)
    six = [(torch.randn(1, 2, 96, 32, generator=g) * 0.6).to("cuda").requires_grad_() for _ in range(6)]
    torch.library.opcheck(torch.ops.castle_hip.attention.default, (*six, 32 ** -0.5, True, 0, True),
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
    proj = (torch.randn(2, 70, 6 * 2 * 32, generator=g) * 0.6).to("cuda").requires_grad_()
    torch.library.opcheck(torch.ops.castle_hip.attention_packed.default, (proj, 2, 32 ** -0.5, True, 128, 0, True),
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))


@pytest.mark.gpu
def test_compiled_module_equals_eager_on_the_gpu():
    """torch.compile traces Castle.forward as one graph through the registered operator (fake
    implementation for the shapes, autograd formula for the backward graph); the compiled forward and
    backward run the same kernels as eager mode, so the results are identical.  The `aot_eager`
    backend keeps code generation out of the test: what is checked is the tracing, not a compiler."""
    torch.manual_seed(0)
    m = Castle(64, heads=2, dim_head=32, use_triton=True, prenorm=True).to("cuda")
    x = torch.randn(2, 70, 64, device="cuda", requires_grad=True)
    y = m(x)
    y.square().sum().backward()
    want = [x.grad.clone()] + [p.grad.clone() for p in m.parameters()]
    x.grad = None
    m.zero_grad()
    compiled = torch.compile(m, backend="aot_eager", fullgraph=True)
    yc = compiled(x)
    yc.square().sum().backward()
    got = [x.grad] + [p.grad for p in m.parameters()]
    assert torch.equal(yc, y)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
