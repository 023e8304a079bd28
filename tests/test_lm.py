"""The language model around the layer and its sampler (reference: train_triton.py:56-175).

CPU tests pin the oracle's lm_forward (causality, parallel == cached, a closed-form loss) and check
the product's dense PyTorch formulation and sampling helpers against it; GPU tests compare the
native path (HIP prefill + cached decode) with the oracle.
"""
import math

import pytest
import torch

from lookahead_keys_attention_amd.lm import CastleLM, GraphedDecoder, gumbel_sample, top_k
from oracle import castle_oracle as O

VOCAB = 256


def make_lm(depth=2, dim=64, heads=2, dim_head=16, rotary=False, native=False, tie=False, seed=0):
    torch.manual_seed(seed)
    return CastleLM(num_tokens=VOCAB, dim=dim, depth=depth, heads=heads, dim_head=dim_head,
                    use_triton=native, rotary_emb=rotary, prenorm=True, tie_embedding=tie)


def params_of(model):
    return {k: v.detach().double().cpu() for k, v in model.state_dict().items()}


def tokens(B, n, seed=1):
    return torch.randint(0, VOCAB, (B, n), generator=torch.Generator().manual_seed(seed))


# ---------------------------------------------------------------- oracle pins
def test_oracle_lm_is_causal_and_cached_equals_parallel():
    model = make_lm()
    p = params_of(model)
    x = tokens(2, 12)
    full = O.lm_forward(x, p, heads=2, depth=2)
    assert full.shape == (2, 12, VOCAB)
    x2 = x.clone()
    x2[:, 8:] = (x2[:, 8:] + 7) % VOCAB
    assert torch.allclose(O.lm_forward(x2, p, 2, 2)[:, :8], full[:, :8], atol=1e-12)   # causality
    logits, cache = O.lm_forward(x[:, :5], p, 2, 2, return_next_cache=True)
    steps = [logits[:, -1]]
    for t in range(5, 12):
        logits, cache = O.lm_forward(x[:, t:t + 1], p, 2, 2, cache=cache, return_next_cache=True)
        steps.append(logits[:, -1])
    assert torch.allclose(torch.stack(steps, 1), full[:, 4:], atol=1e-10)


def test_oracle_lm_loss_is_log_vocab_for_zero_logits():
    model = make_lm()
    p = params_of(model)
    p["to_logits.weight"] = torch.zeros_like(p["to_logits.weight"])
    loss = O.lm_forward(tokens(2, 9), p, 2, 2, return_loss=True)
    assert abs(loss.item() - math.log(VOCAB)) < 1e-12


def test_oracle_lm_wiring_residuals_and_norms():
    """What a missing residual or a misplaced norm would fail.  (1) Output projections of every
    attention and feed-forward block zeroed: only the residual stream is left, so the logits are
    rms_norm(embedding) @ W.  (2) Only the feed-forward projections zeroed: the stream before the
    final norm is embedding + attention(layer 0) + attention(layer 1), each attention evaluated
    by module_forward on the running stream (pre-norm inside the layer, LKA:67,95).  (3) Only the
    attention projections zeroed: the stream is x + ff0(x) + ff1(x + ff0(x)), ff = W2 gelu(W1 rms_norm(.))."""
    F = torch.nn.functional
    model = make_lm(depth=2, rotary=True)
    p = params_of(model)
    x = tokens(2, 9)
    emb = p["token_emb.weight"][x]
    head = lambda h: F.rms_norm(h, (h.shape[-1],), p["final_norm.weight"]) @ p["to_logits.weight"].t()
    zero = lambda q, keys: {k: (torch.zeros_like(v) if k.endswith(keys) else v) for k, v in q.items()}
    both = zero(p, ("0.combine_heads.weight", "1.3.weight"))
    assert torch.allclose(O.lm_forward(x, both, 2, 2), head(emb), atol=1e-12)
    no_ff = zero(p, ("1.3.weight",))
    layer = lambda i: {k[len(f"layers.{i}.0."):]: v for k, v in p.items() if k.startswith(f"layers.{i}.0.")}
    h = emb + O.module_forward(emb, layer(0), 2)
    h = h + O.module_forward(h, layer(1), 2)
    assert torch.allclose(O.lm_forward(x, no_ff, 2, 2), head(h), atol=1e-10)
    no_attn = zero(p, ("0.combine_heads.weight",))
    ff = lambda i, h: F.gelu(F.rms_norm(h, (h.shape[-1],), p[f"layers.{i}.1.0.weight"]) @ p[f"layers.{i}.1.1.weight"].t()) @ p[f"layers.{i}.1.3.weight"].t()
    h = emb + ff(0, emb)
    h = h + ff(1, h)
    assert torch.allclose(O.lm_forward(x, no_attn, 2, 2), head(h), atol=1e-10)


def test_oracle_module_with_rotary_parallel_equals_cached_and_is_causal():
    """The reference's own properties for rotary_emb=True (tests/test_lookahead.py:10-64,145-182 of
    the reference), on the oracle: 8 parallel tokens + 8 cached steps == 16 parallel tokens; the
    first half does not see the second."""
    torch.manual_seed(3)
    dim, heads, d = 32, 2, 16
    p = O.default_init(dim, heads, d, seed=3)
    p = {k: v.double() for k, v in p.items()}
    p["rotary_emb.freqs"] = torch.zeros(d // 2)
    x = torch.randn(2, 16, dim, dtype=torch.float64)
    full = O.module_forward(x, p, heads)
    y, cache = O.module_forward(x[:, :8], p, heads, return_next_cache=True)
    outs = [y]
    for t in range(8, 16):
        y, cache = O.module_forward(x[:, t:t + 1], p, heads, cache=cache)
        outs.append(y)
    assert torch.allclose(torch.cat(outs, 1), full, atol=1e-9)
    assert torch.allclose(O.module_forward(x[:, :8], p, heads), full[:, :8], atol=1e-12)
    q = dict(p)
    del q["rotary_emb.freqs"]
    assert not torch.allclose(O.module_forward(x, q, heads), full, atol=1e-3)   # the rotation does something


# ---------------------------------------------------------------- host logic
def test_top_k_keeps_the_largest_fraction():
    logits = torch.randn(3, 50, generator=torch.Generator().manual_seed(0))
    kept = top_k(logits, thres=0.9)
    assert (kept > float("-inf")).sum(-1).tolist() == [5, 5, 5]          # ceil(0.1 * 50)
    assert torch.equal(kept.max(-1).values, logits.max(-1).values)
    assert torch.equal(kept[kept > float("-inf")].sort().values, logits.topk(5).values.flatten().sort().values)


def test_gumbel_sample_draws_from_the_softmax():
    logits = torch.tensor([1.0, 0.0, -1.0, 2.0])
    g = torch.Generator().manual_seed(0)
    draws = gumbel_sample(logits.expand(40000, 4), temperature=1.0, generator=g).flatten()
    freq = torch.bincount(draws, minlength=4).double() / draws.numel()
    assert torch.allclose(freq, logits.double().softmax(0), atol=0.01)
    cold = gumbel_sample(logits.expand(100, 4), temperature=1e-6, generator=g).flatten()
    assert torch.all(cold == 3)


@pytest.mark.parametrize("tie", [False, True])
def test_dense_model_matches_oracle(tie):
    model = make_lm(tie=tie).double()
    p = params_of(model)
    x = tokens(2, 17)
    assert torch.allclose(model(x), O.lm_forward(x, p, 2, 2), atol=1e-10)
    loss = model(x, return_loss=True)
    assert torch.allclose(loss, O.lm_forward(x, p, 2, 2, return_loss=True), atol=1e-10)
    if not tie:   # near-uniform prediction at initialisation (a tied N(0,1) embedding gives large logits)
        assert abs(loss.item() - math.log(VOCAB)) < 0.5
    assert (model.to_logits.weight is model.token_emb.weight) == tie


def test_dense_model_with_rotary_cached_equals_parallel():
    model = make_lm(rotary=True).double()
    x = tokens(2, 14)
    full = model(x)
    logits, cache = model(x[:, :6], return_next_cache=True)
    steps = [logits[:, -1]]
    for t in range(6, 14):
        logits, cache = model(x[:, t:t + 1], cache=cache, return_next_cache=True)
        steps.append(logits[:, -1])
    assert len(cache) == 2 and cache[0].kc_cache.shape[-2] == 14
    assert torch.allclose(torch.stack(steps, 1), full[:, 5:], atol=1e-9)


def test_sample_is_a_greedy_rollout_at_zero_temperature():
    model = make_lm().double()
    prompt = tokens(2, 5)
    new = model.sample(prompt, seq_len=11, temperature=0.0)
    assert new.shape == (2, 6)
    seq = prompt
    for _ in range(6):
        seq = torch.cat((seq, model(seq)[:, -1].argmax(-1, keepdim=True)), dim=-1)
    assert torch.equal(new, seq[:, 5:])
    g1, g2 = torch.Generator().manual_seed(3), torch.Generator().manual_seed(3)
    assert torch.equal(model.sample(prompt, 9, generator=g1), model.sample(prompt, 9, generator=g2))
    assert model.sample(prompt, 5).shape == (2, 0)


# ---------------------------------------------------------------- native path
@pytest.mark.gpu
def test_native_model_matches_oracle_forward_and_backward():
    model = make_lm(depth=2, dim=128, heads=2, dim_head=64, native=True).cuda()
    p = params_of(model)
    x = tokens(2, 150)
    logits = model(x.cuda())
    ref = O.lm_forward(x, p, 2, 2)
    assert (logits.cpu().double() - ref).abs().max() <= 1e-3
    loss = model(x.cuda(), return_loss=True)
    loss.backward()
    leaves = {k: v.clone().requires_grad_() for k, v in p.items()}
    ref_loss = O.lm_forward(x, leaves, 2, 2, return_loss=True)
    ref_loss.backward()
    assert abs(loss.item() - ref_loss.item()) <= 1e-4
    for name, param in model.named_parameters():
        got, want = param.grad.cpu().double(), leaves[name].grad
        assert (got - want).abs().max() <= 2e-2 * max(want.abs().max().item(), 1e-6) + 1e-6, name


@pytest.mark.gpu
@pytest.mark.parametrize("graph", [False, True])
@pytest.mark.parametrize("rotary", [False, True])
def test_native_sampler_follows_the_parallel_logits(rotary, graph):
    """Greedy generation through HIP prefill + cached decode steps across layers (step by step, or
    as replays of one captured graph): every token it picks must be (within rounding) the arg-max
    of the logits a full parallel pass assigns."""
    model = make_lm(depth=3, dim=128, heads=2, dim_head=64, rotary=rotary, native=True).cuda()
    prompt = tokens(2, 37)
    new = model.sample(prompt.cuda(), seq_len=37 + 20, temperature=0.0, graph=graph).cpu()
    assert new.shape == (2, 20)
    seq = torch.cat((prompt, new), dim=-1)
    if rotary:      # no oracle for rotary: the product's dense formulation on the CPU is the comparison
        dense = make_lm(depth=3, dim=128, heads=2, dim_head=64, rotary=True, native=False)
        dense.load_state_dict(model.state_dict())
        ref = dense.double()(seq)
    else:
        ref = O.lm_forward(seq, params_of(model), 2, 3)
    at_pick = ref[:, 36:-1].gather(-1, new.unsqueeze(-1)).squeeze(-1)
    assert torch.all(ref[:, 36:-1].max(-1).values - at_pick <= 2e-3)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_graphed_decode_replays_match_eager_steps(dtype):
    """Every replay of the captured step is compared with the eager step on a second set of caches,
    with that eager work (and a synchronisation) between the replays; afterwards both cache sets
    must hold the same rows."""
    model = make_lm(depth=3, dim=128, heads=2, dim_head=64, rotary=True, native=True).cuda().to(dtype)
    x = tokens(2, 60).cuda()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    with torch.no_grad():
        _, eager_cache = model(x[:, :20], return_next_cache=True)
        _, graph_cache = model(x[:, :20], return_next_cache=True)
        decoder = GraphedDecoder(model, graph_cache, max_len=60)
        for t in range(20, 60):
            want, eager_cache = model(x[:, t:t + 1], cache=eager_cache, return_next_cache=True)
            got = decoder.step(x[:, t:t + 1])
            torch.cuda.synchronize()
            assert (got.float() - want.float()).abs().max() <= tol * max(want.float().abs().max().item(), 1.0), t
        for layer_eager, layer_graph in zip(eager_cache, decoder.caches()):
            for a, b in zip(layer_eager, layer_graph):
                assert a.shape == b.shape
                assert (a.float() - b.float()).abs().max() <= tol * max(a.float().abs().max().item(), 1.0)
        decoder.length = decoder.capacity   # as if the caches the graph was captured for were full
        with pytest.raises(RuntimeError):
            decoder.step(x[:, :1])


@pytest.mark.gpu
def test_sampler_reuses_its_captured_graph_for_a_new_prompt():
    model = make_lm(depth=2, dim=128, heads=2, dim_head=64, rotary=True, native=True).cuda()
    first = model.sample(tokens(2, 30, seed=3).cuda(), seq_len=50, temperature=0.0, graph=True)
    kept = model._kept_decoder
    for seed, n in ((4, 30), (5, 17)):   # same graph, other prompts (also a shorter one)
        prompt = tokens(2, n, seed=seed).cuda()
        again = model.sample(prompt, seq_len=n + 20, temperature=0.0, graph=True)
        assert model._kept_decoder is kept
        eager = model.sample(prompt, seq_len=n + 20, temperature=0.0, graph=False)
        assert torch.equal(again, eager)
    assert first.shape == (2, 20)
    with torch.no_grad():   # new weights (other addresses): the kept graph must not be used again
        model.to_logits.weight = torch.nn.Parameter(model.to_logits.weight.clone())
    model.sample(tokens(2, 30, seed=3).cuda(), seq_len=50, temperature=0.0, graph=True)
    assert model._kept_decoder is not kept
    model.release_decoder()
    assert "_kept_decoder" not in model.__dict__


@pytest.mark.gpu
def test_decode_step_with_an_out_of_range_device_count_writes_nothing():
    from lookahead_keys_attention_amd import ops
    from lookahead_keys_attention_amd.castle import _CacheStore

    torch.manual_seed(0)
    B, H, d, cap = 2, 2, 64, 48
    store = _CacheStore(B, H, d, cap, torch.bfloat16, torch.device("cuda"))
    for buf in store.buffers:
        buf.copy_(torch.randn(buf.shape, device="cuda"))
    before = [buf.clone() for buf in store.buffers]
    proj = torch.randn(B, 1, 6 * H * d, device="cuda", dtype=torch.bfloat16)
    out = torch.full((B, 1, H, d), 7.0, device="cuda", dtype=torch.bfloat16)
    for count in (cap, cap + 5, -1):
        t_device = torch.tensor([count], dtype=torch.int32, device="cuda")
        ops.castle_decode_step_packed(store.views, cap, 0, proj, H, d ** -0.5, out, store.workspace, t_device=t_device)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(before, store.buffers))
    assert torch.all(out == 7.0)
    # and a count inside the range gives what the host-side count gives
    t_device = torch.tensor([17], dtype=torch.int32, device="cuda")
    other = _CacheStore(B, H, d, cap, torch.bfloat16, torch.device("cuda"))
    for dst, src in zip(other.buffers, before):
        dst.copy_(src)
    out_host = torch.empty_like(out)
    ops.castle_decode_step_packed(store.views, cap, 0, proj, H, d ** -0.5, out, store.workspace, t_device=t_device)
    ops.castle_decode_step_packed(other.views, cap, 17, proj, H, d ** -0.5, out_host, other.workspace)
    torch.cuda.synchronize()
    assert torch.equal(out, out_host)
    assert all(torch.equal(a[:, :, :18], b[:, :, :18]) for a, b in zip(store.buffers, other.buffers))


@pytest.mark.gpu
def test_config5_language_model_step_bf16():
    """benchmark configuration 5 at full size: 12 x [Castle(512, 8 heads, 64) + MLP], tied embedding,
    rotary + prenorm, (16, 1024) tokens, bf16, forward + loss + backward on the native path, against
    the oracle's lm_forward in fp32 on the same bf16-rounded weights (CPU): the full-size loss
    (forward only on the CPU: the dense autograd graph of 16 x 12 x 8 heads does not fit), then the
    loss and the gradients of the embedding and of the first and last layers' parameters for two of
    the sequences, under the bf16 rule."""
    torch.manual_seed(0)
    depth = 12
    model = CastleLM(num_tokens=VOCAB, dim=512, depth=depth, heads=8, dim_head=64, use_triton=True,
                     tie_embedding=True).cuda().bfloat16()
    x = tokens(16, 1025)
    loss = model(x.cuda(), return_loss=True)
    loss.backward()
    assert math.isfinite(loss.item())
    for name, param in model.named_parameters():
        if param.requires_grad:
            assert param.grad is not None and torch.isfinite(param.grad).all(), name
    torch.set_num_threads(16)
    weights = {k: v.detach().float().cpu() for k, v in model.state_dict().items()}
    with torch.no_grad():
        ref_loss = sum(O.lm_forward(x[b:b + 4], weights, 8, depth, return_loss=True).item() for b in range(0, 16, 4)) / 4
    assert abs(loss.item() - ref_loss) <= 2e-2 * abs(ref_loss)

    model.zero_grad()
    sub = x[:2]
    loss2 = model(sub.cuda(), return_loss=True)
    loss2.backward()
    leaves = {k: v.clone().requires_grad_(not k.endswith("freqs")) for k, v in weights.items()}
    leaves["to_logits.weight"] = leaves["token_emb.weight"]          # tied
    ref2 = O.lm_forward(sub, leaves, 8, depth, return_loss=True)
    ref2.backward()
    assert abs(loss2.item() - ref2.item()) <= 2e-2 * abs(ref2.item())
    grads = dict(model.named_parameters())
    checked = ["token_emb.weight"] + [n for n in grads if n.startswith(("layers.0.", "layers.11.")) and not n.endswith("freqs")]
    for name in checked:
        got, want = grads[name].grad.float().cpu(), leaves[name].grad
        rel = ((got - want).norm() / want.norm()).item()
        assert rel <= 2e-2, f"{name}: relative norm error {rel:.3e}"


def test_token_feed_forward_equals_the_block_on_the_cpu():
    """Off the GPU the single-token form of the feed-forward block (train_triton.py:102-107, 162)
    runs the layers themselves: h + W2 gelu(W1 norm(h)), exactly what the block plus the residual give;
    the same holds for Castle._project with a norm in front and a residual behind."""
    from lookahead_keys_attention_amd import Castle
    from lookahead_keys_attention_amd.lm import token_feed_forward

    torch.manual_seed(2)
    model = make_lm(depth=1, dim=32, heads=2, dim_head=16, rotary=False, native=False)
    _, feed_forward = model.layers[0]
    h = torch.randn(3, 1, 32)
    assert torch.allclose(token_feed_forward(feed_forward, h), h + feed_forward(h), atol=1e-6)
    got = Castle._project(model.to_logits, h, True, norm=model.final_norm)
    assert torch.allclose(got, model.to_logits(model.final_norm(h)), atol=1e-6)
    assert torch.allclose(Castle._project(feed_forward[1], h, False, norm=torch.nn.Identity(), activation="gelu", residual=None),
                          torch.nn.functional.gelu(feed_forward[1](h)), atol=1e-6)
