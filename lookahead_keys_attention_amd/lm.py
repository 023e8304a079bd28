"""A small decoder-only language model around `Castle`, and its sampler.

Counterpart of the reference's training-script model (train_triton.py:73-175 `CastleLM`,
train_triton.py:56-71 sampling helpers): `depth` x [Castle attention, feed-forward], both
residual, a final RMSNorm and a logits projection.  `forward(x, return_loss, cache,
return_next_cache)` and `sample(prompt, seq_len, temperature, filter_thres)` keep the reference's
argument meaning.  With `use_triton=True` the attention layers run the HIP kernels: a prompt is
pre-filled by the parallel forward kernels, every further token by the in-place cached decode
step, one `Cache` per layer.

Differences a user can switch: `tie_embedding=True` shares the token embedding with the logits
projection (the reference keeps them separate, train_triton.py:86,111); `rotary_emb` / `prenorm`
default to the reference's choice (both on, train_triton.py:99-100).
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import nn

from . import _native
from .castle import Castle, _linear


# -- sampling helpers (train_triton.py:56-71) ------------------------------------------------
def safe_log(t: torch.Tensor, eps: float = 1e-20) -> torch.Tensor:
    return t.clamp(min=eps).log()


def gumbel_noise(t: torch.Tensor, generator: torch.Generator | None = None) -> torch.Tensor:
    u = torch.rand(t.shape, dtype=t.dtype, device=t.device, generator=generator)
    return -safe_log(-safe_log(u))


def gumbel_sample(logits, temperature=1.0, dim=-1, keepdim=True, generator=None):
    """argmax(logits / temperature + Gumbel noise): a draw from softmax(logits / temperature)."""
    return (logits / max(temperature, 1e-10) + gumbel_noise(logits, generator)).argmax(dim=dim, keepdim=keepdim)


def top_k(logits: torch.Tensor, thres: float = 0.9) -> torch.Tensor:
    """Keeps the ceil((1 - thres) * vocabulary) largest logits of each row, -inf elsewhere."""
    k = math.ceil((1.0 - thres) * logits.shape[-1])
    values, index = logits.topk(k, dim=-1)
    return torch.full_like(logits, float("-inf")).scatter_(-1, index, values)


def token_feed_forward(feed_forward: nn.Sequential, h: torch.Tensor) -> torch.Tensor:
    """h + feed_forward(h) for a single-token step (inference), the block being [norm, linear,
    GELU, linear]: two launches of the small-M linear kernel (norm and GELU ride on the first, the
    residual on the second) when it can take them (16-bit GPU tensors), the layers themselves otherwise."""
    norm, up, act, down = feed_forward
    hidden = Castle._project(up, h, True, norm=norm, activation="gelu")
    return Castle._project(down, hidden, True, residual=h)


def block_feed_forward(feed_forward: nn.Sequential, h: torch.Tensor) -> torch.Tensor:
    """feed_forward(h) for the block [norm, linear, GELU, linear] over many rows: the layers themselves,
    with the two weight gradients formed in row ranges where that pays (castle._linear)."""
    norm, up, act, down = feed_forward
    return _linear(down, act(_linear(up, norm(h))))


class GraphedDecoder:
    """One captured HIP graph of a whole single-token step of a `CastleLM` on the native path.

    A token step of a small model is a few hundred tiny launches, bound by the host; captured once
    and replayed, it costs one launch.  The cached attention step supports this through a row
    count kept in device memory (`Castle.graph_step`): the graph reads it, uses it and increments
    it, so every replay is the next step.  The graph ends at the logits; sampling stays outside.

    `caches`: the per-layer caches of a native prefill (they are consumed: the graph updates their
    buffers in place; read them back with `caches()`).  `max_len`: rows the caches must hold."""

    def __init__(self, model: "CastleLM", caches, max_len: int):
        stores = [getattr(c, "_store", None) for c in caches]
        if len(stores) != len(model.layers) or any(st is None for st in stores):
            raise RuntimeError("GraphedDecoder needs the native caches of every layer (use_triton=True on a GPU)")
        lengths = {st.length for st in stores}
        if len(lengths) != 1:
            raise RuntimeError("the layer caches disagree about their length")
        self.length = lengths.pop()
        for st in stores:
            st.flush()   # the graph starts from complete lookahead keys
        self.stores = [st if st.capacity >= max_len else st.grown(max_len) for st in stores]
        self.base0 = self.length
        self.model = model
        device = self.stores[0].buffers[0].device
        batch = self.stores[0].buffers[0].shape[0]
        self.capacity = min(st.capacity for st in self.stores)
        # while warming up and capturing, the count is out of range for every layer: such a step writes nothing
        # [row count, row count up to which the stored lookahead keys are complete]
        self.counters = torch.full((2,), max(st.capacity for st in self.stores), dtype=torch.int32, device=device)
        self.t_device, self.base_device = self.counters[:1], self.counters[1:]
        self.token = torch.zeros((batch, 1), dtype=torch.long, device=device)
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side), torch.no_grad():
            for _ in range(2):   # library handles and workspaces are created outside the capture
                self._step()
        torch.cuda.current_stream(device).wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph), torch.no_grad():
            self.logits = self._step()
            self.t_device += 1
        self._set_counters()
        self.signature = self._signature()

    def _set_counters(self):
        self.counters.copy_(torch.tensor([self.length, self.base0], dtype=torch.int32), non_blocking=False)

    def _signature(self):
        """What the captured graph has baked in: the addresses of the weights it reads."""
        return tuple(p.data_ptr() for p in self.model.parameters())

    def fits(self, caches, max_len: int) -> bool:
        """True if `load(caches)` can reuse this graph for a generation of up to max_len rows."""
        first = getattr(caches[0], "_store", None)
        mine = self.stores[0].buffers[0]
        return (first is not None and max_len <= self.capacity and self.signature == self._signature()
                and first.buffers[0].shape[:2] == mine.shape[:2] and first.buffers[0].shape[3] == mine.shape[3]
                and first.buffers[0].dtype == mine.dtype and first.buffers[0].device == mine.device
                and first.u_half == self.stores[0].u_half)

    def load(self, caches):
        """Restarts the decoder from the caches of a new prefill: their rows are copied into the
        buffers the graph was captured on (the graph holds those addresses)."""
        stores = [getattr(c, "_store", None) for c in caches]
        if len(stores) != len(self.stores) or any(st is None for st in stores):
            raise RuntimeError("GraphedDecoder.load needs the native caches of every layer")
        length = stores[0].length
        if any(st.length != length for st in stores) or length > self.capacity:
            raise RuntimeError("these caches do not fit the buffers the graph was captured on")
        for mine, theirs in zip(self.stores, stores):
            theirs.flush()
            for dst, src in zip(mine.buffers, theirs.buffers):
                dst[:, :, :length].copy_(src[:, :, :length])
        self.length = self.base0 = length
        self._set_counters()

    def _step(self):
        model = self.model
        h = model.token_emb(self.token)
        for (attention, feed_forward), store in zip(model.layers, self.stores):
            h = attention.graph_step(h, store, self.t_device, self.base_device, residual=h)
            h = token_feed_forward(feed_forward, h)
        return Castle._project(model.to_logits, h, True, norm=model.final_norm)

    def step(self, token):
        """Feeds `token` (batch, 1) and returns the logits (batch, 1, num_tokens) of the next
        position: a view of the graph's output buffer, overwritten by the next call."""
        if self.length >= self.capacity:
            raise RuntimeError(f"the graph was captured for caches of {self.capacity} rows")
        self.token.copy_(token)
        self.graph.replay()
        self.length += 1
        return self.logits

    def caches(self):
        """The per-layer caches as they stand after the steps replayed so far."""
        for st in self.stores:
            st.length, st.base0 = self.length, self.base0
            st.flush()   # the lookahead keys complete; the graph's counters must know, or a later replay would add the pending sources twice
        self.base0 = self.length
        self._set_counters()
        return [st.as_cache() for st in self.stores]


class CastleLM(nn.Module):
    def __init__(self, *, num_tokens, dim, depth, max_seq_len=512, dim_head=64, heads=8, use_triton=True,
                 rotary_emb=True, prenorm=True, tie_embedding=False):
        super().__init__()
        self.max_seq_len = max_seq_len
        self.token_emb = nn.Embedding(num_tokens, dim)
        self.layers = nn.ModuleList()
        for _ in range(depth):
            attention = Castle(dim=dim, heads=heads, dim_head=dim_head, use_triton=use_triton,
                               rotary_emb=rotary_emb, prenorm=prenorm)
            feed_forward = nn.Sequential(
                nn.RMSNorm(dim),
                nn.Linear(dim, 4 * dim, bias=False),
                nn.GELU(),
                nn.Linear(4 * dim, dim, bias=False),
            )
            self.layers.append(nn.ModuleList([attention, feed_forward]))
        self.final_norm = nn.RMSNorm(dim)
        self.to_logits = nn.Linear(dim, num_tokens, bias=False)
        if tie_embedding:
            self.to_logits.weight = self.token_emb.weight

    def forward(self, x, return_loss=False, cache=None, return_next_cache=False):
        """x: (batch, n) token ids.  With return_loss the last position is the target of the one
        before it (shift by one) and the mean cross entropy is returned; otherwise the logits
        (batch, n, num_tokens), plus the list of per-layer caches when return_next_cache."""
        if return_loss:
            x, target = x[:, :-1], x[:, 1:]
        h = self.token_emb(x)
        # one token per sequence, no graph to record: the few rows of every projection go through the small-M kernel
        # (only for a model whose layers run the native kernels: one built with use_triton=False stays on
        # the PyTorch layers throughout, so it remains an independent baseline for the native one)
        token_step = h.shape[1] == 1 and not torch.is_grad_enabled() and self._native_on_gpu(h.device)
        next_cache = []
        for index, (attention, feed_forward) in enumerate(self.layers):
            layer_cache = cache[index] if cache is not None and index < len(cache) else None
            if return_next_cache:
                attended, layer_next = attention(h, cache=layer_cache, return_next_cache=True)
                next_cache.append(layer_next)
            else:
                attended = attention(h, cache=layer_cache, return_next_cache=False)
            h = h + attended
            h = token_feed_forward(feed_forward, h) if token_step else h + block_feed_forward(feed_forward, h)
        logits = Castle._project(self.to_logits, h, token_step, norm=self.final_norm)
        if return_loss:
            return F.cross_entropy(logits.transpose(1, 2), target)
        return (logits, next_cache) if return_next_cache else logits

    def _decoder_for(self, cache, max_len):
        """A GraphedDecoder positioned on `cache`: the one kept from an earlier call when its graph
        still fits (same weights, batch, type; enough rows), else a newly captured one."""
        kept = self.__dict__.get("_kept_decoder")
        if kept is not None and kept.fits(cache, max_len):
            kept.load(cache)
            return kept
        decoder = GraphedDecoder(self, cache, max_len)
        self.__dict__["_kept_decoder"] = decoder   # not a module attribute: never part of the state
        return decoder

    def release_decoder(self):
        """Drops the graph (and the cache buffers it was captured on) kept from the last `sample` call."""
        self.__dict__.pop("_kept_decoder", None)

    def _native_on_gpu(self, device) -> bool:
        return device.type == "cuda" and _native.is_built() and all(attention.use_triton for attention, _ in self.layers)

    @torch.no_grad()
    def sample(self, prompt, seq_len, temperature=1.0, filter_thres=0.9, generator=None, graph=None):
        """Extends `prompt` (batch, p) to `seq_len` tokens and returns the seq_len - p new ones.
        The prompt goes through the parallel path once; afterwards each step feeds the last token
        and the per-layer caches.  temperature = 0 picks the arg-max (no noise).
        graph: replay the token steps as one captured HIP graph (`GraphedDecoder`).  None = when
        the model runs the native kernels on a GPU and more than a few steps follow; True insists."""
        prompt_len = prompt.shape[-1]
        steps = max(0, seq_len - prompt_len)
        if graph is None:
            graph = self._native_on_gpu(prompt.device) and steps > 8
        elif graph and not self._native_on_gpu(prompt.device):
            raise RuntimeError("graph=True needs the native kernels on a GPU")

        def pick(logits):
            logits = top_k(logits[:, -1].float(), thres=filter_thres)
            if temperature == 0:
                return logits.argmax(dim=-1, keepdim=True)
            return gumbel_sample(logits, temperature=temperature, generator=generator)

        out, cache, decoder = prompt, None, None
        for _ in range(steps):
            if decoder is not None:
                logits = decoder.step(out[:, -1:])
            else:
                step_input = out if cache is None else out[:, -1:]
                logits, cache = self.forward(step_input, cache=cache, return_next_cache=True)
                if graph:
                    decoder = self._decoder_for(cache, seq_len)
            out = torch.cat((out, pick(logits)), dim=-1)
        return out[..., prompt_len:]
