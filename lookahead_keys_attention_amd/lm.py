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

from .castle import Castle


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
        next_cache = []
        for index, (attention, feed_forward) in enumerate(self.layers):
            layer_cache = cache[index] if cache is not None and index < len(cache) else None
            if return_next_cache:
                attended, layer_next = attention(h, cache=layer_cache, return_next_cache=True)
                next_cache.append(layer_next)
            else:
                attended = attention(h, cache=layer_cache, return_next_cache=False)
            h = h + attended
            h = h + feed_forward(h)
        logits = self.to_logits(self.final_norm(h))
        if return_loss:
            return F.cross_entropy(logits.transpose(1, 2), target)
        return (logits, next_cache) if return_next_cache else logits

    @torch.no_grad()
    def sample(self, prompt, seq_len, temperature=1.0, filter_thres=0.9, generator=None):
        """Extends `prompt` (batch, p) to `seq_len` tokens and returns the seq_len - p new ones.
        The prompt goes through the parallel path once; afterwards each step feeds the last token
        and the per-layer caches.  temperature = 0 picks the arg-max (no noise)."""
        prompt_len = prompt.shape[-1]
        out, cache = prompt, None
        for _ in range(max(0, seq_len - prompt_len)):
            step_input = out if cache is None else out[:, -1:]
            logits, cache = self.forward(step_input, cache=cache, return_next_cache=True)
            logits = top_k(logits[:, -1].float(), thres=filter_thres)
            if temperature == 0:
                token = logits.argmax(dim=-1, keepdim=True)
            else:
                token = gumbel_sample(logits, temperature=temperature, generator=generator)
            out = torch.cat((out, token), dim=-1)
        return out[..., prompt_len:]
