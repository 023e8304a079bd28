"""`Castle`: causal attention with lookahead keys, host side of the MI355X kernels.

Same constructor, forward signature, state_dict keys and cache layout as the reference
module (lookahead_keys_attention.py:41-214), so it can replace it where the reference's
`use_triton` path is used:

    Castle(dim, heads=8, dim_head=64, use_triton=None, rotary_emb=False, prenorm=False)
    forward(x, cache=None, return_next_cache=None) -> out | (out, Cache)

`use_triton` keeps its name for drop-in compatibility and selects the native kernels:
  None  -> native HIP kernels when a GPU is present and the library is built (the reference
           resolves None the same way, lookahead_keys_attention.py:58); such a module handed CPU
           tensors uses the dense formulation, as the reference does when `not qc.is_cuda`
           (lookahead_keys_attention.py:120)
  True  -> native HIP kernels; anything that prevents them raises (missing library, CPU tensors)
  False -> the dense PyTorch formulation (the reference's own non-Triton path), any device
On the native path both the parallel pass (seq_len > 1) and the cached single-token step
run in HIP.  The native step is inference-only; a single-token call that autograd would have to
differentiate (grad mode on and the projection requires grad) takes the dense step instead, which
is differentiable like the reference's (lookahead_keys_attention.py:166-203).

Decode cache.  `Cache(U, qu_cache, kc_cache, vc_cache)` holds four (B, H, n, d) tensors as in
the reference (lookahead_keys_attention.py:26).  Caches made by the native path are views into
preallocated capacity buffers and the step updates them IN PLACE (U rows are advanced, one row
is appended); a cache handed to a native decode step is consumed by it and must not be reused.
Plain 4-tuples of tensors are accepted too (they are copied into a fresh buffer first).
"""
from __future__ import annotations

from collections import namedtuple

import warnings

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from . import _native

_CacheFields = namedtuple("Cache", ("U", "qu_cache", "kc_cache", "vc_cache"))


class Cache(_CacheFields):
    """Four (B, H, n, d) tensors; field names as in the reference (lookahead_keys_attention.py:26).

    A cache made by the native path is a set of views into its capacity buffers.  The native step
    writes the lookahead keys back on every 4th step only (the tokens in between are kept as pending
    (ku, vu) rows and applied on the fly), and a bf16 cache keeps them in a half-precision format of
    its own (`ops.LOOKAHEAD_KEYS_HALF`).  Whoever READS `U` (the attribute, index 0, unpacking) gets
    the true U in the cache's type: the pending sources are folded in first, and a buffer in the
    half-precision format is converted into a new tensor (a copy: a later step does not change it)."""

    _store = None   # set on caches that live in a native capacity buffer

    def _read(self):
        raw = tuple.__getitem__(self, slice(None))
        if self._store is None:
            return raw
        self._store.flush()
        if self._store.u_half:
            return (ops.decode_lookahead_keys(raw[0]),) + raw[1:]
        return raw

    @property
    def U(self):
        return self._read()[0]

    def __getitem__(self, index):
        return self._read()[index]

    def __iter__(self):
        return iter(self._read())


class _CacheStore:
    """Capacity buffers behind a native cache: four (B, H, capacity, d) tensors and a row count."""

    def __init__(self, B, H, d, capacity, dtype, device, U_buffer=None):
        # U_buffer: an existing (B, H, capacity, d) tensor to adopt as the lookahead-key buffer
        first = U_buffer if U_buffer is not None else torch.empty((B, H, capacity, d), dtype=dtype, device=device)
        self.buffers = (first,) + tuple(torch.empty((B, H, capacity, d), dtype=dtype, device=device) for _ in range(3))
        self.capacity = capacity
        self.length = 0
        # deferred write-back of the lookahead keys: pending (ku, vu) rows, and the row count up to
        # which every U row is known to be complete
        self.rings = (torch.empty((B, H, _native.DECODE_DEFER, d), dtype=dtype, device=device),                 # pending vu rows
                      torch.empty((B, H, capacity, _native.DECODE_DEFER), dtype=torch.float32, device=device))   # their gates per cached row
        self.base0 = 0
        self.scale = d ** -0.5
        # bf16 buffers hold the lookahead keys in the half-precision cache format (fp16 bits of U / 64)
        self.u_half = dtype == torch.bfloat16 and ops.LOOKAHEAD_KEYS_HALF
        self._geometry = (B, H, d, device)
        self._workspace = None
        self._views = None

    @property
    def workspace(self):
        """Partial-result workspace of the decode kernels, allocated when the first step needs it."""
        if self._workspace is None:
            B, H, d, device = self._geometry
            self._workspace = ops.decode_workspace(B, H, d, device)
        return self._workspace

    @property
    def views(self):
        """castle_view4 of the four buffers, built once and reused by every step on them."""
        if self._views is None:
            self._views = tuple(_native.view4(buf) for buf in self.buffers)
        return self._views

    def deferred(self, base_device=None):
        """struct castle_deferred of this store, for a step at row count `self.length` (None when the
        deferred write-back is switched off and nothing is pending: such steps write U themselves)."""
        if not ops.DEFER_LOOKAHEAD_WRITES and self.pending() == 0:
            return None
        return ops.make_deferred(self.rings[0], self.rings[1], self.base0, base_device)

    def pending(self) -> int:
        """Sources not yet folded into the stored lookahead keys."""
        t = self.length
        return t - max(self.base0, t - t % _native.DECODE_DEFER)

    def flush(self):
        """Completes the stored lookahead keys (no-op when nothing is pending)."""
        if self.pending() > 0:
            ops.castle_decode_flush(self.buffers[0], self.buffers[1], self.length, self.deferred(), self.scale,
                                    u_half=self.u_half)
        self.base0 = self.length

    def as_cache(self) -> Cache:
        n = self.length
        cache = Cache(*(buf[:, :, :n] for buf in self.buffers))
        cache._store = self
        return cache

    def grown(self, min_capacity):
        B, H, _, d = self.buffers[0].shape
        self.flush()
        new = _CacheStore(B, H, d, max(min_capacity, 2 * self.capacity), self.buffers[0].dtype, self.buffers[0].device)
        new.u_half = self.u_half   # the rows are copied as they are stored
        for dst, src in zip(new.buffers, self.buffers):
            dst[:, :, : self.length].copy_(src[:, :, : self.length])
        new.length = new.base0 = self.length
        new.scale = self.scale
        return new

    def adopt(self, cache):
        """Fills the buffers from a plain 4-tuple of (B, H, t, d) tensors."""
        t = cache[0].shape[-2]
        for buf, src in zip(self.buffers, cache):
            buf[:, :, :t].copy_(src)
        if self.u_half:
            ops.encode_lookahead_keys(cache[0], self.buffers[0][:, :, :t])
        self.length = self.base0 = t


# The weight gradient of a projection over many rows, dW = dY^T x, is a product with a small
# output (out_features x in_features) and a long contraction (the rows): the GEMM the library picks
# leaves most of the GPU idle there (one tile per output block walking all rows serially).  Above this
# row count it is formed as SPLIT_ROWS_INTO partial products over row ranges (one batched GEMM with
# fp32 partial results, then their sum): same rounding as the single product (fp32 accumulation, one
# rounding at the end), 2-3 times faster at 16384 rows.
SPLIT_WGRAD_MIN_ROWS = 8192
SPLIT_ROWS_INTO = 8


class _ManyRowLinear(torch.autograd.Function):
    """x @ weight.T (the bias-free nn.Linear of lookahead_keys_attention.py:75, 80) whose backward forms
    the weight gradient in row ranges; forward and input gradient are the library GEMMs."""

    @staticmethod
    def forward(ctx, x, weight):
        ctx.save_for_backward(x, weight)
        return F.linear(x, weight)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        dx = dw = None
        if ctx.needs_input_grad[0]:
            dx = dy @ weight
        if ctx.needs_input_grad[1]:
            x2, dy2 = x.reshape(-1, x.shape[-1]), dy.reshape(-1, dy.shape[-1])
            rows, parts = x2.shape[0], SPLIT_ROWS_INTO
            partial = torch.bmm(dy2.view(parts, rows // parts, -1).transpose(1, 2), x2.view(parts, rows // parts, -1),
                                out_dtype=torch.float32)
            dw = partial.sum(0).to(weight.dtype)
        return dx, dw


def _linear(layer, t):
    """layer(t) for a bias-free nn.Linear, through _ManyRowLinear where its weight gradient pays."""
    rows = t.numel() // t.shape[-1] if t.shape[-1] else 0
    if (t.is_cuda and layer.bias is None and t.dtype in (torch.bfloat16, torch.float16) and layer.weight.dtype == t.dtype
            and rows >= SPLIT_WGRAD_MIN_ROWS and rows % SPLIT_ROWS_INTO == 0 and t.is_contiguous()
            and torch.is_grad_enabled() and layer.weight.requires_grad):
        return _ManyRowLinear.apply(t, layer.weight)
    return layer(t)


def _reserve_rows(n: int) -> int:
    """Capacity for a cache that currently needs n rows: room for max(n/2, 1024) more steps."""
    return n + max(n // 2, 1024)


def rotate_half_pairs(t, positions, theta=10000.0):
    """Rotary position embedding over interleaved pairs (x0,x1),(x2,x3),.. of the last axis.

    t: (..., n, d); positions: (n,) absolute positions.  Frequencies theta^(-2i/d), the usual
    RoPE.  The reference delegates this to a third-party package (lookahead_keys_attention.py:73,112)
    that is not available for comparison, so exact agreement with it is unverified; the
    properties the reference tests (parallel == cached sequential, causality) hold."""
    d = t.shape[-1]
    inv = theta ** (-torch.arange(0, d, 2, device=t.device, dtype=torch.float32) / d)
    ang = positions.to(torch.float32)[:, None] * inv[None, :]
    cos, sin = ang.cos().repeat_interleave(2, -1), ang.sin().repeat_interleave(2, -1)
    x = t.float()
    pairs = x.unflatten(-1, (d // 2, 2))
    rot = torch.stack((-pairs[..., 1], pairs[..., 0]), dim=-1).flatten(-2)
    return (x * cos + rot * sin).to(t.dtype)


class RotaryFrequencies(nn.Module):
    """Holds `freqs` = theta^(-2i/d), i = 0 .. d/2 - 1, as a frozen parameter: the one entry the
    reference's third-party rotary module contributes to a state_dict (`rotary_emb.freqs`), so
    checkpoints interchange with strict loading.  It is held for that purpose only: the kernels and
    the dense path both evaluate the closed form in fp32 (a `.bfloat16()` model would otherwise
    rotate by bf16-rounded frequencies on one path and exact ones on the other)."""

    def __init__(self, dim, theta=10000.0):
        super().__init__()
        freqs = theta ** (-torch.arange(0, dim, 2, dtype=torch.float32) / dim)
        self.freqs = nn.Parameter(freqs, requires_grad=False)


class Castle(nn.Module):
    _warned_dense_step = False   # the grad-mode fallback of the cached step warns once per process

    def __init__(self, dim, heads=8, dim_head=64, use_triton=None, rotary_emb=False, prenorm=False):
        super().__init__()
        self.dim, self.heads, self.dim_head = dim, heads, dim_head
        self._explicit_native = use_triton is True
        if use_triton is None:
            use_triton = torch.cuda.is_available() and _native.is_built()
            if torch.cuda.is_available() and not use_triton:
                # the reference falls back silently when Triton is missing (lookahead_keys_attention.py:58);
                # here a GPU without the kernel library is almost certainly a build problem, so say so
                warnings.warn("libcastle_hip.so is not built: Castle(use_triton=None) uses the dense PyTorch "
                              "formulation (python -m lookahead_keys_attention_amd.build builds the kernels)",
                              RuntimeWarning, stacklevel=2)
        if use_triton and not _native.is_built():
            raise AssertionError(
                "native kernels requested but libcastle_hip.so is not built "
                "(python -m lookahead_keys_attention_amd.build), or pass use_triton=False"
            )
        self.use_triton = bool(use_triton)
        self.scale = dim_head ** -0.5
        self.norm = nn.RMSNorm(dim) if prenorm else nn.Identity()
        # same state_dict entry as the reference's RotaryEmbedding(dim=dim_head) submodule
        # (lookahead_keys_attention.py:71-73): `rotary_emb.freqs`, shape (dim_head / 2,)
        self.use_rotary = bool(rotary_emb)
        self.rotary_emb = RotaryFrequencies(dim_head) if rotary_emb else None
        inner = heads * dim_head
        self.to_all_qkv = nn.Linear(dim, inner * 6, bias=False)
        self.combine_heads = nn.Linear(inner, dim, bias=False)

    # -- helpers ------------------------------------------------------------
    def _split(self, proj):
        B, n, _ = proj.shape
        six = proj.view(B, n, 6, self.heads, self.dim_head).permute(2, 0, 3, 1, 4)
        return six.unbind(0)   # qu, ku, vu, qc, kc, vc : (B, H, n, d) views

    def _rotate(self, tensors, offset, n, device):
        pos = torch.arange(offset, offset + n, device=device)
        return tuple(rotate_half_pairs(t, pos) for t in tensors)

    # -- forward ------------------------------------------------------------
    def forward(self, x, cache=None, return_next_cache=None):
        n = x.shape[1]
        single = n == 1
        if return_next_cache is None:
            return_next_cache = single
        native = self.use_triton
        if native and not x.is_cuda:
            if self._explicit_native:
                raise RuntimeError("Castle(use_triton=True) runs HIP kernels and needs GPU tensors; "
                                   "construct with use_triton=False for the PyTorch formulation")
            native = False   # auto-selected kernels, CPU tensors: the dense formulation (lookahead_keys_attention.py:120)
        if native and not self._explicit_native and not ops.kernels_support(self.dim_head, x.dtype):
            native = False   # auto-selected kernels that do not cover this head dimension / type: dense as well
        if single and native and torch.is_grad_enabled() and (
                x.requires_grad or any(p.requires_grad for p in self.parameters())):
            # the native step records no autograd graph; the dense step does.  A native cache handed to it
            # is read out into plain tensors that grow by concatenation: O(t) copies per step from here on
            if self._explicit_native:
                raise RuntimeError("Castle(use_triton=True): the native single-token step is inference-only; call it under "
                                   "torch.no_grad() / torch.inference_mode(), or construct with use_triton=None / False "
                                   "for a differentiable (dense) step")
            if getattr(cache, "_store", None) is not None and not Castle._warned_dense_step:
                Castle._warned_dense_step = True
                warnings.warn("a single-token call with grad mode on takes the dense PyTorch step (the native step is "
                              "inference-only); its native cache is copied out and every later step stays dense. "
                              "Decode under torch.no_grad() to keep the HIP kernels", RuntimeWarning, stacklevel=2)
            native = False
        native_step = single and native
        proj = self._project(self.to_all_qkv, x, native_step, norm=self.norm)
        if not single:
            assert cache is None, "must be inferencing single tokens if receiving cache"
            merged, next_cache = (self._parallel_native if native else self._parallel_dense)(proj, return_next_cache)
        else:
            merged, next_cache = (self._step_native if native else self._step_dense)(proj, cache)
        y = self._project(self.combine_heads, merged, native_step)
        return (y, next_cache) if return_next_cache else y

    @staticmethod
    def _project(layer, t, native_step, norm=None, activation=None, residual=None):
        """A bias-free projection with what surrounds it in a block: `norm` (an nn.RMSNorm or
        nn.Identity) in front, GELU (`activation="gelu"`) and a residual behind.  On the native
        single-token step the few rows go through the library's own small-M kernel, which does all
        of it in one launch (inference only); otherwise the layers themselves run."""
        if isinstance(norm, nn.Identity):
            norm = None
        if native_step and ops.small_linear_ok(t, layer.weight) and (norm is None or isinstance(norm, nn.RMSNorm)):
            return ops.small_linear(t, layer.weight, norm=norm, activation=activation, residual=residual)
        y = _linear(layer, t if norm is None else norm(t))
        if activation == "gelu":
            y = F.gelu(y)
        return y if residual is None else residual + y

    # -- native HIP paths ---------------------------------------------------
    def _parallel_native(self, proj, want_cache):
        B, n, _ = proj.shape
        H, d = self.heads, self.dim_head
        if not want_cache:
            return ops.castle_attention_packed(proj, H, self.scale, rotary=self.use_rotary), None
        capacity = _reserve_rows(n)
        # the kernels write the lookahead keys straight into what becomes the cache's U buffer
        u_half = proj.dtype == torch.bfloat16 and ops.LOOKAHEAD_KEYS_HALF
        merged, U = ops.castle_attention_packed(proj, H, self.scale, True, capacity, rotary=self.use_rotary, u_half=u_half)
        store = _CacheStore(B, H, d, capacity, proj.dtype, proj.device, U_buffer=U._base.detach())
        store.u_half = u_half
        qu, _, _, _, kc, vc = self._split(proj)
        with torch.no_grad():
            if self.use_rotary:   # the cache holds the rotated qu / kc rows
                ops.castle_rope_hip(qu, store.buffers[1][:, :, :n])
                ops.castle_rope_hip(kc, store.buffers[2][:, :, :n])
            else:
                store.buffers[1][:, :, :n].copy_(qu)
                store.buffers[2][:, :, :n].copy_(kc)
            store.buffers[3][:, :, :n].copy_(vc)
        store.length = store.base0 = n
        store.scale = self.scale
        return merged, store.as_cache()

    def _step_native(self, proj, cache):
        B = proj.shape[0]
        H, d = self.heads, self.dim_head
        qu, ku, vu, qc, kc, vc = self._split(proj)
        store = getattr(cache, "_store", None) if cache is not None else None
        if cache is None:
            store = _CacheStore(B, H, d, _reserve_rows(1), proj.dtype, proj.device)
        elif store is None:
            store = _CacheStore(B, H, d, _reserve_rows(cache[0].shape[-2] + 1), proj.dtype, proj.device)
            store.adopt(cache)
        elif store.length != cache.kc_cache.shape[-2]:   # (not cache.U: reading it would write the pending keys back)
            raise RuntimeError("this cache was already advanced by a later decode step; the native "
                               "decode updates its cache in place, so a cache can be used once")
        store.scale = self.scale
        t = store.length
        if t + 1 > store.capacity:
            store = store.grown(_reserve_rows(t + 1))
        out = torch.empty((B, 1, H, d), dtype=proj.dtype, device=proj.device)
        deferred = store.deferred()
        if proj.is_contiguous() and proj.data_ptr() % 16 == 0:
            ops.castle_decode_step_packed(store.views, store.capacity, t, proj, H, self.scale, out, store.workspace,
                                          rotary=self.use_rotary, deferred=deferred, u_half=store.u_half)
        else:
            ops.castle_decode_step_hip(*store.buffers, t, qc, kc, vc, qu, ku, vu, self.scale,
                                       out.permute(0, 2, 1, 3), store.workspace, rotary=self.use_rotary,
                                       deferred=deferred, u_half=store.u_half)
        if deferred is None:
            store.base0 = t + 1   # this step wrote the lookahead keys itself: nothing is pending
        store.length = t + 1
        return out.view(B, 1, H * d), store.as_cache()

    def graph_step(self, x, store, t_device, base_device=None, residual=None):
        """The cached single-token step in the form a captured HIP graph needs: the same GPU work
        as forward(x, cache) on the native path, but the row count is read by the kernels from the
        one-element int32 GPU tensor `t_device`, and nothing on the host depends on it (no cache
        object is built, `store.length` is left alone: the owner of the graph keeps the count).
        `base_device` (one-element int32 GPU tensor: the row count up to which the stored lookahead
        keys are complete, e.g. the prefill length) switches the deferred write-back on.
        x: (B, 1, dim); store: the `_CacheStore` behind a native cache.  Returns (B, 1, dim), plus
        `residual` when one is given (added inside the output projection's launch)."""
        B = x.shape[0]
        proj = self._project(self.to_all_qkv, x, True, norm=self.norm)
        out = torch.empty((B, 1, self.heads, self.dim_head), dtype=proj.dtype, device=proj.device)
        ops.castle_decode_step_packed(store.views, store.capacity, 0, proj, self.heads, self.scale, out,
                                      store.workspace, rotary=self.use_rotary, t_device=t_device,
                                      deferred=store.deferred(base_device) if base_device is not None else None,
                                      u_half=store.u_half)
        return self._project(self.combine_heads, out.view(B, 1, self.heads * self.dim_head), True, residual=residual)

    # -- dense PyTorch formulation (use_triton=False) -------------------------
    def _parallel_dense(self, proj, want_cache):
        B, n, _ = proj.shape
        qu, ku, vu, qc, kc, vc = self._split(proj)
        if self.use_rotary:
            qc, kc, qu, ku, vu = self._rotate((qc, kc, qu, ku, vu), 0, n, proj.device)
        s = self.scale
        future = torch.ones(n, n, dtype=torch.bool, device=proj.device).triu(1)
        T = ((qc * s) @ vu.mT).masked_fill(future, 0.0)
        A = torch.sigmoid((qu * s) @ ku.mT).masked_fill(~future, 0.0)
        S = (qc * s) @ kc.mT - F.silu(T @ A.mT)
        P = S.masked_fill(future, -torch.finfo(S.dtype).max).softmax(dim=-1)
        o = P @ vc
        merged = o.permute(0, 2, 1, 3).reshape(B, n, -1)
        return merged, (Cache(A @ vu, qu, kc, vc) if want_cache else None)

    def _step_dense(self, proj, cache):
        B = proj.shape[0]
        qu, ku, vu, qc, kc, vc = self._split(proj)
        if cache is None:
            empty = qu[..., :0, :]
            cache = (empty,) * 4
        U, qu_hist, kc_hist, vc_hist = cache
        t = kc_hist.shape[-2]
        if self.use_rotary:
            qc, kc, qu, ku, vu = self._rotate((qc, kc, qu, ku, vu), t, 1, proj.device)
        s = self.scale
        gate = torch.sigmoid((qu_hist * s) @ ku.mT)
        U = torch.cat((U + gate * vu, torch.zeros_like(qu)), dim=-2)
        kc_all, vc_all = torch.cat((kc_hist, kc), dim=-2), torch.cat((vc_hist, vc), dim=-2)
        q = qc * s
        P = (q @ kc_all.mT - F.silu(q @ U.mT)).softmax(dim=-1)
        merged = (P @ vc_all).permute(0, 2, 1, 3).reshape(B, 1, -1)
        return merged, Cache(U, torch.cat((qu_hist, qu), dim=-2), kc_all, vc_all)
