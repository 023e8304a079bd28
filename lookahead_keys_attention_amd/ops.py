"""Operators over the HIP kernels.

`castle_attention_hip` has the call contract of the reference's Triton operator
(castle_attention_triton, lookahead_keys_attention_triton.py:605 / :417-602): six unscaled
(B, H, L, d) tensors, a scale, a flag asking for the lookahead keys U of the decode cache;
it is differentiable in the six tensors and U carries no gradient.

`castle_attention_packed` is the same operator fed straight from the module's fused
projection (B, L, 6*H*d) in the order qu, ku, vu, qc, kc, vc (lookahead_keys_attention.py:77,104):
the kernels read the six operands through strides, write the output already merged as
(B, L, H*d) and return one packed gradient, so no operand is ever copied or re-laid-out.

`castle_decode_step_hip` is the cached single-token step (lookahead_keys_attention.py:166-203)
over preallocated capacity buffers, updated in place.

The parallel operators are registered with torch.library (torch.ops.castle_hip.attention,
.attention_packed and their backward passes) with fake implementations and autograd formulas, so
they trace under FakeTensorMode / torch.compile; the functions above are thin callers of them.
"""
from __future__ import annotations

import torch

from . import _native as N


# flags handed to castle_fwd / castle_bwd (0, or _native.FLAG_BF16_OPERANDS); read when the
# forward runs and remembered for its backward.  The `rotary` arguments below add FLAG_ROTARY.
DEFAULT_FLAGS = 0
# A forward call keeps its state snapshots (B*H*L^2*d/128 elements) for its backward pass when they
# take at most this many bytes; beyond it they are dropped after the forward pass and the backward
# pass runs the scan again first (what a call keeps is then O(L d)).  0 = never keep.
KEEP_STATE_LIMIT_BYTES = 8 << 30
# The native cached step writes the lookahead keys back on every 4th step only (pending tokens are
# applied on the fly; see castle_deferred in include/castle_hip.h).  False: every step writes U.
DEFER_LOOKAHEAD_WRITES = True
# bf16 decode caches made by the module keep their lookahead keys in the half-precision cache format
# (fp16 bits of U / 64 in the same buffer: CASTLE_FLAG_U_HALF in include/castle_hip.h), which takes the
# rounding noise of a long decode down by a factor of 8.  False: the buffer holds plain bf16.
LOOKAHEAD_KEYS_HALF = True
# Debugging aid: when True every parallel forward waits for its kernels and raises if they had to
# clamp a value to the fp16 range (an input element of a bf16 tensor beyond +-65504, or a T' entry):
# the result is then that of the clamped operands.  Off by default because it synchronises.
CHECK_RANGE = False


def _require_gpu(t: torch.Tensor, what: str):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: the HIP kernels need tensors on the GPU (got {t.device})")


def kernels_support(d: int, dtype: torch.dtype) -> bool:
    """True if the HIP kernels cover this head dimension and tensor type."""
    if d not in N.SUPPORTED_HEAD_DIMS or dtype not in (torch.float32, torch.bfloat16, torch.float16):
        return False
    return not (dtype == torch.float32 and d > 64)


def _check_dims(d: int, dtype: torch.dtype):
    if d not in N.SUPPORTED_HEAD_DIMS:
        raise ValueError(f"dim_head must be one of {N.SUPPORTED_HEAD_DIMS} for the HIP kernels, got {d}")
    if dtype == torch.float32 and d > 64:
        raise ValueError("float32 HIP kernels support dim_head <= 64")


def _fwd_raw(qc, kc, vc, qu, ku, vu, scale, out, U, flags=0, keep_state=True):
    """Launch castle_fwd; returns (workspace, state): the tensors the backward pass needs back.
    `state` is an empty tensor when the caller does not keep the snapshots (`keep_state` False)."""
    B, H, L, d = qc.shape
    code = N.dtype_code(qc.dtype)
    lib = N.lib()
    nbytes = N.check(lib.castle_fwd_workspace_bytes(B, H, L, d, code), "castle_fwd_workspace_bytes")
    sbytes = N.check(lib.castle_fwd_state_bytes(B, H, L, d, code), "castle_fwd_state_bytes")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=qc.device)
    state = torch.empty(sbytes, dtype=torch.uint8, device=qc.device)
    views = [N.view4(t) for t in (qc, kc, vc, qu, ku, vu)]
    vo = N.view4(out)
    vU = N.view4(U) if U is not None else N.View4(None, 0, 0, 0)
    with torch.cuda.device(qc.device):
        rc = lib.castle_fwd(*views, B, H, L, d, code, float(scale), int(flags), vo, vU, ws.data_ptr(), nbytes,
                            state.data_ptr(), sbytes, N.stream_ptr(qc.device))
    N.check(rc, "castle_fwd")
    if not keep_state:
        state = torch.empty(0, dtype=torch.uint8, device=qc.device)   # the caching allocator keeps the block until the stream is done with it
    if CHECK_RANGE:
        status = range_status(ws)
        if status:
            raise RuntimeError(f"castle_fwd clamped values to the fp16 range (status bits {status:#x}: "
                               "1 = input element, 2 = T' = s qc.vu entry)")
    return ws, state


def range_status(ws: torch.Tensor) -> int:
    """Status word the forward kernels leave at the start of their workspace (synchronises):
    bit 0 = an input element was clamped to +-65504, bit 1 = an entry of T' = s qc.vu was."""
    return int(ws[:4].view(torch.int32).item())


def _bwd_raw(qc, kc, vc, qu, ku, vu, out, dout, scale, grads, ws, state, flags=0):
    B, H, L, d = qc.shape
    code = N.dtype_code(qc.dtype)
    lib = N.lib()
    flags &= ~N.FLAG_U_HALF   # describes the forward's U output only
    if state.numel() == 0:
        flags |= N.FLAG_RECOMPUTE_STATE
    nbytes = N.check(lib.castle_bwd_workspace_bytes(B, H, L, d, code, int(flags)), "castle_bwd_workspace_bytes")
    bws = torch.empty(nbytes, dtype=torch.uint8, device=qc.device)
    views = [N.view4(t) for t in (qc, kc, vc, qu, ku, vu, out, dout)]
    gviews = [N.view4(t) for t in grads]
    with torch.cuda.device(qc.device):
        rc = lib.castle_bwd(*views, B, H, L, d, code, float(scale), int(flags), *gviews,
                            ws.data_ptr(), ws.numel(), state.data_ptr() if state.numel() else None, state.numel(),
                            bws.data_ptr(), nbytes, N.stream_ptr(qc.device))
    N.check(rc, "castle_bwd")


def _as_readable(t: torch.Tensor) -> torch.Tensor:
    return t if N.vector_ok(t) else t.contiguous()


# ---------------------------------------------------------------------------------------------
# Registered operators (torch.library): the kernels are reachable as torch.ops.castle_hip.*, with
# fake (meta) implementations for shape propagation / tracing and autograd formulas that call the
# backward entry point.  The Python functions below them are what callers use.
#
#   castle_hip::attention         six (B,H,L,d) operands -> (out, U, workspace)
#   castle_hip::attention_packed  (B,L,6*H*d) projection -> (merged out, workspace); U written into
#                                 the optional (B,H,L,d) view `U_out` (a cache buffer)
#   castle_hip::attention_bwd / attention_packed_bwd   their backward passes
# `U` is an empty tensor when the lookahead keys are not asked for.  The workspace output is what
# the backward pass needs back (operand copies, snapshots, log-sum-exp); it carries no gradient.
def _out_like(q):
    B, H, L, d = q.shape
    return torch.empty((B, L, H, d), dtype=q.dtype, device=q.device).permute(0, 2, 1, 3)


def _state_bytes(B, H, L, d, dtype):
    return N.check(N.lib().castle_fwd_state_bytes(int(B), int(H), int(L), int(d), N.dtype_code(dtype)), "castle_fwd_state_bytes")


def _fake_state(B, H, L, d, like, keep_state):
    return torch.empty(_state_bytes(B, H, L, d, like.dtype) if keep_state else 0, dtype=torch.uint8, device=like.device)


def state_bytes_formula(B, H, L, d, element_size) -> int:
    """castle_fwd_state_bytes in plain Python (64-row blocks over L rounded up to 128; one snapshot row
    of d elements per key and later block), for callers that a tracing compiler looks into."""
    nblk = (L + 127) // 128 * 2
    n = B * H * 64 * (nblk * (nblk - 1) // 2) * d * element_size
    return max(256, (n + 255) // 256 * 256)


def keeps_state(B, H, L, d, dtype) -> bool:
    """The decision KEEP_STATE_LIMIT_BYTES stands for, taken once per call by the Python callers and
    handed to the registered operators as an argument (so a traced graph and its execution agree)."""
    return state_bytes_formula(B, H, L, d, dtype.itemsize) <= KEEP_STATE_LIMIT_BYTES


def _fwd_ws_bytes(B, H, L, d, dtype):
    return N.check(N.lib().castle_fwd_workspace_bytes(int(B), int(H), int(L), int(d), N.dtype_code(dtype)),
                   "castle_fwd_workspace_bytes")


@torch.library.custom_op("castle_hip::attention", mutates_args=())
def _attention_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, qu: torch.Tensor, ku: torch.Tensor,
                  vu: torch.Tensor, scale: float, want_U: bool, flags: int,
                  keep_state: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    _require_gpu(q, "castle_attention_hip")
    B, H, L, d = q.shape
    _check_dims(d, q.dtype)
    ops = [_as_readable(t) for t in (q, k, v, qu, ku, vu)]
    out = _out_like(q)
    U = torch.empty((B, H, L, d) if want_U else (0,), dtype=q.dtype, device=q.device)
    ws, state = _fwd_raw(*ops, scale, out, U if want_U else None, flags, keep_state)
    return out, U, ws, state


@_attention_op.register_fake
def _(q, k, v, qu, ku, vu, scale, want_U, flags, keep_state):
    B, H, L, d = q.shape
    _check_dims(d, q.dtype)
    U = torch.empty((B, H, L, d) if want_U else (0,), dtype=q.dtype, device=q.device)
    ws = torch.empty(_fwd_ws_bytes(B, H, L, d, q.dtype), dtype=torch.uint8, device=q.device)
    return _out_like(q), U, ws, _fake_state(B, H, L, d, q, keep_state)


@torch.library.custom_op("castle_hip::attention_bwd", mutates_args=())
def _attention_bwd_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, qu: torch.Tensor, ku: torch.Tensor,
                      vu: torch.Tensor, out: torch.Tensor, dout: torch.Tensor, ws: torch.Tensor, state: torch.Tensor,
                      scale: float, flags: int) -> torch.Tensor:
    B, H, L, d = q.shape
    ops = [_as_readable(t) for t in (q, k, v, qu, ku, vu)]
    packed = torch.empty((6, B, H, L, d), dtype=out.dtype, device=out.device)
    _bwd_raw(*ops, _as_readable(out), _as_readable(dout), scale, list(packed.unbind(0)), ws, state, flags)
    return packed


@_attention_bwd_op.register_fake
def _(q, k, v, qu, ku, vu, out, dout, ws, state, scale, flags):
    return torch.empty((6, *q.shape), dtype=out.dtype, device=out.device)


def _attention_setup(ctx, inputs, output):
    q, k, v, qu, ku, vu, scale, want_U, flags, keep_state = inputs
    out, U, ws, state = output
    ctx.save_for_backward(q, k, v, qu, ku, vu, out, ws, state)
    ctx.scale, ctx.flags = scale, flags
    ctx.mark_non_differentiable(U, ws, state)   # U carries no gradient (lookahead_keys_attention_triton.py:513-515)
    # without this autograd hands the backward formula zero tensors for the unused outputs: a fill of
    # the whole workspace and state buffers (hundreds of MB) on every backward pass
    ctx.set_materialize_grads(False)


def _attention_backward(ctx, dout, dU, dws, dstate):
    q, k, v, qu, ku, vu, out, ws, state = ctx.saved_tensors
    if dout is None:
        dout = torch.zeros_like(out)
    grads = torch.ops.castle_hip.attention_bwd(q, k, v, qu, ku, vu, out, dout, ws, state, ctx.scale, ctx.flags)
    return (*grads.unbind(0), None, None, None, None)


_attention_op.register_autograd(_attention_backward, setup_context=_attention_setup)


def _six_views(proj, heads):
    B, L, width = proj.shape
    d = width // (6 * heads)
    six = proj.view(B, L, 6, heads, d).permute(2, 0, 3, 1, 4)      # (6, B, H, L, d) views
    return six.unbind(0)                                            # qu, ku, vu, qc, kc, vc


def _packed_ok(t):
    return t if (t.is_contiguous() and t.data_ptr() % 16 == 0) else t.contiguous()


@torch.library.custom_op("castle_hip::attention_packed", mutates_args=())
def _attention_packed_op(proj: torch.Tensor, heads: int, scale: float, want_U: bool, row_capacity: int,
                         flags: int, keep_state: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    # The lookahead keys come back as the first L rows of a (B, H, row_capacity, d) buffer, so that a
    # caller can hand over the U buffer of a decode cache without copying (row_capacity >= L).
    _require_gpu(proj, "castle_attention_packed")
    B, L, width = proj.shape
    d = width // (6 * heads)
    _check_dims(d, proj.dtype)
    qu, ku, vu, qc, kc, vc = _six_views(_packed_ok(proj), heads)
    merged = torch.empty((B, L, heads * d), dtype=proj.dtype, device=proj.device)
    out = merged.view(B, L, heads, d).permute(0, 2, 1, 3)
    U = torch.empty((B, heads, max(row_capacity, L), d) if want_U else (0,), dtype=proj.dtype, device=proj.device)
    ws, state = _fwd_raw(qc, kc, vc, qu, ku, vu, scale, out, U[:, :, :L] if want_U else None, flags, keep_state)
    return merged, U, ws, state


@_attention_packed_op.register_fake
def _(proj, heads, scale, want_U, row_capacity, flags, keep_state):
    B, L, width = proj.shape
    d = width // (6 * heads)
    _check_dims(d, proj.dtype)
    ws = torch.empty(_fwd_ws_bytes(B, heads, L, d, proj.dtype), dtype=torch.uint8, device=proj.device)
    U = torch.empty((B, heads, max(row_capacity, L), d) if want_U else (0,), dtype=proj.dtype, device=proj.device)
    return torch.empty((B, L, heads * d), dtype=proj.dtype, device=proj.device), U, ws, _fake_state(B, heads, L, d, proj, keep_state)


@torch.library.custom_op("castle_hip::attention_packed_bwd", mutates_args=())
def _attention_packed_bwd_op(proj: torch.Tensor, merged: torch.Tensor, dmerged: torch.Tensor, ws: torch.Tensor,
                             state: torch.Tensor, heads: int, scale: float, flags: int) -> torch.Tensor:
    B, L, width = proj.shape
    d = width // (6 * heads)
    qu, ku, vu, qc, kc, vc = _six_views(_packed_ok(proj), heads)
    out = merged.view(B, L, heads, d).permute(0, 2, 1, 3)
    dout = _packed_ok(dmerged).view(B, L, heads, d).permute(0, 2, 1, 3)
    dproj = torch.empty((B, L, width), dtype=proj.dtype, device=proj.device)
    dqu, dku, dvu, dqc, dkc, dvc = _six_views(dproj, heads)
    _bwd_raw(qc, kc, vc, qu, ku, vu, out, dout, scale, (dqc, dkc, dvc, dqu, dku, dvu), ws, state, flags)
    return dproj


@_attention_packed_bwd_op.register_fake
def _(proj, merged, dmerged, ws, state, heads, scale, flags):
    return torch.empty(proj.shape, dtype=proj.dtype, device=proj.device)


def _packed_setup(ctx, inputs, output):
    proj, heads, scale, want_U, row_capacity, flags, keep_state = inputs
    merged, U, ws, state = output
    ctx.save_for_backward(proj, merged, ws, state)
    ctx.heads, ctx.scale, ctx.flags = heads, scale, flags
    ctx.mark_non_differentiable(U, ws, state)
    ctx.set_materialize_grads(False)   # see _attention_setup


def _packed_backward(ctx, dmerged, dU, dws, dstate):
    proj, merged, ws, state = ctx.saved_tensors
    if dmerged is None:
        dmerged = torch.zeros_like(merged)
    dproj = torch.ops.castle_hip.attention_packed_bwd(proj, merged, dmerged, ws, state, ctx.heads, ctx.scale, ctx.flags)
    return dproj, None, None, None, None, None, None


_attention_packed_op.register_autograd(_packed_backward, setup_context=_packed_setup)


def castle_attention_hip(q, k, v, qu, ku, vu, scale, return_U_for_cache=False, rotary=False):
    """Drop-in for castle_attention_triton: returns out, or (out, U).  rotary=True applies the
    rotary position embedding (positions 0..L-1) to q, k, qu, ku, vu inside the kernels."""
    flags = DEFAULT_FLAGS | (N.FLAG_ROTARY if rotary else 0)
    B, H, L, d = q.shape
    _check_dims(d, q.dtype)
    out, U, _, _ = torch.ops.castle_hip.attention(q, k, v, qu, ku, vu, float(scale), bool(return_U_for_cache), int(flags),
                                                  keeps_state(B, H, L, d, q.dtype))
    return (out, U) if return_U_for_cache else out


def castle_attention_packed(proj, heads, scale, return_U_for_cache=False, row_capacity=0, rotary=False, u_half=False):
    """proj (B, L, 6*H*d) -> merged out (B, L, H*d), or (out, U).  U is (B,H,L,d); with
    `row_capacity` > L it is the first L rows of a freshly allocated (B,H,row_capacity,d) buffer
    (reachable as U._base), which a decode cache can adopt as its U buffer without a copy.
    `u_half` (bf16 only): U comes back in the half-precision cache format (`decode_lookahead_keys`
    reads it), the format the cached step then keeps it in."""
    flags = DEFAULT_FLAGS | (N.FLAG_ROTARY if rotary else 0) | (N.FLAG_U_HALF if u_half and return_U_for_cache else 0)
    B, L, width = proj.shape
    _check_dims(width // (6 * int(heads)), proj.dtype)
    merged, U, _, _ = torch.ops.castle_hip.attention_packed(proj, int(heads), float(scale), bool(return_U_for_cache),
                                                         int(row_capacity), int(flags),
                                                         keeps_state(B, int(heads), L, width // (6 * int(heads)), proj.dtype))
    return (merged, U[:, :, : proj.shape[1]]) if return_U_for_cache else merged


def decode_lookahead_keys(raw: torch.Tensor) -> torch.Tensor:
    """A bf16-typed buffer in the half-precision cache format -> the lookahead keys as a new bf16 tensor."""
    return (raw.view(torch.float16).to(torch.float32) * N.U_HALF_UNSCALE).to(raw.dtype)


def encode_lookahead_keys(U: torch.Tensor, out: torch.Tensor):
    """Writes lookahead keys into `out` (same shape, bf16-typed) in the half-precision cache format."""
    out.view(torch.float16).copy_((U.to(torch.float32) / N.U_HALF_UNSCALE).clamp_(-65504.0, 65504.0))


def decode_workspace(B, H, d, device):
    nbytes = N.check(N.lib().castle_decode_workspace_bytes(B, H, d, 0), "castle_decode_workspace_bytes")
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


@torch.no_grad()
def castle_decode_step_hip(U, qu_cache, kc_cache, vc_cache, t, qc, kc, vc, qu, ku, vu, scale, out, workspace,
                           rotary=False, deferred=None, u_half=False):
    """In-place cached step.  The four cache tensors are (B,H,capacity,d) buffers with t valid
    rows (capacity > t); the new-token operands and `out` are (B,H,1,d).  rotary=True rotates the
    new token by position t inside the kernels (the cache rows are stored rotated).  `deferred`: a
    `_native.Deferred` (pending-token buffers and a base row count, `make_deferred`) makes the kernels write the
    lookahead keys on every 4th step only; `castle_decode_flush` completes them in between.
    `u_half` (bf16 only): the U buffer is in the half-precision cache format."""
    _require_gpu(U, "castle_decode_step_hip")
    B, H, cap, d = U.shape
    if not (0 <= t < cap):
        raise ValueError(f"cache capacity {cap} cannot take row {t}")
    if d not in N.SUPPORTED_HEAD_DIMS:
        raise ValueError(f"dim_head must be one of {N.SUPPORTED_HEAD_DIMS} for the HIP kernels, got {d}")
    code = N.dtype_code(U.dtype)
    toks = [_as_readable(x) for x in (qc, kc, vc, qu, ku, vu)]
    views = [N.view4(x) for x in (U, qu_cache, kc_cache, vc_cache)]
    tviews = [N.view4(x) for x in toks]
    with torch.cuda.device(U.device):
        rc = N.lib().castle_decode_step(*views, int(t), int(cap), *tviews, B, H, d, code, float(scale),
                                        (N.FLAG_ROTARY if rotary else 0) | (N.FLAG_U_HALF if u_half else 0), N.view4(out), deferred,
                                        workspace.data_ptr(), workspace.numel(), N.stream_ptr(U.device))
    N.check(rc, "castle_decode_step")
    return out


def make_deferred(vu_ring, gates, base, base_device=None):
    """struct castle_deferred: `vu_ring` (B, H, 4, d) in the cache's element type, `gates`
    (B, H, capacity, 4) fp32 contiguous; `base_device`: optional int32 GPU tensor whose first
    element the kernels read instead of `base` (graph replay)."""
    assert gates.dtype == torch.float32 and gates.is_contiguous() and gates.shape[-1] == N.DECODE_DEFER
    return N.Deferred(N.view4(vu_ring), N.view4(gates), int(base), base_device.data_ptr() if base_device is not None else None)


@torch.no_grad()
def castle_decode_flush(U, qu_cache, t, deferred, scale, u_half=False):
    """Folds the pending sources into the stored lookahead keys U[:, :, :t] (see castle_deferred).  The
    caller then sets the base row count of its castle_deferred (host and device copy) to t."""
    B, H, _, d = U.shape
    with torch.cuda.device(U.device):
        rc = N.lib().castle_decode_flush(N.view4(U), N.view4(qu_cache), int(t), deferred, B, H, d, N.dtype_code(U.dtype),
                                         float(scale), N.FLAG_U_HALF if u_half else 0, N.stream_ptr(U.device))
    N.check(rc, "castle_decode_flush")


SMALL_LINEAR_MAX_ROWS = 64


def small_linear_ok(x: torch.Tensor, weight: torch.Tensor) -> bool:
    """True if `small_linear` can replace F.linear(x, weight) for this call: a few rows, 16-bit GPU
    tensors, K-contiguous rows that the kernels can read 16 bytes at a time."""
    return (N.is_built() and x.is_cuda and x.dtype in (torch.bfloat16, torch.float16) and weight.dtype == x.dtype
            and x.dim() == 3 and x.shape[1] == 1 and x.shape[0] <= SMALL_LINEAR_MAX_ROWS
            and x.stride(2) == 1 and weight.stride(1) == 1 and x.shape[2] % 8 == 0 and weight.shape[0] % 2 == 0
            and x.stride(0) % 8 == 0 and weight.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0)


@torch.no_grad()
def small_linear(x: torch.Tensor, weight: torch.Tensor, norm=None, activation=None, residual=None) -> torch.Tensor:
    """(B, 1, K) x (N, K) -> (B, 1, N): the projections around the cached single-token step
    (lookahead_keys_attention.py:99, 209 with seq_len == 1), without bias, for inference.

    The per-row work next to such a projection in a token step can ride along (one launch instead
    of up to four): `norm` an nn.RMSNorm applied to x first (lookahead_keys_attention.py:95,
    train_triton.py:103, 164), `activation="gelu"` the erf GELU of train_triton.py:105 on the
    product, `residual` a (B, 1, N) tensor added last (train_triton.py:161-162)."""
    B, _, K = x.shape
    n = weight.shape[0]
    y = torch.empty((B, 1, n), dtype=x.dtype, device=x.device)
    norm_weight, eps = None, 0.0
    if norm is not None:
        norm_weight = norm.weight
        eps = norm.eps if norm.eps is not None else torch.finfo(x.dtype).eps   # what F.rms_norm uses for eps=None
        if norm_weight.dtype != x.dtype or norm_weight.numel() != K or not norm_weight.is_contiguous():
            raise ValueError("small_linear: the norm weight must be a contiguous (K,) tensor of the input type")
    if activation not in (None, "gelu"):
        raise ValueError(f"small_linear: unknown activation {activation!r}")
    if residual is not None and (residual.shape != y.shape or residual.dtype != x.dtype or residual.stride(2) != 1):
        raise ValueError("small_linear: the residual must have the output's shape and type")
    with torch.cuda.device(x.device):
        rc = N.lib().castle_small_linear_fused(
            x.data_ptr(), weight.data_ptr(), y.data_ptr(), B, n, K, x.stride(0), weight.stride(0), n, N.dtype_code(x.dtype),
            norm_weight.data_ptr() if norm_weight is not None else None, eps, 1 if activation == "gelu" else 0,
            residual.data_ptr() if residual is not None else None, residual.stride(0) if residual is not None else 0,
            N.stream_ptr(x.device))
    N.check(rc, "castle_small_linear_fused")
    return y


@torch.no_grad()
def castle_rope_hip(x, out, first_position=0):
    """out[b,h,l,:] = R(first_position + l) x[b,h,l,:]: the rotary position embedding the kernels
    apply under FLAG_ROTARY, for one (B,H,L,d) tensor, out of place (used to fill cache rows)."""
    _require_gpu(x, "castle_rope_hip")
    B, H, L, d = x.shape
    x = _as_readable(x)
    with torch.cuda.device(x.device):
        rc = N.lib().castle_rope(N.view4(x), N.view4(out), B, H, L, d, N.dtype_code(x.dtype), int(first_position),
                                 N.stream_ptr(x.device))
    N.check(rc, "castle_rope")
    return out


@torch.no_grad()
def castle_decode_step_packed(cache_views, capacity, t, proj, heads, scale, out, workspace, rotary=False,
                              t_device=None, deferred=None, u_half=False):
    """The cached step for a fused projection: `proj` is the contiguous (B, 1, 6*H*d) output of the
    layer's projection for the new token (order qu, ku, vu, qc, kc, vc), `cache_views` the four
    castle_view4 of the (B, H, capacity, d) cache buffers (built once per buffer set), `out` a
    (B, 1, H, d) tensor.  Same kernels as castle_decode_step_hip, without per-call view building.

    With `t_device` (a one-element int32 GPU tensor) the kernels read the row count from it and `t`
    is ignored: the launch is then identical for every step, which is what a captured HIP graph of
    the step needs (the caller advances the counter, e.g. with an in-graph `t_device += 1`)."""
    B, n, width = proj.shape
    d = width // (6 * heads)
    if n != 1 or not proj.is_contiguous() or proj.data_ptr() % 16 != 0 or not proj.is_cuda:
        raise ValueError("castle_decode_step_packed needs a contiguous, 16-byte aligned (B, 1, 6*H*d) GPU tensor")
    es, base, part = proj.element_size(), proj.data_ptr(), heads * d
    qu, ku, vu, qc, kc, vc = (N.View4(base + i * part * es, width, d, width) for i in range(6))
    vout = N.View4(out.data_ptr(), heads * d, d, heads * d)
    flags = (N.FLAG_ROTARY if rotary else 0) | (N.FLAG_U_HALF if u_half else 0)
    with torch.cuda.device(proj.device):
        if t_device is None:
            if not (0 <= t < capacity):
                raise ValueError(f"cache capacity {capacity} cannot take row {t}")
            rc = N.lib().castle_decode_step(*cache_views, int(t), int(capacity), qc, kc, vc, qu, ku, vu, B, heads, d,
                                            N.dtype_code(proj.dtype), float(scale), flags, vout, deferred,
                                            workspace.data_ptr(), workspace.numel(), N.stream_ptr(proj.device))
        else:
            if t_device.dtype != torch.int32 or t_device.numel() != 1 or t_device.device != proj.device:
                raise ValueError("t_device must be a one-element int32 tensor on the GPU of the step")
            rc = N.lib().castle_decode_step_device_count(
                *cache_views, t_device.data_ptr(), int(capacity), qc, kc, vc, qu, ku, vu, B, heads, d,
                N.dtype_code(proj.dtype), float(scale), flags, vout, deferred,
                workspace.data_ptr(), workspace.numel(), N.stream_ptr(proj.device))
    N.check(rc, "castle_decode_step")
    return out
