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
"""
from __future__ import annotations

import torch

from . import _native as N


# flags handed to castle_fwd / castle_bwd (0, or _native.FLAG_BF16_OPERANDS); read when the
# forward runs and remembered for its backward.  The `rotary` arguments below add FLAG_ROTARY.
DEFAULT_FLAGS = 0
# Debugging aid: when True every parallel forward waits for its kernels and raises if they had to
# clamp a value to the fp16 range (an input element of a bf16 tensor beyond +-65504, or a T' entry):
# the result is then that of the clamped operands.  Off by default because it synchronises.
CHECK_RANGE = False


def _require_gpu(t: torch.Tensor, what: str):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: the HIP kernels need tensors on the GPU (got {t.device})")


def _check_dims(d: int, dtype: torch.dtype):
    if d not in N.SUPPORTED_HEAD_DIMS:
        raise ValueError(f"dim_head must be one of {N.SUPPORTED_HEAD_DIMS} for the HIP kernels, got {d}")
    if dtype == torch.float32 and d > 64:
        raise ValueError("float32 HIP kernels support dim_head <= 64")


def _fwd_raw(qc, kc, vc, qu, ku, vu, scale, out, U, flags=0):
    """Launch castle_fwd; returns the forward workspace tensor."""
    B, H, L, d = qc.shape
    code = N.dtype_code(qc.dtype)
    lib = N.lib()
    nbytes = N.check(lib.castle_fwd_workspace_bytes(B, H, L, d, code), "castle_fwd_workspace_bytes")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=qc.device)
    views = [N.view4(t) for t in (qc, kc, vc, qu, ku, vu)]
    vo = N.view4(out)
    vU = N.view4(U) if U is not None else N.View4(None, 0, 0, 0)
    with torch.cuda.device(qc.device):
        rc = lib.castle_fwd(*views, B, H, L, d, code, float(scale), int(flags), vo, vU, ws.data_ptr(), nbytes, N.stream_ptr(qc.device))
    N.check(rc, "castle_fwd")
    if CHECK_RANGE:
        status = range_status(ws)
        if status:
            raise RuntimeError(f"castle_fwd clamped values to the fp16 range (status bits {status:#x}: "
                               "1 = input element, 2 = T' = s qc.vu entry)")
    return ws


def range_status(ws: torch.Tensor) -> int:
    """Status word the forward kernels leave at the start of their workspace (synchronises):
    bit 0 = an input element was clamped to +-65504, bit 1 = an entry of T' = s qc.vu was."""
    return int(ws[:4].view(torch.int32).item())


def _bwd_raw(qc, kc, vc, qu, ku, vu, out, dout, scale, grads, ws, flags=0):
    B, H, L, d = qc.shape
    code = N.dtype_code(qc.dtype)
    lib = N.lib()
    nbytes = N.check(lib.castle_bwd_workspace_bytes(B, H, L, d, code, int(flags)), "castle_bwd_workspace_bytes")
    bws = torch.empty(nbytes, dtype=torch.uint8, device=qc.device)
    views = [N.view4(t) for t in (qc, kc, vc, qu, ku, vu, out, dout)]
    gviews = [N.view4(t) for t in grads]
    with torch.cuda.device(qc.device):
        rc = lib.castle_bwd(*views, B, H, L, d, code, float(scale), int(flags), *gviews,
                            ws.data_ptr(), ws.numel(), bws.data_ptr(), nbytes, N.stream_ptr(qc.device))
    N.check(rc, "castle_bwd")


def _as_readable(t: torch.Tensor) -> torch.Tensor:
    return t if N.vector_ok(t) else t.contiguous()


class _CastleAttention(torch.autograd.Function):
    """Six separate operands (the reference operator's signature)."""

    @staticmethod
    def forward(ctx, q, k, v, qu, ku, vu, scale, want_U, rotary=False):
        _require_gpu(q, "castle_attention_hip")
        B, H, L, d = q.shape
        _check_dims(d, q.dtype)
        ops = [_as_readable(t) for t in (q, k, v, qu, ku, vu)]
        out = torch.empty((B, L, H, d), dtype=q.dtype, device=q.device).permute(0, 2, 1, 3)
        U = torch.empty((B, H, L, d), dtype=q.dtype, device=q.device) if want_U else None
        ctx.flags = DEFAULT_FLAGS | (N.FLAG_ROTARY if rotary else 0)
        ws = _fwd_raw(*ops, scale, out, U, ctx.flags)
        ctx.save_for_backward(*ops, out, ws)
        ctx.scale = scale
        if want_U:
            ctx.mark_non_differentiable(U)
            return out, U
        return out

    @staticmethod
    def backward(ctx, dout, dU=None):
        *ops, out, ws = ctx.saved_tensors
        B, H, L, d = ops[0].shape
        dout = _as_readable(dout)
        packed = torch.empty((6, B, H, L, d), dtype=out.dtype, device=out.device)
        grads = list(packed.unbind(0))
        _bwd_raw(*ops, out, dout, ctx.scale, grads, ws, ctx.flags)
        return (*grads, None, None, None)


class _CastleAttentionPacked(torch.autograd.Function):
    """Fused-projection layout in, merged heads out."""

    @staticmethod
    def forward(ctx, proj, heads, scale, U_out, rotary=False):
        # U_out: None, or a (B,H,L,d) view without gradient history that receives the lookahead keys
        _require_gpu(proj, "castle_attention_packed")
        B, L, width = proj.shape
        d = width // (6 * heads)
        _check_dims(d, proj.dtype)
        proj = proj if (proj.is_contiguous() and proj.data_ptr() % 16 == 0) else proj.contiguous()
        six = proj.view(B, L, 6, heads, d).permute(2, 0, 3, 1, 4)      # (6, B, H, L, d) views
        qu, ku, vu, qc, kc, vc = six.unbind(0)
        merged = torch.empty((B, L, heads * d), dtype=proj.dtype, device=proj.device)
        out = merged.view(B, L, heads, d).permute(0, 2, 1, 3)
        ctx.flags = DEFAULT_FLAGS | (N.FLAG_ROTARY if rotary else 0)
        ws = _fwd_raw(qc, kc, vc, qu, ku, vu, scale, out, U_out, ctx.flags)
        ctx.save_for_backward(proj, merged, ws)
        ctx.heads, ctx.scale = heads, scale
        return merged

    @staticmethod
    def backward(ctx, dmerged):
        proj, merged, ws = ctx.saved_tensors
        heads, scale = ctx.heads, ctx.scale
        B, L, width = proj.shape
        d = width // (6 * heads)
        six = proj.view(B, L, 6, heads, d).permute(2, 0, 3, 1, 4)
        qu, ku, vu, qc, kc, vc = six.unbind(0)
        out = merged.view(B, L, heads, d).permute(0, 2, 1, 3)
        dmerged = dmerged if (dmerged.is_contiguous() and dmerged.data_ptr() % 16 == 0) else dmerged.contiguous()
        dout = dmerged.view(B, L, heads, d).permute(0, 2, 1, 3)
        dproj = torch.empty_like(proj)
        dqu, dku, dvu, dqc, dkc, dvc = dproj.view(B, L, 6, heads, d).permute(2, 0, 3, 1, 4).unbind(0)
        _bwd_raw(qc, kc, vc, qu, ku, vu, out, dout, scale, (dqc, dkc, dvc, dqu, dku, dvu), ws, ctx.flags)
        return dproj, None, None, None, None


def castle_attention_hip(q, k, v, qu, ku, vu, scale, return_U_for_cache=False, rotary=False):
    """Drop-in for castle_attention_triton: returns out, or (out, U).  rotary=True applies the
    rotary position embedding (positions 0..L-1) to q, k, qu, ku, vu inside the kernels."""
    return _CastleAttention.apply(q, k, v, qu, ku, vu, float(scale), bool(return_U_for_cache), bool(rotary))


def castle_attention_packed(proj, heads, scale, return_U_for_cache=False, U_out=None, rotary=False):
    """proj (B, L, 6*H*d) -> merged out (B, L, H*d), or (out, U (B,H,L,d)).  `U_out`, if given,
    is the (B,H,L,d) view (any row stride) the lookahead keys are written into."""
    if not return_U_for_cache:
        return _CastleAttentionPacked.apply(proj, int(heads), float(scale), None, bool(rotary))
    if U_out is None:
        B, L, width = proj.shape
        U_out = torch.empty((B, heads, L, width // (6 * heads)), dtype=proj.dtype, device=proj.device)
    return _CastleAttentionPacked.apply(proj, int(heads), float(scale), U_out, bool(rotary)), U_out


def decode_workspace(B, H, d, device):
    nbytes = N.check(N.lib().castle_decode_workspace_bytes(B, H, d, 0), "castle_decode_workspace_bytes")
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


@torch.no_grad()
def castle_decode_step_hip(U, qu_cache, kc_cache, vc_cache, t, qc, kc, vc, qu, ku, vu, scale, out, workspace,
                           rotary=False):
    """In-place cached step.  The four cache tensors are (B,H,capacity,d) buffers with t valid
    rows (capacity > t); the new-token operands and `out` are (B,H,1,d).  rotary=True rotates the
    new token by position t inside the kernels (the cache rows are stored rotated)."""
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
                                        N.FLAG_ROTARY if rotary else 0, N.view4(out),
                                        workspace.data_ptr(), workspace.numel(), N.stream_ptr(U.device))
    N.check(rc, "castle_decode_step")
    return out


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
                              t_device=None):
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
    flags = N.FLAG_ROTARY if rotary else 0
    with torch.cuda.device(proj.device):
        if t_device is None:
            if not (0 <= t < capacity):
                raise ValueError(f"cache capacity {capacity} cannot take row {t}")
            rc = N.lib().castle_decode_step(*cache_views, int(t), int(capacity), qc, kc, vc, qu, ku, vu, B, heads, d,
                                            N.dtype_code(proj.dtype), float(scale), flags, vout,
                                            workspace.data_ptr(), workspace.numel(), N.stream_ptr(proj.device))
        else:
            if t_device.dtype != torch.int32 or t_device.numel() != 1 or t_device.device != proj.device:
                raise ValueError("t_device must be a one-element int32 tensor on the GPU of the step")
            rc = N.lib().castle_decode_step_device_count(
                *cache_views, t_device.data_ptr(), int(capacity), qc, kc, vc, qu, ku, vu, B, heads, d,
                N.dtype_code(proj.dtype), float(scale), flags, vout,
                workspace.data_ptr(), workspace.numel(), N.stream_ptr(proj.device))
    N.check(rc, "castle_decode_step")
    return out
