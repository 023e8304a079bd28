"""castle_decode_step_static: the cached step for callers that cannot allocate.

It has no counterpart in the reference; it must give what castle_decode_step gives (same kernels,
the partial results in the library's own per-GPU array instead of a caller workspace).  Checked
bit for bit, through the C ABI, on two calls in a row, the second on a smaller problem (fewer
cached rows, fewer heads: fewer and smaller partials than the call before left in the array).
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _state(B, H, cap, t, d, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    caches = [(torch.randn(B, H, cap, d, generator=g) * 0.6).to(dtype) for _ in range(4)]
    toks = [(torch.randn(B, H, 1, d, generator=g) * 0.6).to(dtype) for _ in range(6)]
    return caches, toks


def _step(lib, N, static, caches, toks, t, cap, dtype, t_device=None):
    B, H, _, d = caches[0].shape
    bufs = [c.clone().to(DEV) for c in caches]
    dev_toks = [x.to(DEV) for x in toks]
    out = torch.full((B, H, 1, d), 3.0, dtype=dtype, device=DEV)
    cviews = [N.view4(b) for b in bufs]
    tviews = [N.view4(x) for x in dev_toks]
    code, scale = N.dtype_code(dtype), d ** -0.5
    stream = N.stream_ptr(torch.device(DEV))
    if static:
        td = t_device.data_ptr() if t_device is not None else None
        rc = lib.castle_decode_step_static(*cviews, int(t), td, int(cap), *tviews, B, H, d, code, scale, 0, N.view4(out), None, stream)
    else:
        nbytes = lib.castle_decode_workspace_bytes(B, H, d, cap)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        rc = lib.castle_decode_step(*cviews, int(t), int(cap), *tviews, B, H, d, code, scale, 0, N.view4(out), None,
                                    ws.data_ptr(), nbytes, stream)
    assert rc == 0, lib.castle_error_string(rc)
    torch.cuda.synchronize()
    return out.cpu(), [b.cpu() for b in bufs]


def test_static_scratch_step_equals_workspace_step_twice_in_a_row():
    from lookahead_keys_attention_amd import _native as N

    lib = N.lib()
    # first a problem with many partials (12 heads x 53 splits), then a smaller one (4 heads x 3 splits)
    for (B, H, cap, t, d, dtype, seed) in ((3, 4, 3500, 3400, 64, torch.bfloat16, 1), (2, 2, 200, 150, 32, torch.float32, 2)):
        caches, toks = _state(B, H, cap, t, d, dtype, seed)
        out_s, bufs_s = _step(lib, N, True, caches, toks, t, cap, dtype)
        out_w, bufs_w = _step(lib, N, False, caches, toks, t, cap, dtype)
        assert torch.equal(out_s, out_w)
        for a, b in zip(bufs_s, bufs_w):
            assert torch.equal(a[:, :, : t + 1], b[:, :, : t + 1])
        assert not torch.equal(bufs_s[0][:, :, :t], caches[0][:, :, :t])   # the lookahead keys did move
    # the row count in device memory: same result as the host count
    B, H, cap, t, d, dtype = 2, 2, 200, 150, 32, torch.float32
    caches, toks = _state(B, H, cap, t, d, dtype, 2)
    t_device = torch.tensor([t], dtype=torch.int32, device=DEV)
    out_d, bufs_d = _step(lib, N, True, caches, toks, 0, cap, dtype, t_device=t_device)
    out_w, bufs_w = _step(lib, N, False, caches, toks, t, cap, dtype)
    assert torch.equal(out_d, out_w)
    assert all(torch.equal(a[:, :, : t + 1], b[:, :, : t + 1]) for a, b in zip(bufs_d, bufs_w))


def test_static_scratch_step_rejects_what_does_not_fit():
    from lookahead_keys_attention_amd import _native as N

    lib = N.lib()
    # B*H = 9000 heads at d = 128: 9000 * 130 * 4 bytes of partials > 4 MiB; nothing is launched
    v = N.View4(4096, 128, 128, 128)
    rc = lib.castle_decode_step_static(v, v, v, v, 5, None, 8, v, v, v, v, v, v, 9000, 1, 128, 1, 0.1, 0, v, None, None)
    assert rc == -6
    assert b"static scratch" in lib.castle_error_string(rc)
    # row t must fit the buffers, as in castle_decode_step
    rc = lib.castle_decode_step_static(v, v, v, v, 8, None, 8, v, v, v, v, v, v, 1, 1, 128, 1, 0.1, 0, v, None, None)
    assert rc == -2
