"""The C-ABI shared library: builds, loads, exports every symbol include/castle_hip.h
declares, and validates arguments on the host (no kernel is launched here)."""
import ctypes
import os
import re

import pytest

from lookahead_keys_attention_amd import _native as N

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "castle_hip.h")


@pytest.fixture(scope="module")
def lib():
    if not N.is_built():
        from lookahead_keys_attention_amd.build import build

        build()
    return N.lib()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(castle_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    names = declared_functions()
    assert sorted(N.EXPORTED_SYMBOLS) == names
    raw = ctypes.CDLL(N.LIB_PATH)
    for name in names:
        assert hasattr(raw, name), f"{name} missing from libcastle_hip.so"


def test_version_and_error_strings(lib):
    assert lib.castle_abi_version() == 5
    assert lib.castle_error_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert len(lib.castle_error_string(code)) > 3


def test_workspace_sizes(lib):
    # B4 H8 L4096 d64 bf16.  Kept for backward (O(L d)): header + lse + three T arrays (T', T'^T, cross quarter) +
    # six operand copies; state buffer (O(L^2 d / 128)): snapshots, 64 * nblk*(nblk-1)/2 rows per head
    n = lib.castle_fwd_workspace_bytes(4, 8, 4096, 64, 1)
    BH, Lp, nblk = 32, 4096, 64
    header = 256 + 4 * 256   # status / scale header + partial maxima
    snaps = BH * 64 * nblk * (nblk - 1) // 2 * 64 * 2
    assert n == header + BH * Lp * 4 + 3 * BH * Lp * 64 * 2 + 6 * BH * Lp * 64 * 2
    assert lib.castle_fwd_state_bytes(4, 8, 4096, 64, 1) == snaps
    bwd = header + snaps + BH * Lp * 4 + BH * Lp * 64 * 2 + 2 * BH * Lp * Lp * 2
    assert lib.castle_bwd_workspace_bytes(4, 8, 4096, 64, 1, 0) == bwd
    assert lib.castle_bwd_workspace_bytes(4, 8, 4096, 64, 1, N.FLAG_RECOMPUTE_STATE) == bwd + snaps
    assert lib.castle_bwd_workspace_bytes(4, 8, 4096, 64, 1, N.FLAG_RECOMPUTE_SCORES) == bwd - 2 * BH * Lp * Lp * 2
    # ragged L rounds up to 128 rows
    assert lib.castle_fwd_workspace_bytes(1, 1, 129, 64, 0) == lib.castle_fwd_workspace_bytes(1, 1, 256, 64, 0)
    assert lib.castle_decode_workspace_bytes(32, 8, 64, 4096) > 0


def test_state_size_formula_of_the_python_callers_matches_the_library(lib):
    from lookahead_keys_attention_amd import ops

    for B, H, L, d, dtype, es in ((4, 8, 4096, 64, 1, 2), (1, 16, 16384, 128, 1, 2), (2, 2, 100, 32, 0, 4), (1, 1, 129, 16, 2, 2),
                                  (3, 5, 128, 64, 0, 4)):
        assert ops.state_bytes_formula(B, H, L, d, es) == lib.castle_fwd_state_bytes(B, H, L, d, dtype)


def test_rejects_bad_shapes_and_types(lib):
    assert lib.castle_fwd_workspace_bytes(1, 1, 16, 48, 1) == -2      # head dim not supported
    assert lib.castle_fwd_workspace_bytes(1, 1, 16, 128, 0) == -2     # fp32 needs d <= 64
    assert lib.castle_fwd_workspace_bytes(1, 1, 16, 64, 7) == -1      # unknown dtype
    assert lib.castle_fwd_workspace_bytes(0, 1, 16, 64, 1) == -2
    assert lib.castle_decode_workspace_bytes(1, 1, 24, 8) == -2


def test_null_and_misaligned_views_are_rejected_on_the_host(lib):
    ok = N.View4(4096, 64, 64, 64)
    null = N.View4(None, 0, 0, 0)
    odd = N.View4(4098, 64, 64, 64)          # not 16-byte aligned
    bad_stride = N.View4(4096, 64, 64, 3)    # rows not 16-byte aligned
    args = lambda v: ([ok] * 5 + [v], [1, 1, 16, 64, 1, 0.125, 0, ok, null, 4096, 1 << 30, 8192, 1 << 30, None])
    for bad in (null, odd, bad_stride):
        a, b = args(bad)
        assert lib.castle_fwd(*a, *b) == -5
    a, b = args(ok)
    b[9] = None                                # no workspace
    assert lib.castle_fwd(*a, *b) == -4
    b[9], b[10] = 4096, 16                     # too small
    assert lib.castle_fwd(*a, *b) == -4
    b[10], b[11] = 1 << 30, None               # no state buffer
    assert lib.castle_fwd(*a, *b) == -4


def test_small_linear_and_static_step_validate_on_the_host(lib):
    assert lib.castle_small_linear(4096, 4096, 4096, 4, 64, 30, 64, 64, 64, 1, None) == -2     # K % 8
    assert lib.castle_small_linear(4096, 4096, 4096, 4, 64, 32, 64, 64, 64, 0, None) == -1     # fp32 not offered
    assert lib.castle_small_linear(None, 4096, 4096, 4, 64, 32, 64, 64, 64, 1, None) == -5
    assert lib.castle_small_linear(4100, 4096, 4096, 4, 64, 32, 64, 64, 64, 1, None) == -5     # misaligned x
    # castle_decode_step_static: partials beyond the 4 MiB array, and a row beyond the capacity
    v = N.View4(4096, 128, 128, 128)
    rc = lib.castle_decode_step_static(v, v, v, v, 5, None, 8, v, v, v, v, v, v, 9000, 1, 128, 1, 0.1, 0, v, None, None)
    assert rc == -6 and b"static scratch" in lib.castle_error_string(rc)
    assert lib.castle_decode_step_static(v, v, v, v, 8, None, 8, v, v, v, v, v, v, 1, 1, 128, 1, 0.1, 0, v, None, None) == -2
    assert lib.castle_decode_step(v, v, v, v, 8, 8, v, v, v, v, v, v, 1, 1, 128, 1, 0.1, 0, v, None, 4096, 1 << 30, None) == -2


def test_check_raises_with_message(lib):
    with pytest.raises(RuntimeError, match="unsupported shape"):
        N.check(-2, "castle_fwd")
