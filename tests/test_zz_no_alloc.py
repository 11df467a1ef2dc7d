"""The decode attention entry point that allocates nothing (`holon_attention_decode_bf16_static`), called through
ctypes as a caller without an allocator would: its split partials live in a device array inside the library. It must
give bit for bit what the entry point with a caller's workspace gives, on two calls in a row (the second smaller, so
that it runs over what the first left in the array), stay within the bfloat16 budget of the plain attention computed in
float64 (the two entry points share their launch: a fault in it would not show between them), and refuse what does
not fit."""
from __future__ import annotations

import ctypes

import pytest
import torch

from tests import helpers as H
from tests.plain.ops import TorchKernels
from tests.test_kernels_gpu import _paged_case

pytestmark = pytest.mark.gpu
_P, _I, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
HEAD = [_P, _P, _P, _P, _I, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I]       # q .. window


@pytest.fixture(scope="module")
def lib():
    from holon_amd.kernels import build
    path = build.find_library()
    assert path is not None, "libholon_hip.so is not built"
    lib = ctypes.CDLL(str(path))
    lib.holon_last_error.restype = ctypes.c_char_p
    lib.holon_decode_scratch_bytes.restype = ctypes.c_int64
    lib.holon_attention_decode_bf16.argtypes = HEAD + [_P, _P, _I, _I, _P]
    lib.holon_attention_decode_bf16_static.argtypes = HEAD + [_I, _I, _P]
    return lib


def _both(lib, rows, heads, kv_heads, head_dim, splits, seed, window=0):
    page = 16
    q, pages, table, attn = _paged_case(rows, heads, kv_heads, head_dim, page, torch.bfloat16, seed, max_seqs=len(rows))
    n, longest = len(rows), max(s + c for s, c in rows)
    per = -(-(-(-longest // splits)) // 32) * 32
    head = (q.data_ptr(), None, pages.data_ptr(), table.data_ptr(), table.shape[1], attn.slots.data_ptr(),
            attn.lens.data_ptr(), attn.query_start.data_ptr(), attn.decode_rows.data_ptr(), n, longest, heads, kv_heads,
            head_dim, page, head_dim ** -0.5, window)
    stream = torch.cuda.current_stream().cuda_stream
    want, got = torch.full_like(q, 7.0), torch.full_like(q, -7.0)
    part_o = torch.empty(n * heads * splits * head_dim, dtype=torch.float32, device="cuda")
    part_ml = torch.empty(n * heads * splits * 2, dtype=torch.float32, device="cuda")
    rc = lib.holon_attention_decode_bf16(head[0], want.data_ptr(), *head[2:], part_o.data_ptr(), part_ml.data_ptr(),
                                         splits, per, stream)
    assert rc == 0, lib.holon_last_error().decode()
    before = torch.cuda.memory_allocated()
    rc = lib.holon_attention_decode_bf16_static(head[0], got.data_ptr(), *head[2:], splits, per, stream)
    assert rc == 0, lib.holon_last_error().decode()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    plain = TorchKernels().paged_attention(q.double(), pages.double(), table, attn, page, head_dim ** -0.5, window)
    assert H.op_budget_usage(got, plain, torch.bfloat16, head_dim + longest) <= 1, (rows, heads, kv_heads, head_dim)
    return got, want


def test_two_calls_in_a_row_equal_the_entry_point_with_a_workspace(lib):
    assert lib.holon_decode_scratch_init() == 0, lib.holon_last_error().decode()
    big = [(900 + 37 * i, 1) for i in range(8)]
    got, want = _both(lib, big, 32, 8, 128, splits=16, seed=1)
    assert torch.equal(got, want) and torch.isfinite(got.float()).all()
    small = [(70, 1), (15, 1), (0, 1)]                       # fewer rows, fewer splits: over the first call's leavings
    got, want = _both(lib, small, 32, 8, 128, splits=3, seed=2)
    assert torch.equal(got, want)
    got, want = _both(lib, [(300, 1), (31, 1)], 6, 2, 64, splits=5, seed=3, window=100)   # another geometry, a window
    assert torch.equal(got, want)


def test_what_does_not_fit_is_refused(lib):
    q = torch.zeros(1, device="cuda")
    limit = lib.holon_decode_scratch_bytes()
    rows = limit // (32 * 64 * 130 * 4) + 1                  # one row more than the array holds at 64 splits
    rc = lib.holon_attention_decode_bf16_static(q.data_ptr(), q.data_ptr(), q.data_ptr(), q.data_ptr(), 1, q.data_ptr(),
                                                q.data_ptr(), q.data_ptr(), q.data_ptr(), rows, 4096, 32, 8, 128, 16,
                                                0.1, 0, 64, 64, None)
    assert rc != 0 and "built-in buffer holds" in lib.holon_last_error().decode()
