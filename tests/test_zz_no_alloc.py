"""The entry point that takes no workspace (oslo_bias_gelu_bwd_static), called
through the C ABI: its dy and dbias must equal oslo_bias_gelu_bwd's bit for bit
(same kernels, the partial rows in the library's own device buffer instead of
the caller's), on two calls in a row, the second on a smaller problem, so that
what the first call left in the shared buffer is seen not to leak into the
second. Collected last on purpose: the suite stops at the first failure."""

import ctypes

import pytest
import torch

from oslo_amd import _lib
from tests.util import randn

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}
STATIC_BYTES = 32 << 20


def _p(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _both(rows, cols, dtype, seed, want_dbias=True):
    lib = _lib.load()
    g = randn((rows, cols), dtype, seed=seed).to(DEV)
    y = randn((rows, cols), dtype, seed=seed + 1, std=2.0).to(DEV)
    b = randn((cols,), dtype, seed=seed + 2, std=0.5).to(DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = []
    for static in (False, True):
        dy = torch.full_like(y, float("nan"))
        db = torch.full_like(b, float("nan")) if want_dbias else None
        if static:
            st = lib.oslo_bias_gelu_bwd_static(_p(dy), _p(db), _p(g), _p(y), _p(b), rows, cols, CODE[dtype], stream)
        else:
            nbytes = lib.oslo_colsum_workspace_bytes(rows, cols)
            ws = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=DEV)
            st = lib.oslo_bias_gelu_bwd(_p(dy), _p(db), _p(ws), _p(g), _p(y), _p(b), rows, cols, CODE[dtype], stream)
        assert st == 0, lib.oslo_last_error()
        torch.cuda.synchronize()
        out.append((dy, db))
    (dy0, db0), (dy1, db1) = out
    assert torch.isfinite(dy0.float()).all()
    assert torch.equal(dy0, dy1), (rows, cols, dtype)
    if want_dbias:
        assert torch.isfinite(db0.float()).all()
        assert torch.equal(db0, db1), (rows, cols, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16], ids=["bf16", "fp32", "fp16"])
def test_static_workspace_equals_caller_workspace_twice_in_a_row(dtype):
    _both(2048, 4096, dtype, seed=11)      # 64 partial rows
    _both(129, 1000, dtype, seed=12)       # smaller, ragged: 5 partial rows of the same buffer
    _both(33, 8, dtype, seed=13)
    _both(300, 4096, dtype, seed=14, want_dbias=False)


def test_static_workspace_largest_problem_and_limit():
    lib = _lib.load()
    assert lib.oslo_colsum_workspace_bytes(16384, 16384) == STATIC_BYTES
    _both(16384, 16384, torch.bfloat16, seed=21)       # fills the buffer exactly
    _both(64, 16384, torch.bfloat16, seed=22)
    # one row block more than fits: refused before anything is launched
    one = ctypes.c_void_p(256)
    st = lib.oslo_bias_gelu_bwd_static(one, one, one, one, one, 16384 + 1, 16384, 2, None)
    assert st == -2
    msg = lib.oslo_last_error().decode()
    assert "static" in msg and str(STATIC_BYTES) in msg
    # without dbias no workspace is needed and the size is not limited by it
    assert lib.oslo_bias_gelu_bwd_static(None, None, None, None, None, 0, 16384, 2, None) == 0
