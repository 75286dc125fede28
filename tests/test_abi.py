"""The C-ABI library loads without a GPU, exports every symbol the header
declares, and answers the calls that need no device (integer helpers and
argument screening that fails before any launch)."""

import ctypes
import os
import re

import pytest

from oracle import oslo_oracle as orc
from oslo_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "oslo_amd.h")


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(oslo_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree(lib):
    names = declared_symbols()
    assert len(names) >= 14
    assert sorted(_lib.PROTOTYPES) == names
    for name in names:
        assert getattr(lib, name) is not None


def test_header_compiles_as_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "oslo_amd.h"\nint main(void){return OSLO_OK + OSLO_F32 + OSLO_MASK_ADD;}\n')
    import subprocess

    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic",
                           f"-I{os.path.dirname(HEADER)}", "-c", str(src), "-o", str(tmp_path / "t.o")])


def test_identity(lib):
    assert lib.oslo_abi_version() == _lib.ABI_VERSION
    assert lib.oslo_softmax_max_cols() == 8192
    assert lib.oslo_status_string(0) == b"ok"
    assert lib.oslo_status_string(-2) == b"unsupported shape"


def test_get_batch_per_block_equals_reference_table(lib):
    for sk in list(range(1, 300)) + [511, 512, 513, 1023, 1024, 1025, 2047, 2048]:
        assert lib.oslo_get_batch_per_block(5, sk, 2, 3) == orc.get_batch_per_block(5, sk, 2, 3), sk


def test_workspace_bytes(lib):
    assert lib.oslo_colsum_workspace_bytes(0, 128) == 0
    assert lib.oslo_colsum_workspace_bytes(128, 0) == 0
    # one fp32 partial row per 32 rows
    assert lib.oslo_colsum_workspace_bytes(1, 8) == 1 * 8 * 4
    assert lib.oslo_colsum_workspace_bytes(16384, 16384) == 512 * 16384 * 4
    assert lib.oslo_colsum_workspace_bytes(16385, 10) == 513 * 10 * 4


def test_softmax_row_limit_is_on_rows_not_elements(lib):
    """A call takes at most 2^31 - 1 rows (batch * heads * S); more is refused
    with OSLO_E_UNSUPPORTED before any pointer is looked at. The number of
    elements is not limited: the gate admits [32,16,2048,2048] (2^31 elements)
    and [4,16,8192,8192] (2^32)."""
    import torch

    from oslo_amd import FusedScaleMaskSoftmax

    null, one = ctypes.c_void_p(0), ctypes.c_void_p(16)
    rows_ok, rows_too_many = (2 ** 31 - 8) // 8, 2 ** 31 // 8      # heads of S = 8
    assert lib.oslo_softmax_causal_fwd(one, one, null, 1.0, 1, rows_too_many, 8, 1, null) == -2
    assert b"rows" in lib.oslo_last_error()
    assert lib.oslo_softmax_causal_bwd(one, one, one, 1.0, rows_too_many, 8, 1, null) == -2
    assert lib.oslo_softmax_causal_window_fwd(one, one, null, 1.0, 4, 1, rows_too_many, 8, 1, null) == -2
    assert lib.oslo_softmax_masked_fwd(one, one, null, 0, 0, 0, 1.0, 2 ** 16, 2 ** 15, 1, 8, 1, null) == -2
    assert lib.oslo_softmax_masked_bwd(one, one, one, 1.0, 2 ** 31, 8, 1, null) == -2
    assert rows_ok * 8 < 2 ** 31
    for dtype in (torch.half, torch.bfloat16, torch.float32):
        assert FusedScaleMaskSoftmax.is_available(dtype, 32, 16, 2048, 2048, True)
        assert FusedScaleMaskSoftmax.is_available(dtype, 4, 16, 8192, 8192, True)
        assert FusedScaleMaskSoftmax.is_available(dtype, 64, 16, 2048, 1024, False)
        assert not FusedScaleMaskSoftmax.is_available(dtype, 2 ** 16, 2 ** 12, 8, 8, True)   # 2^31 rows
        assert FusedScaleMaskSoftmax.is_available(dtype, 2 ** 16 - 1, 2 ** 12, 8, 8, True)


def test_argument_screening_without_a_device(lib):
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)  # never dereferenced: every call below fails or returns first
    # negative sizes
    assert lib.oslo_softmax_causal_fwd(one, one, null, 1.0, -1, 1, 8, 1, null) == -1
    assert lib.oslo_softmax_masked_bwd(one, one, one, 1.0, -1, 8, 1, null) == -1
    assert lib.oslo_bias_gelu_fwd(one, one, one, 4, -8, 1, null) == -1
    # rows longer than the limit
    assert lib.oslo_softmax_causal_fwd(one, one, null, 1.0, 1, 1, 8200, 1, null) == -2
    assert b"8200" in lib.oslo_last_error()
    assert lib.oslo_softmax_masked_fwd(one, one, null, 0, 0, 0, 1.0, 1, 1, 2, 8193, 1, null) == -2
    # null tensors, unknown enums
    assert lib.oslo_softmax_causal_bwd(null, one, one, 1.0, 1, 8, 1, null) == -1
    assert lib.oslo_softmax_masked_fwd(one, one, null, 0, 0, 7, 1.0, 1, 1, 2, 8, 1, null) == -1
    assert lib.oslo_softmax_causal_fwd(one, one, null, 1.0, 1, 1, 8, 9, null) == -1
    assert lib.oslo_bias_gelu_bwd(one, one, null, one, one, one, 4, 8, 1, null) == -1  # dbias without workspace
    # dropout probability outside [0, 1)
    assert lib.oslo_bias_dropout_add_fwd(one, one, null, null, 1.0, 1, 0, 4, 8, 1, null) == -1
    assert lib.oslo_bias_dropout_add_fwd(one, one, null, null, -0.1, 1, 0, 4, 8, 1, null) == -1
    assert lib.oslo_bias_dropout_add_bwd(one, null, null, one, float("nan"), 1, 0, 4, 8, 1, null) == -1
    # a second residual needs a first; the variant screens like the one-residual entry
    assert lib.oslo_bias_dropout_add2_fwd(one, one, null, null, one, 0.1, 1, 0, 4, 8, 1, null) == -1
    assert b"second residual" in lib.oslo_last_error()
    assert lib.oslo_bias_dropout_add2_fwd(one, one, null, one, one, 1.0, 1, 0, 4, 8, 1, null) == -1
    assert lib.oslo_bias_dropout_add2_fwd(null, null, null, null, null, 0.1, 1, 0, 0, 8, 1, null) == 0
    # softmax with fused dropout: p, the statistics buffer, sizes
    assert lib.oslo_softmax_causal_dropout_fwd(one, one, one, null, 1.0, 1.0, 1, 0, 1, 1, 8, 1, null) == -1
    assert lib.oslo_softmax_causal_dropout_fwd(one, null, one, null, 1.0, 0.1, 1, 0, 1, 1, 8, 1, null) == -1
    assert lib.oslo_softmax_causal_dropout_bwd(one, one, one, null, null, 1.0, 0.1, 1, 0, 1, 1, 8, 1, null) == -1
    assert lib.oslo_softmax_causal_dropout_bwd(one, one, one, one, null, 1.0, 0.1, 1, 0, 1, 1, 9000, 1, null) == -2
    assert lib.oslo_softmax_causal_dropout_fwd(null, null, null, null, 1.0, 0.1, 1, 0, 0, 1, 8, 1, null) == 0
    # rotary: odd or oversized rotary_dim, head_dim not a multiple of the vector, table too short,
    # one pointer of a pair, in place
    two = ctypes.c_void_p(32)
    assert lib.oslo_rotary_qkv(one, null, null, two, null, null, one, one, 8, 1, 8, 2, 16, 0, 3, 0, 0, 1, null) == -1
    assert lib.oslo_rotary_qkv(one, null, null, two, null, null, one, one, 8, 1, 8, 2, 16, 0, 32, 0, 0, 1, null) == -1
    assert lib.oslo_rotary_qkv(one, null, null, two, null, null, one, one, 8, 1, 8, 2, 12, 0, 4, 0, 0, 1, null) == -2
    assert lib.oslo_rotary_qkv(one, null, null, two, null, null, one, one, 8, 1, 8, 2, 16, 0, 4, 1, 0, 1, null) == -1
    assert b"table" in lib.oslo_last_error()
    assert lib.oslo_rotary_qkv(one, null, null, null, null, null, one, one, 8, 1, 8, 2, 16, 0, 4, 0, 0, 1, null) == -1
    assert lib.oslo_rotary_qkv(two, null, null, two, null, null, one, one, 8, 1, 8, 2, 16, 0, 4, 0, 0, 1, null) == -1
    assert lib.oslo_rotary_qkv(one, null, null, two, null, null, one, one, 8, 1, 8, 2, 16, 24, 4, 0, 0, 1, null) == -1
    assert b"row_stride" in lib.oslo_last_error()      # smaller than heads*head_dim
    assert lib.oslo_rotary_qkv(null, null, null, null, null, null, null, null, 0, 1, 8, 2, 16, 0, 4, 0, 0, 1, null) == 0
    # few-row linear layer: too many rows, ragged rows, unknown epilogue, aliasing, misalignment
    three = ctypes.c_void_p(48)
    assert lib.oslo_linear_rows_max() == 8
    assert lib.oslo_linear_rows_fwd(one, two, three, null, null, 9, 4, 8, 0, 1, null) == -2
    assert lib.oslo_linear_rows_fwd(one, two, three, null, null, 1, 4, 12, 0, 1, null) == -2
    assert lib.oslo_linear_rows_fwd(one, two, three, null, null, 1, 4, 8, 5, 1, null) == -1
    assert lib.oslo_linear_rows_fwd(two, two, three, null, null, 1, 4, 8, 0, 1, null) == -1
    assert lib.oslo_linear_rows_fwd(one, ctypes.c_void_p(40), three, null, null, 1, 4, 8, 0, 1, null) == -1
    assert lib.oslo_linear_rows_fwd(one, two, three, null, null, 1, 1 << 30, 8, 0, 1, null) == -2
    assert lib.oslo_linear_rows_fwd(one, two, null, null, null, 1, 4, 8, 0, 1, null) == -1
    assert lib.oslo_linear_rows_fwd(null, null, null, null, null, 0, 4, 8, 0, 1, null) == 0
    assert lib.oslo_linear_rows_kn_fwd(one, two, three, null, null, 9, 8, 8, 0, 1, null) == -2
    assert lib.oslo_linear_rows_kn_fwd(one, two, three, null, null, 1, 12, 8, 0, 1, null) == -2     # ragged weight rows
    assert lib.oslo_linear_rows_kn_fwd(one, two, three, null, null, 1, 8, 8, 0, 7, null) == -1
    assert lib.oslo_linear_rows_kn_fwd(null, null, null, null, null, 0, 8, 8, 0, 1, null) == 0
    table = (ctypes.c_void_p * 3)(16, 32, 48)
    assert lib.oslo_linear_rows_fwd_multi(table, one, table, null, 4, 1, 4, 8, 0, 1, null) == -1     # four layers
    assert lib.oslo_linear_rows_fwd_multi(null, one, table, null, 2, 1, 4, 8, 0, 1, null) == -1
    assert lib.oslo_linear_rows_fwd_multi(table, ctypes.c_void_p(64), table, null, 3, 1, 4, 8, 0, 1, null) == -1  # out[j] is weight[j]
    # attention of a decoding step: head size, position, null pointers, workspace size
    assert lib.oslo_attention_decode_fwd(one, two, three, three, null, null, 0, 0, one, null, 0, 0, 1.0, 4, 64, 48, 1, null) == -2
    assert lib.oslo_attention_decode_fwd(one, two, three, three, null, null, 0, 0, one, null, 64, 0, 1.0, 4, 64, 64, 1, null) == -1
    assert lib.oslo_attention_decode_fwd(one, two, three, three, null, null, 0, 0, null, null, 3, 0, 1.0, 4, 64, 64, 1, null) == -1
    assert lib.oslo_attention_decode_fwd(one, two, three, three, null, null, 0, 0, one, null, 3, -1, 1.0, 4, 64, 64, 1, null) == -1
    assert lib.oslo_attention_decode_fwd(null, null, null, null, null, null, 0, 0, null, null, 0, 0, 1.0, 0, 64, 64, 1, null) == 0
    assert lib.oslo_attention_decode_fwd(one, two, three, three, one, null, 2, 0, one, null, 3, 0, 1.0, 4, 64, 64, 1, null) == -1  # k_new alone
    assert lib.oslo_attention_decode_fwd(one, two, three, three, one, one, 3, 0, one, null, 3, 0, 1.0, 4, 64, 64, 1, null) == -1  # 3 heads, 4 rows
    assert lib.oslo_attention_decode_fwd(one, two, three, three, one, one, 2, 100, one, null, 3, 0, 1.0, 4, 64, 64, 1, null) == -1  # stride below heads*head_dim
    assert lib.oslo_attention_decode_workspace_bytes(16, 1152, 256, 2) == 16 * 18 * 258 * 4
    assert lib.oslo_attention_decode_workspace_bytes(16, 1152, 48, 2) == 0
    # the attention's backward with a tile store: its size, a store too small for 8 heads, none at all
    assert lib.oslo_attention_prefill_bwd_store_bytes(0, 16, 2048) == 0
    assert lib.oslo_attention_prefill_bwd_store_bytes(8, 16, 2048) == 128 * (64 * 65 // 2) * 4096
    assert lib.oslo_attention_prefill_bwd_store_bytes(1, 3, 100) == 8 * (4 * 5 // 2) * 4096    # 8 heads, one block of 128
    strides = (ctypes.c_int64 * 24)(*(8 * [2 * 100 * 64, 100 * 64, 64]))
    args = (one, one, one, one, one, one, one, one, one, one)
    tail = (null, 0.125, 0.0, 0, 0, 1, 2, 100, 64, 0, strides, 2, null)
    assert lib.oslo_attention_prefill_bwd_stored(*args, null, 1 << 20, *tail) == -1
    assert b"null store" in lib.oslo_last_error()
    assert lib.oslo_attention_prefill_bwd_stored(*args, one, 8 * 10 * 4096 - 1, *tail) == -1
    assert b"8 heads" in lib.oslo_last_error()
    assert lib.oslo_attention_prefill_bwd_stored(*args, ctypes.c_void_p(24), 1 << 30, *tail) == -2   # misaligned
    assert lib.oslo_attention_prefill_bwd_stored(*args, one, 1 << 30, *(tail[:6] + (0,) + tail[7:])) == 0  # no positions
    # n-gram blocking
    assert lib.oslo_ngram_repeat_block(one, one, 2, 4, 3, 8, 0, null) == -1
    assert lib.oslo_ngram_repeat_block(null, one, 2, 4, 3, 8, 2, null) == -1
    # empty problems succeed without touching the device
    assert lib.oslo_softmax_causal_fwd(null, null, null, 1.0, 0, 4, 8, 1, null) == 0
    assert lib.oslo_softmax_masked_fwd(null, null, null, 0, 0, 0, 1.0, 2, 2, 0, 8, 1, null) == 0
    assert lib.oslo_bias_gelu_fwd(null, null, null, 0, 8, 1, null) == 0
    assert lib.oslo_bias_dropout_add_fwd(null, null, null, null, 0.5, 1, 0, 0, 8, 1, null) == 0


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/liboslo_amd.so")
    with pytest.raises(EnvironmentError):
        _lib.load()
