"""ctypes binding of ``liboslo_amd.so``: one prototype per entry point of
``include/oslo_amd.h``. Loading never compiles anything and never falls back to
another implementation: if the library is missing the import of a kernel fails
with ``EnvironmentError`` (the reference raises the same type when its JIT
build fails, oslo/fused_kernels_utils.py:226-230)."""

import ctypes
import os

# The library lies beside this file. OSLO_AMD_LIB names another build of it
# (``python -m oslo_amd.build`` writes there too when the variable is set): a
# library built with other tuning switches, for measurements.
LIB_PATH = os.environ.get("OSLO_AMD_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "liboslo_amd.so")

_c = ctypes
_P = _c.c_void_p
_I64 = _c.c_int64
_U64 = _c.c_uint64

# name -> (restype, argtypes); mirrors include/oslo_amd.h line by line
PROTOTYPES = {
    "oslo_abi_version": (_c.c_int, []),
    "oslo_softmax_max_cols": (_c.c_int, []),
    "oslo_status_string": (_c.c_char_p, [_c.c_int]),
    "oslo_last_error": (_c.c_char_p, []),
    "oslo_softmax_causal_fwd": (
        _c.c_int, [_P, _P, _P, _c.c_float, _I64, _I64, _I64, _c.c_int, _P]),
    "oslo_softmax_causal_bwd": (
        _c.c_int, [_P, _P, _P, _c.c_float, _I64, _I64, _c.c_int, _P]),
    "oslo_softmax_causal_dropout_fwd": (
        _c.c_int, [_P, _P, _P, _P, _c.c_float, _c.c_float, _U64, _U64, _I64, _I64, _I64, _c.c_int, _P]),
    "oslo_softmax_causal_dropout_bwd": (
        _c.c_int, [_P, _P, _P, _P, _P, _c.c_float, _c.c_float, _U64, _U64, _I64, _I64, _I64, _c.c_int, _P]),
    "oslo_softmax_causal_window_fwd": (
        _c.c_int, [_P, _P, _P, _c.c_float, _I64, _I64, _I64, _I64, _c.c_int, _P]),
    "oslo_softmax_causal_window_bwd": (
        _c.c_int, [_P, _P, _P, _c.c_float, _I64, _I64, _I64, _c.c_int, _P]),
    "oslo_softmax_masked_fwd": (
        _c.c_int, [_P, _P, _P, _I64, _I64, _c.c_int, _c.c_float,
                   _I64, _I64, _I64, _I64, _c.c_int, _P]),
    "oslo_softmax_masked_bwd": (
        _c.c_int, [_P, _P, _P, _c.c_float, _I64, _I64, _c.c_int, _P]),
    "oslo_get_batch_per_block": (_c.c_int, [_c.c_int] * 4),
    "oslo_bias_gelu_fwd": (_c.c_int, [_P, _P, _P, _I64, _I64, _c.c_int, _P]),
    "oslo_colsum_workspace_bytes": (_c.c_size_t, [_I64, _I64]),
    "oslo_bias_gelu_bwd": (
        _c.c_int, [_P, _P, _P, _P, _P, _P, _I64, _I64, _c.c_int, _P]),
    "oslo_bias_gelu_bwd_static": (
        _c.c_int, [_P, _P, _P, _P, _P, _I64, _I64, _c.c_int, _P]),
    "oslo_bias_dropout_add_fwd": (
        _c.c_int, [_P, _P, _P, _P, _c.c_float, _U64, _U64, _I64, _I64, _c.c_int, _P]),
    "oslo_bias_dropout_add2_fwd": (
        _c.c_int, [_P, _P, _P, _P, _P, _c.c_float, _U64, _U64, _I64, _I64, _c.c_int, _P]),
    "oslo_bias_dropout_add_bwd": (
        _c.c_int, [_P, _P, _P, _P, _c.c_float, _U64, _U64, _I64, _I64, _c.c_int, _P]),
    "oslo_rotary_qkv": (
        _c.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I64, _I64,
                   _c.c_int, _c.c_int, _P]),
    "oslo_linear_rows_max": (_c.c_int, []),
    "oslo_linear_rows_fwd": (_c.c_int, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _c.c_int, _c.c_int, _P]),
    "oslo_linear_rows_kn_fwd": (_c.c_int, [_P, _P, _P, _P, _P, _I64, _I64, _I64, _c.c_int, _c.c_int, _P]),
    "oslo_linear_rows_fwd_multi": (
        _c.c_int, [_P, _P, _P, _P, _c.c_int, _I64, _I64, _I64, _c.c_int, _c.c_int, _P]),
    "oslo_attention_decode_workspace_bytes": (_c.c_size_t, [_I64, _I64, _I64, _c.c_int]),
    "oslo_attention_decode_fwd": (
        _c.c_int, [_P, _P, _P, _P, _P, _P, _I64, _I64, _P, _P, _I64, _I64, _c.c_float, _I64, _I64, _I64, _c.c_int,
                   _P]),
    "oslo_attention_prefill_fwd": (
        _c.c_int, [_P, _P, _P, _P, _P, _c.c_float, _I64, _I64, _I64, _I64, _I64, _c.POINTER(_c.c_int64), _c.c_int, _P]),
    "oslo_attention_prefill_fwd_lse": (
        _c.c_int, [_P, _P, _P, _P, _P, _P, _c.c_float, _c.c_float, _U64, _U64, _I64, _I64, _I64, _I64, _I64,
                   _c.POINTER(_c.c_int64), _c.c_int, _P]),
    "oslo_attention_prefill_bwd_workspace_bytes": (_c.c_size_t, [_I64, _I64, _I64]),
    "oslo_attention_prefill_bwd": (
        _c.c_int, [_P] * 11 + [_c.c_float, _c.c_float, _U64, _U64, _I64, _I64, _I64, _I64, _I64,
                               _c.POINTER(_c.c_int64), _c.c_int, _P]),
    "oslo_attention_prefill_bwd_store_bytes": (_c.c_size_t, [_I64, _I64, _I64]),
    "oslo_attention_prefill_bwd_stored": (
        _c.c_int, [_P] * 11 + [_c.c_size_t, _P, _c.c_float, _c.c_float, _U64, _U64, _I64, _I64, _I64, _I64, _I64,
                               _c.POINTER(_c.c_int64), _c.c_int, _P]),
    "oslo_ngram_repeat_block": (
        _c.c_int, [_P, _P, _I64, _I64, _I64, _I64, _c.c_int, _P]),
    "oslo_sample_idx_rows": (_I64, [_c.c_int32, _c.c_int32, _I64]),
    "oslo_build_sample_idx": (
        _c.c_int, [_P, _I64, _P, _I64, _P, _I64, _c.c_int32, _c.c_int32, _I64]),
    "oslo_build_blending_indices": (_c.c_int, [_P, _P, _P, _c.c_int32, _I64]),
    "oslo_build_mapping": (
        _I64, [_P, _I64, _c.c_int, _P, _I64, _P, _I64, _c.c_int32, _U64, _c.c_int32, _c.c_double, _c.c_int32,
               _c.c_int32]),
    "oslo_build_blocks_mapping": (
        _I64, [_P, _I64, _c.c_int, _P, _I64, _P, _I64, _P, _c.c_int32, _U64, _c.c_int32, _c.c_int32, _c.c_int]),
}

ABI_VERSION = 1

_lib = None


def load():
    """Returns the loaded library (cached). Raises EnvironmentError if it has
    not been built or does not match this binding."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise EnvironmentError(
            f"{LIB_PATH} is missing: build it with `python -m oslo_amd.build` "
            "(needs hipcc; no GPU required to build)."
        )
    try:
        lib = ctypes.CDLL(LIB_PATH)
    except OSError as e:
        raise EnvironmentError(f"could not load {LIB_PATH}: {e}") from e
    for name, (restype, argtypes) in PROTOTYPES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as e:
            raise EnvironmentError(f"{LIB_PATH} does not export {name}; rebuild it") from e
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.oslo_abi_version() != ABI_VERSION:
        raise EnvironmentError(
            f"{LIB_PATH} has ABI {lib.oslo_abi_version()}, binding expects {ABI_VERSION}; rebuild it"
        )
    _lib = lib
    return lib


def check(status):
    """Turns a non-zero status into RuntimeError, the exception type Python
    callers of the reference's native module see for rejected arguments
    (TORCH_INTERNAL_ASSERT / AT_ASSERTM, oslo/fused_kernels/fused_softmax.cu:48-53)."""
    if status != 0:
        lib = load()
        raise RuntimeError(
            f"oslo_amd: {lib.oslo_status_string(status).decode()}: {lib.oslo_last_error().decode()}"
        )
