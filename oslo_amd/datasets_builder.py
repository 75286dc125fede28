"""The functions of the reference's native module ``oslo_datasets``
(oslo/fused_kernels/bindings/pybind_datasets.cpp:576-592) that its data
pipeline calls, with the same names and arguments: ``build_sample_idx``
(oslo/data/datasets/dataset_causal_lm.py:289-295) and
``build_blending_indices`` (oslo/data/utils/blenders.py:65-71). They take and
return numpy arrays in host memory and run in ``liboslo_amd.so``."""

import ctypes

import numpy as np

from . import _lib


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


def _array(a, dtype, what):
    if not isinstance(a, np.ndarray) or a.dtype != dtype or a.ndim != 1:
        raise RuntimeError(f"{what} must be a 1-D numpy array of {np.dtype(dtype).name}")
    return np.ascontiguousarray(a)


def build_sample_idx(sizes, doc_idx, seq_length, num_epochs, tokens_per_epoch):
    """int32 [num_samples + 1, 2]: for every sample the position in ``doc_idx``
    and the offset inside that document where it starts."""
    sizes = _array(sizes, np.int32, "sizes")
    doc_idx = _array(doc_idx, np.int32, "doc_idx")
    lib = _lib.load()
    rows = lib.oslo_sample_idx_rows(int(seq_length), int(num_epochs), int(tokens_per_epoch))
    if rows < 0:
        raise RuntimeError("build_sample_idx: needs seq_length > 1, num_epochs > 0, tokens_per_epoch > 1")
    sample_idx = np.empty((rows, 2), dtype=np.int32)
    _lib.check(lib.oslo_build_sample_idx(
        _ptr(sample_idx), rows, _ptr(sizes), sizes.shape[0], _ptr(doc_idx), doc_idx.shape[0],
        int(seq_length), int(num_epochs), int(tokens_per_epoch)))
    return sample_idx


def build_blending_indices(dataset_index, dataset_sample_index, weights, num_datasets, size):
    """Fills ``dataset_index`` (int32 [size]) and ``dataset_sample_index``
    (int64 [size]) in place so that the mix of datasets follows ``weights``."""
    weights = np.ascontiguousarray(np.asarray(weights, dtype=np.float64))
    if weights.ndim != 1 or weights.shape[0] < num_datasets:
        raise RuntimeError("weights must hold one number per dataset")
    for a, dtype, what in ((dataset_index, np.int32, "dataset_index"),
                           (dataset_sample_index, np.int64, "dataset_sample_index")):
        if not isinstance(a, np.ndarray) or a.dtype != dtype or a.ndim != 1 or a.shape[0] < size \
                or not a.flags.c_contiguous or not a.flags.writeable:
            raise RuntimeError(f"{what} must be a writable contiguous 1-D {np.dtype(dtype).name} array of "
                               f"at least {size} elements")
    _lib.check(_lib.load().oslo_build_blending_indices(
        _ptr(dataset_index), _ptr(dataset_sample_index), _ptr(weights), int(num_datasets), int(size)))
