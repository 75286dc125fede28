"""The functions of the reference's native module ``oslo_datasets``
(oslo/fused_kernels/bindings/pybind_datasets.cpp:576-592) that its data
pipeline calls, with the same names and arguments: ``build_sample_idx``
(oslo/data/datasets/dataset_causal_lm.py:289-295) and
``build_blending_indices`` (oslo/data/utils/blenders.py:65-71), and the two
sentence-span builders the module also exports, ``build_mapping`` and
``build_blocks_mapping``. They take and return numpy arrays in host memory and
run in ``liboslo_amd.so``."""

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


def _span_rows(call, docs, sizes, width):
    """Two calls of a span builder: the row count, then the rows. uint32 rows
    unless there are more than 2^32 sentences, like the reference."""
    dtype = np.uint64 if sizes.shape[0] > np.iinfo(np.uint32).max else np.uint32
    nbytes = np.dtype(dtype).itemsize
    rows = call(None, 0, nbytes)
    if rows < 0:
        _lib.check(int(rows))
    maps = np.empty((rows, width), dtype=dtype)
    got = call(_ptr(maps), rows, nbytes)
    if got < 0:
        _lib.check(int(got))
    return maps


def build_mapping(docs, sizes, num_epochs, max_num_samples, max_seq_length, short_seq_prob, seed, min_num_sent):
    """[num_samples, 3] (first sentence, one past the last, target length) of
    the samples of consecutive sentences cut from the documents ``docs`` (int64,
    sentence index where each document starts, one more entry than documents)
    with ``sizes`` tokens per sentence, over ``num_epochs`` epochs, shuffled
    (oslo/fused_kernels/bindings/pybind_datasets.cpp:346-372)."""
    docs = _array(docs, np.int64, "docs")
    sizes = _array(sizes, np.int32, "sizes")
    lib = _lib.load()
    return _span_rows(lambda maps, rows, nbytes: lib.oslo_build_mapping(
        maps, rows, nbytes, _ptr(docs), docs.shape[0], _ptr(sizes), sizes.shape[0], int(num_epochs),
        int(max_num_samples), int(max_seq_length), float(short_seq_prob), int(seed), int(min_num_sent)), docs, sizes, 3)


def build_blocks_mapping(docs, sizes, titles_sizes, num_epochs, max_num_samples, max_seq_length, seed,
                         use_one_sent_blocks):
    """[num_blocks, 4] (first sentence, one past the last, document, serial
    number of the block in its epoch) of the blocks cut from the documents, each
    leaving room for its document's title (``titles_sizes``, int32 per document),
    shuffled (oslo/fused_kernels/bindings/pybind_datasets.cpp:557-574)."""
    docs = _array(docs, np.int64, "docs")
    sizes = _array(sizes, np.int32, "sizes")
    titles_sizes = _array(titles_sizes, np.int32, "titles_sizes")
    if titles_sizes.shape[0] < docs.shape[0] - 1:
        raise RuntimeError("titles_sizes must hold one entry per document")
    lib = _lib.load()
    return _span_rows(lambda maps, rows, nbytes: lib.oslo_build_blocks_mapping(
        maps, rows, nbytes, _ptr(docs), docs.shape[0], _ptr(sizes), sizes.shape[0], _ptr(titles_sizes),
        int(num_epochs), int(max_num_samples), int(max_seq_length), int(seed), 1 if use_one_sent_blocks else 0),
        docs, sizes, 4)
