"""Index builders of the data pipeline (host code in liboslo_amd.so): against
the oracle, against what the definitions fix (sample k starts at token
k*seq_length of the document stream; blending keeps every dataset within one
sample of its share), and against the reference's own C++ module where
oracle/_ref holds a build of it."""

import importlib.util
import os

import numpy as np
import pytest

from oracle import oslo_oracle as orc
from oracle.build_ref import output_path
from oslo_amd.fused_kernels_utils import get_datasets_builder


def reference_module():
    path = output_path()
    if not os.path.exists(path):
        return None
    import torch  # noqa: F401  (the module links against torch's libraries)

    spec = importlib.util.spec_from_file_location("oslo_datasets", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def corpus(seed, num_docs, max_len, epochs=1, with_empty=False):
    rng = np.random.default_rng(seed)
    sizes = rng.integers(0 if with_empty else 1, max_len + 1, num_docs).astype(np.int32)
    sizes[rng.integers(0, num_docs)] = max_len            # at least one non-empty document
    doc_idx = np.concatenate([rng.permutation(num_docs) for _ in range(epochs)]).astype(np.int32)
    return sizes, doc_idx, int(sizes.sum())


CASES = [  # seed, num_docs, max_len, seq_length, epochs, with_empty
    (0, 5, 9, 4, 1, False),
    (1, 50, 30, 7, 1, False),
    (2, 200, 5, 16, 1, True),       # many documents per sample, some empty
    (3, 40, 3000, 128, 2, False),   # many samples per document, two epochs
    (4, 1, 100, 2, 1, False),
    (5, 300, 64, 64, 3, True),
]


@pytest.mark.parametrize("case", CASES)
def test_build_sample_idx(case):
    seed, num_docs, max_len, seq_length, epochs, with_empty = case
    sizes, doc_idx, tokens = corpus(seed, num_docs, max_len, epochs, with_empty)
    got = get_datasets_builder().build_sample_idx(sizes, doc_idx, seq_length, epochs, tokens)
    want = orc.build_sample_idx(sizes, doc_idx, seq_length, epochs, tokens)
    assert got.dtype == np.int32 and got.shape == want.shape
    assert np.array_equal(got, want)
    # what the definition fixes: sample k starts at token k*seq_length of the stream
    starts = np.concatenate([[0], np.cumsum(sizes[doc_idx].astype(np.int64))])
    pos = np.arange(got.shape[0], dtype=np.int64) * seq_length
    at = np.searchsorted(starts, pos, side="right") - 1
    assert np.array_equal(got[:, 0], at)
    assert np.array_equal(got[:, 1], pos - starts[at])
    ref = reference_module()
    if ref is not None:
        assert np.array_equal(got, ref.build_sample_idx(sizes, doc_idx, seq_length, epochs, tokens))


def test_build_sample_idx_rejects_what_the_reference_would_read_out_of_bounds():
    b = get_datasets_builder()
    sizes = np.array([4, 4], dtype=np.int32)
    with pytest.raises(RuntimeError, match="too few tokens"):
        b.build_sample_idx(sizes, np.array([0, 1], dtype=np.int32), 4, 1, 100)
    with pytest.raises(RuntimeError, match="outside"):
        b.build_sample_idx(sizes, np.array([0, 7], dtype=np.int32), 4, 1, 8)
    with pytest.raises(RuntimeError, match="seq_length"):
        b.build_sample_idx(sizes, np.array([0, 1], dtype=np.int32), 1, 1, 8)
    with pytest.raises(RuntimeError, match="int32"):
        b.build_sample_idx(sizes.astype(np.int64), np.array([0, 1], dtype=np.int32), 4, 1, 8)


@pytest.mark.parametrize("weights,size", [
    ([0.5, 0.3, 0.2], 10),
    ([0.5, 0.3, 0.2], 1000),
    ([1.0], 17),
    ([0.25, 0.25, 0.25, 0.25], 101),      # ties go to the lowest dataset
    ([0.9, 0.05, 0.03, 0.02], 5000),
    ([0.0, 1.0], 50),
    ([0.3, 0.7], 0),
])
def test_build_blending_indices(weights, size):
    n = len(weights)
    w = np.array(weights, dtype=np.float64)
    di = np.full(size, -1, dtype=np.int32)
    dsi = np.full(size, -1, dtype=np.int64)
    get_datasets_builder().build_blending_indices(di, dsi, w, n, size)
    want_di, want_dsi = orc.build_blending_indices(w, n, size)
    assert np.array_equal(di, want_di) and np.array_equal(dsi, want_dsi)
    # what the definition fixes: running counts per dataset, shares within one sample of the weights
    for d in range(n):
        where = np.flatnonzero(di == d)
        assert np.array_equal(dsi[where], np.arange(where.size))
        if size:
            assert abs(where.size - w[d] * size) <= 1.0 + 1e-9
    ref = reference_module()
    if ref is not None and size:
        rdi, rdsi = np.zeros(size, dtype=np.int32), np.zeros(size, dtype=np.int64)
        ref.build_blending_indices(rdi, rdsi, w, n, size)
        assert np.array_equal(di, rdi) and np.array_equal(dsi, rdsi)


def test_build_blending_indices_argument_errors():
    b = get_datasets_builder()
    with pytest.raises(RuntimeError, match="dataset_index"):
        b.build_blending_indices(np.zeros(3, dtype=np.int64), np.zeros(3, dtype=np.int64), [1.0], 1, 3)
    with pytest.raises(RuntimeError, match="at least"):
        b.build_blending_indices(np.zeros(2, dtype=np.int32), np.zeros(3, dtype=np.int64), [1.0], 1, 3)
    with pytest.raises(RuntimeError, match="weights"):
        b.build_blending_indices(np.zeros(3, dtype=np.int32), np.zeros(3, dtype=np.int64), [1.0], 2, 3)


def test_reference_build_is_used_when_present():
    """Says in the test report whether the comparisons above included the
    reference's own module."""
    if reference_module() is None:
        pytest.skip("oracle/_ref holds no build of the reference's pybind_datasets.cpp "
                    "(python oracle/build_ref.py makes it where /root/reference exists)")
    ref = reference_module()
    sizes, doc_idx, tokens = corpus(9, 64, 40)
    assert np.array_equal(ref.build_sample_idx(sizes, doc_idx, 8, 1, tokens),
                          orc.build_sample_idx(sizes, doc_idx, 8, 1, tokens))
