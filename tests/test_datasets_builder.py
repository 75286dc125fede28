"""Index builders of the data pipeline (host code in liboslo_amd.so): against
the oracle, against what the definitions fix (sample k starts at token
k*seq_length of the document stream; blending keeps every dataset within one
sample of its share; a span is the shortest run of sentences that reaches its
target), and against the reference's own C++ module where
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


def sentence_corpus(seed, num_docs, max_sents, max_tokens, long_every=0):
    """docs (int64 [num_docs + 1]) and sizes (int32 per sentence); some documents
    are empty or have one sentence; every `long_every`-th holds a sentence of
    more than 512 tokens."""
    rng = np.random.default_rng(seed)
    counts = rng.integers(0, max_sents + 1, num_docs)
    docs = np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)
    sizes = rng.integers(1, max_tokens + 1, int(docs[-1])).astype(np.int32)
    if long_every:
        for d in range(0, num_docs, long_every):
            if counts[d]:
                sizes[docs[d] + rng.integers(0, counts[d])] = 513 + d
    return docs, sizes


def test_mersenne_twisters_of_the_oracle():
    """[rand.predef] of the C++ standard: the 10000th output of the default
    engines."""
    for width, want in ((32, 4123659995), (64, 9981545732273789042)):
        gen = orc.MersenneTwister(5489, width)
        for _ in range(9999):
            gen()
        assert gen() == want


def greedy_spans(docs, sizes, target_of, min_num_sent, min_behind, long_from):
    """The cutting said another way, for a fixed target per document: a span
    ends at the first sentence where the running token count (from the span's
    start) reaches the target, never before min_num_sent sentences are in it,
    and only while at least min_behind sentences would be left; what is left
    when that fails goes into the document's last span."""
    out = []
    for d in range(len(docs) - 1):
        first, last = int(docs[d]), int(docs[d + 1])
        n = last - first
        if n < min_num_sent or (n >= long_from and (sizes[first:last] > 512).any()):
            continue
        csum = np.concatenate([[0], np.cumsum(sizes[first:last].astype(np.int64))])
        start = 0
        while start < n:
            reach = int(np.searchsorted(csum, csum[start] + target_of(d), side="left"))  # csum[reach] >= ...
            end = max(reach, start + max(min_num_sent, 1))
            if end > n - min_behind:
                end = n
            out.append((first + start, first + end, d))
            start = end
    return out


MAPPING_CASES = [  # seed, num_docs, max_sents, max_tokens, epochs, max_seq_length, short_seq_prob, min_num_sent, long_every
    (1, 20, 6, 40, 1, 64, 0.0, 2, 0),
    (2, 200, 12, 100, 3, 128, 0.1, 2, 7),
    (3, 50, 30, 20, 2, 16, 0.4, 1, 0),      # 1/0.4 = 2.5 rounds to 3, not to 2
    (4, 100, 8, 200, 2, 512, 1.0, 3, 5),    # every sample short
    (5, 1, 1, 10, 1, 8, 0.0, 2, 0),         # nothing to cut
    (6, 300, 5, 300, 4, 256, 0.05, 2, 3),
]


@pytest.mark.parametrize("case", MAPPING_CASES)
def test_build_mapping(case):
    seed, num_docs, max_sents, max_tokens, epochs, max_len, prob, min_sent, long_every = case
    docs, sizes = sentence_corpus(seed, num_docs, max_sents, max_tokens, long_every)
    args = (docs, sizes, epochs, 10**9, max_len, prob, 1234 + seed, min_sent)
    got = get_datasets_builder().build_mapping(*args)
    want = orc.build_mapping(*args)
    assert got.dtype == np.uint32 and got.shape == want.shape and got.shape[1] == 3
    assert np.array_equal(got, want)
    # every row: a run of sentences inside one document, target in [2, max_len];
    # per epoch the rows tile each document they come from
    rows = got[np.lexsort((got[:, 1], got[:, 0]))].astype(np.int64)
    assert ((rows[:, 2] >= 2) & (rows[:, 2] <= max_len)).all()
    doc_of = np.searchsorted(docs, rows[:, 0], side="right") - 1
    assert (rows[:, 1] > rows[:, 0]).all() and (rows[:, 1] <= docs[doc_of + 1]).all()
    covered = np.zeros(len(sizes), dtype=np.int64)
    for a, b, _ in rows:
        covered[a:b] += 1
    assert set(np.unique(covered)) <= {0, epochs}
    if prob == 0.0:
        spans = greedy_spans(docs, sizes, lambda d: max_len, min_sent, 2, 2)
        want_rows = sorted((a, b, max_len) for a, b, _ in spans) * 1
        assert sorted(map(tuple, rows.tolist())) == sorted(want_rows * epochs)
    ref = reference_module()
    if ref is not None:
        assert np.array_equal(got, ref.build_mapping(*args))


def test_build_mapping_stops_starting_epochs_at_max_num_samples():
    docs, sizes = sentence_corpus(11, 40, 6, 50)
    b = get_datasets_builder()
    one = b.build_mapping(docs, sizes, 1, 10**9, 64, 0.0, 7, 2)
    many = b.build_mapping(docs, sizes, 5, len(one) + 1, 64, 0.0, 7, 2)   # a second epoch starts, a third does not
    assert len(many) == 2 * len(one)
    assert np.array_equal(many, orc.build_mapping(docs, sizes, 5, len(one) + 1, 64, 0.0, 7, 2))
    ref = reference_module()
    if ref is not None:
        assert np.array_equal(many, ref.build_mapping(docs, sizes, 5, len(one) + 1, 64, 0.0, 7, 2))


BLOCK_CASES = [  # seed, num_docs, max_sents, max_tokens, epochs, max_seq_length, one_sent_blocks, long_every
    (1, 20, 6, 40, 1, 64, False, 0),
    (2, 200, 12, 100, 3, 128, True, 7),
    (3, 50, 30, 20, 2, 48, False, 0),
    (4, 100, 8, 200, 2, 288, True, 5),
    (5, 1, 1, 10, 1, 40, False, 0),
]


@pytest.mark.parametrize("case", BLOCK_CASES)
def test_build_blocks_mapping(case):
    seed, num_docs, max_sents, max_tokens, epochs, max_len, one_sent, long_every = case
    docs, sizes = sentence_corpus(seed, num_docs, max_sents, max_tokens, long_every)
    titles = np.random.default_rng(seed).integers(1, 32, num_docs).astype(np.int32)
    args = (docs, sizes, titles, epochs, 10**9, max_len, 99 + seed, one_sent)
    got = get_datasets_builder().build_blocks_mapping(*args)
    want = orc.build_blocks_mapping(*args)
    assert got.dtype == np.uint32 and got.shape == want.shape and got.shape[1] == 4
    assert np.array_equal(got, want)
    least = 1 if one_sent else 2
    spans = greedy_spans(docs, sizes, lambda d: max_len - int(titles[d]), least, least, least)
    rows = sorted(map(tuple, got[:, :3].astype(np.int64).tolist()))
    assert rows == sorted(spans * epochs)
    # block ids: 0 .. blocks-per-epoch - 1 in document order, every epoch again
    per_epoch = len(spans)
    if per_epoch:
        order = np.lexsort((got[:, 0], got[:, 3]))
        assert np.array_equal(got[order, 3], np.repeat(np.arange(per_epoch), epochs))
        first_epoch = got[order][::epochs]
        assert np.array_equal(first_epoch[:, 0], np.array(sorted(a for a, _, _ in spans)))
    ref = reference_module()
    if ref is not None:
        assert np.array_equal(got, ref.build_blocks_mapping(*args))


def test_span_builders_reject_bad_input():
    b = get_datasets_builder()
    docs, sizes = sentence_corpus(3, 10, 4, 20)
    with pytest.raises(RuntimeError, match="ascending"):
        b.build_mapping(docs[::-1].copy(), sizes, 1, 100, 64, 0.0, 1, 2)
    with pytest.raises(RuntimeError, match="ascending"):
        b.build_mapping(docs + 1, sizes, 1, 100, 64, 0.0, 1, 2)        # runs past the last sentence
    with pytest.raises(RuntimeError, match="seed"):
        b.build_mapping(docs, sizes, 1, 100, 64, 0.0, 0, 2)
    with pytest.raises(RuntimeError, match="short_seq_prob"):
        b.build_mapping(docs, sizes, 1, 100, 64, 1.5, 1, 2)
    with pytest.raises(RuntimeError, match="titles_sizes"):
        b.build_blocks_mapping(docs, sizes, np.zeros(3, dtype=np.int32), 1, 100, 64, 1, False)


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
