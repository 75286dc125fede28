"""Repeated n-gram blocking: the oracle against the installed transformers'
NoRepeatNGramLogitsProcessor (an independent implementation of the same rule)
and a hand-worked case; the HIP kernel against the oracle."""

import pytest
import torch

from oracle import oslo_oracle as orc


def random_tokens(rows, length, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (rows, length), generator=g)


def oracle_scores(tokens, scores, n):
    out = scores.clone()
    for r in range(tokens.shape[0]):
        for t in orc.ngram_banned_tokens(tokens[r].tolist(), n):
            out[r, t] = float("-inf")
    return out


def test_oracle_hand_worked_case():
    # "a b c a b" with n = 3: the last two tokens (a b) occurred at position 0, followed by c
    assert orc.ngram_banned_tokens([1, 2, 3, 1, 2], 3) == {3}
    assert orc.ngram_banned_tokens([1, 2, 3, 1, 2], 2) == {3}          # "2" was followed by 3
    assert orc.ngram_banned_tokens([1, 2, 3, 1, 2], 1) == {1, 2, 3}    # every token seen
    assert orc.ngram_banned_tokens([1, 2, 3, 1, 2], 4) == set()
    assert orc.ngram_banned_tokens([5, 5, 5, 5], 2) == {5}
    assert orc.ngram_banned_tokens([7], 3) == set()                     # too short for any trigram
    assert orc.ngram_banned_tokens([], 1) == set()


@pytest.mark.parametrize("n", [1, 2, 3, 4])
def test_oracle_matches_transformers_processor(n):
    from transformers.generation.logits_process import NoRepeatNGramLogitsProcessor

    proc = NoRepeatNGramLogitsProcessor(n)
    for length in (1, 2, 3, 5, 17, 40):
        tokens = random_tokens(6, length, 7, seed=length * 10 + n)   # tiny vocabulary: many repeats
        scores = torch.zeros(6, 7)
        want = proc(tokens, scores.clone())
        got = oracle_scores(tokens, scores, n)
        assert torch.equal(torch.isinf(want), torch.isinf(got)), (n, length)


@pytest.mark.parametrize("n", [1, 2, 3, 4])
def test_processor_host_branch_matches_transformers_and_oracle(n):
    """Host tensors take the processor's host branch, as in the reference
    (oslo/fused_kernels_utils.py:505-517): same bans as the installed
    transformers' processor and as the oracle, written into `scores` in place,
    the other scores untouched."""
    from transformers.generation.logits_process import NoRepeatNGramLogitsProcessor

    from oslo_amd.fused_kernels_utils import FusedNoRepeatNGramLogitsProcessor

    for length in (1, 2, 3, 5, 17, 40):
        tokens = random_tokens(6, length, 7, seed=length * 10 + n)
        scores = torch.randn(6, 7, generator=torch.Generator().manual_seed(length))
        want = NoRepeatNGramLogitsProcessor(n)(tokens, scores.clone())
        mine = scores.clone()
        got = FusedNoRepeatNGramLogitsProcessor(n, 3, 2)(tokens, mine)
        assert got.data_ptr() == mine.data_ptr()
        assert torch.equal(got, want), (n, length)
        assert torch.equal(got, oracle_scores(tokens, scores, n)), (n, length)


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 2, 3, 5])
@pytest.mark.parametrize("length", [1, 2, 4, 33, 257, 1500])
def test_kernel_matches_oracle(n, length):
    from oslo_amd import kernels
    from oslo_amd.fused_kernels_utils import FusedNoRepeatNGramLogitsProcessor

    bsz, beams, vocab = 3, 4, 11
    rows = bsz * beams
    tokens = random_tokens(rows, length, vocab, seed=n * 1000 + length)
    scores = torch.randn(rows, vocab, generator=torch.Generator().manual_seed(1))
    want = oracle_scores(tokens, scores, n)
    got = FusedNoRepeatNGramLogitsProcessor(n, bsz, beams)(tokens.cuda(), scores.cuda())
    assert got.dtype == torch.float32
    assert torch.equal(got.cpu(), want)          # bit-exact: untouched scores unchanged, banned ones -inf
    # a token buffer longer than the generated prefix (max_predict_len > step + 1)
    padded = torch.cat([tokens, torch.full((rows, 9), 3)], dim=1).cuda()
    sc = scores.cuda()
    out = kernels.ngram_repeat_block_forward(padded, sc, bsz, length - 1, beams, n)
    assert out.data_ptr() == sc.data_ptr() and torch.equal(out.cpu(), want)


@pytest.mark.gpu
def test_kernel_argument_errors():
    from oslo_amd import kernels
    from oslo_amd.fused_kernels_utils import FusedNoRepeatNGramLogitsProcessor

    tok = torch.zeros(2, 5, dtype=torch.int64, device="cuda")
    sc = torch.zeros(2, 7, device="cuda")
    with pytest.raises(RuntimeError):
        kernels.ngram_repeat_block_forward(tok, sc, 1, 5, 2, 2)          # step + 1 > tokens per row
    with pytest.raises(RuntimeError):
        kernels.ngram_repeat_block_forward(tok.int(), sc, 1, 4, 2, 2)    # not int64
    with pytest.raises(RuntimeError):
        kernels.ngram_repeat_block_forward(tok, sc, 1, 4, 3, 2)          # rows != bsz * beam
    with pytest.raises(RuntimeError):
        FusedNoRepeatNGramLogitsProcessor(2, 1, 2)(tok.cpu(), sc)        # one on the host, one on the device
    with pytest.raises(ValueError):
        FusedNoRepeatNGramLogitsProcessor(0, 1, 2)
    # token ids outside the vocabulary are ignored, not written
    bad = torch.tensor([[9, 1, 9, 1]], dtype=torch.int64, device="cuda")
    out = kernels.ngram_repeat_block_forward(bad, torch.zeros(1, 3, device="cuda"), 1, 3, 1, 2)
    assert torch.isfinite(out).all()                                     # "1" is followed by 9 >= vocab
