"""Pins the oracle's integer / boolean functions against the reference's known answers
and against a per-element brute force of the mask predicate."""

import random

import torch

import oracle
from tests.golden import known_answers as KA


def test_cu_seqlens_with_reset():
    out = oracle.get_cumulative_seq_lengths(torch.tensor(KA.TOKEN_IDS))
    assert out.dtype == torch.int32
    assert out.tolist() == KA.CU_WITH_RESET


def test_cu_seqlens_without_reset():
    out = oracle.get_cumulative_seq_lengths(torch.tensor(KA.TOKEN_IDS), reset_attention_mask=False)
    assert out.dtype == torch.int32
    assert out.tolist() == KA.CU_WITHOUT_RESET


def test_position_ids():
    ids = torch.tensor(KA.TOKEN_IDS)
    assert oracle.get_position_ids(ids, True).tolist() == KA.POSITION_IDS_WITH_RESET
    assert oracle.get_position_ids(ids, False).tolist() == KA.POSITION_IDS_WITHOUT_RESET
    assert oracle.get_position_ids(ids, True).dtype == torch.int64


def test_padding_round_trip():
    cu = torch.tensor(KA.PADDING_INPUT)
    padded = oracle.add_cumulative_seq_lengths_padding(cu, KA.PADDING_PAD_TO)
    assert padded.tolist() == KA.PADDING_EXPECTED
    assert oracle.add_cumulative_seq_lengths_padding(cu, 4).tolist() == KA.PADDING_INPUT
    assert oracle.remove_cumulative_seq_lengths_padding(padded).tolist() == KA.PADDING_INPUT


def test_dense_mask_known_answers():
    cu = torch.tensor(KA.MASK_CU_SEQLENS)
    for causal, allowed in ((True, KA.MASK_ALLOWED_CAUSAL), (False, KA.MASK_ALLOWED_BIDIRECTIONAL)):
        m = oracle.cumulative_seq_lengths_to_dense_attention_mask(cu, KA.MASK_SEQ_LEN, causal)
        assert m.shape == (3, 1, 6, 6) and m.dtype == torch.bool
        assert torch.equal(m[:, 0], ~torch.tensor(allowed, dtype=torch.bool))
    assert oracle.get_max_seq_length(cu) == KA.MASK_MAX_SEQ_LENGTH


def _random_cu(rng, b, s):
    cu = {0}
    for item in range(b):
        for _ in range(rng.randint(0, 4)):
            cu.add(item * s + rng.randint(1, s - 1))
        cu.add((item + 1) * s)
    return sorted(cu)


def test_dense_mask_brute_force():
    rng = random.Random(0)
    for _ in range(25):
        b, s = rng.randint(1, 3), rng.randint(2, 17)
        cu = _random_cu(rng, b, s)
        doc = [0] * (b * s)
        for d, (lo, hi) in enumerate(zip(cu[:-1], cu[1:])):
            for t in range(lo, hi):
                doc[t] = d
        for causal in (True, False):
            m = oracle.cumulative_seq_lengths_to_dense_attention_mask(torch.tensor(cu, dtype=torch.int32), s, causal)
            assert m.shape == (b, 1, s, s)
            for item in range(b):
                for i in range(s):
                    for j in range(s):
                        masked = doc[item * s + i] != doc[item * s + j] or (causal and j > i)
                        assert bool(m[item, 0, i, j]) == masked


def test_decode_mask_is_single_false():
    # a one-token query gives a [1,1,1,1] all-False mask that broadcasts over every cached key
    m = oracle.cumulative_seq_lengths_to_dense_attention_mask(torch.tensor([0, 1], dtype=torch.int32), 1, True)
    assert m.shape == (1, 1, 1, 1) and not bool(m.any())


def test_cu_seqlens_random_against_python_loop():
    g = torch.Generator().manual_seed(1)
    for _ in range(10):
        ids = torch.randint(0, 4, (3, 9), generator=g)
        expect = [0]
        for r in range(3):
            for c in range(9):
                if int(ids[r, c]) == 0 or c == 8:
                    expect.append(r * 9 + c + 1)
        assert oracle.get_cumulative_seq_lengths(ids).tolist() == expect
        # position ids restart exactly where a new document starts
        pos = oracle.get_position_ids(ids)
        cu = set(expect)
        for r in range(3):
            for c in range(9):
                assert (int(pos[r, c]) == 0) == ((r * 9 + c) in cu or c == 0)
