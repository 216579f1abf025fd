"""Pins for the oracle's window normalisation and masks: the reference docstring's truth tables
(flash_attn_npu/flash_attn_npu_interface.py:1484-1492) and element-wise closed forms."""
import itertools

import torch

import fa_oracle as O


def keep_matrix(sq, sk, causal, window):
    wl, wr, ic, il = O.normalize_window(window[0], window[1], causal, sk)
    m = O.masked_matrix(sq, sk, ic, il, wl, wr)
    return torch.ones(sq, sk, dtype=torch.bool) if m is None else ~m


def test_docstring_truth_table_2x5():
    expect = torch.tensor([[1, 1, 1, 1, 0], [1, 1, 1, 1, 1]], dtype=torch.bool)
    assert torch.equal(keep_matrix(2, 5, True, (-1, -1)), expect)


def test_docstring_truth_table_5x2():
    expect = torch.tensor([[0, 0], [0, 0], [0, 0], [1, 0], [1, 1]], dtype=torch.bool)
    assert torch.equal(keep_matrix(5, 2, True, (-1, -1)), expect)


def test_window_closed_form_elementwise():
    # key j visible to query i iff i + off - wl <= j <= i + off + wr (inclusive), off = sk - sq
    for sq, sk, wl, wr in itertools.product([1, 3, 7], [1, 4, 9], [-1, 0, 2, 20], [-1, 0, 1, 20]):
        if sq > sk:
            continue   # with more queries than keys the host normalisation is not mask-neutral (next test)
        got = keep_matrix(sq, sk, False, (wl, wr))
        off = sk - sq
        for i in range(sq):
            for j in range(sk):
                lo_ok = True if wl < 0 else j >= i + off - wl
                hi_ok = True if wr < 0 else j <= i + off + wr
                assert bool(got[i, j]) == (lo_ok and hi_ok), (sq, sk, wl, wr, i, j)


def test_right_window_reaching_sk_is_dropped_even_when_sq_exceeds_sk():
    # reference host behaviour (flash_api.cpp:485-490): Sq=3, Sk=1, right=1 >= Sk -> unbounded, so
    # key 0 stays visible to query 0 although the un-normalised formula (j <= i + Sk - Sq + 1) hides it
    assert torch.equal(keep_matrix(3, 1, False, (-1, 1)), torch.ones(3, 1, dtype=torch.bool))
    # and an unbounded side of a true window becomes Sk (flash_api.cpp:499-504), which with Sq > Sk hides
    # key 0 from query 0: visible iff i - 2 <= 0 <= i - 2 + 1
    assert torch.equal(keep_matrix(3, 1, False, (0, -1)), torch.tensor([[False], [True], [True]]))


def test_normalize_known_answers():
    # (wl, wr, causal, max_sk) -> (wl, wr, is_causal, is_local)   flash_api.cpp:483-505
    assert O.normalize_window(-1, -1, False, 100) == (-1, -1, False, False)
    assert O.normalize_window(-1, -1, True, 100) == (-1, 0, True, False)
    assert O.normalize_window(100, 100, False, 100) == (-1, -1, False, False)     # window >= Sk is no window
    assert O.normalize_window(200, 0, False, 100) == (-1, 0, True, False)         # left covers all + right 0 is causal
    assert O.normalize_window(5, -1, False, 100) == (5, 100, False, True)         # infinite side := max Sk
    assert O.normalize_window(-1, 7, False, 100) == (100, 7, False, True)
    assert O.normalize_window(5, 3, True, 100) == (5, 0, False, True)             # causal forces right = 0


def test_covering_window_equals_no_window_and_causal_equivalence():
    for sq, sk in [(1, 9), (4, 9), (9, 4)]:
        full = torch.ones(sq, sk, dtype=torch.bool)
        assert torch.equal(keep_matrix(sq, sk, False, (sk, sk)), full)
        assert torch.equal(keep_matrix(sq, sk, False, (sk + 5, -1)), full)
        assert torch.equal(keep_matrix(sq, sk, True, (-1, -1)), keep_matrix(sq, sk, False, (-1, 0)))
        assert torch.equal(keep_matrix(sq, sk, True, (sk, 5)), keep_matrix(sq, sk, True, (-1, -1)))


def test_decode_window_is_last_w_keys():
    # Sq = 1, window (W-1, 0): exactly the last W keys
    for sk, w in [(10, 3), (10, 10), (5, 9), (300, 64)]:
        k = keep_matrix(1, sk, False, (w - 1, 0))[0]
        expect = torch.zeros(sk, dtype=torch.bool)
        expect[max(0, sk - w):] = True
        assert torch.equal(k, expect)


def test_backward_golden_rule_gives_same_masks():
    # tests/fa_small_op_golden.py:21-32 normalises with wl >= Sk-1, wr >= Sq-1; same mask as the forward rule
    for sq, sk, wl, wr, causal in itertools.product([1, 3, 6], [2, 6], [-1, 0, 1, 4, 5, 9], [-1, 0, 2, 5, 9], [False, True]):
        a, b = wl, wr
        if a >= sk - 1:
            a = -1
        if b >= sq - 1:
            b = -1
        if causal:
            b = 0
        off = sk - sq
        i = torch.arange(sq)[:, None]
        j = torch.arange(sk)[None, :]
        keep = torch.ones(sq, sk, dtype=torch.bool)
        if a >= 0:
            keep &= j >= i + off - a
        if b >= 0:
            keep &= j <= i + off + b
        # the backward rule drops wr when wr >= Sq-1, which is only mask-neutral for sq <= sk
        if sq <= sk:
            assert torch.equal(keep_matrix(sq, sk, causal, (wl, wr)), keep), (sq, sk, wl, wr, causal)
