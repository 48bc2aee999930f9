"""The oracle's group padding against the reference's own sequence, written out row by row: split the permuted
tokens per expert, append zero rows up to the alignment, concatenate (experts.py:196-209; undone at :262-264)."""

import numpy as np
import pytest

from oracle import mx_oracle as o


def _reference_sequence(x, lens, align):
    rows, padded = [], []
    at = 0
    for n in lens:
        for i in range(n):
            rows.append(x[at + i])
        at += n
        m = -(-n // align) * align
        for _ in range(m - n):
            rows.append(np.zeros_like(x[0]))
        padded.append(m)
    out = np.stack(rows) if rows else np.zeros((0,) + x.shape[1:], x.dtype)
    return out, padded


@pytest.mark.parametrize("lens", [[5, 0, 33, 64], [0, 0, 0], [32], [1] * 9, [31, 33, 0, 1, 0]])
@pytest.mark.parametrize("align", [32, 16, 1, 7])
def test_pad_groups_is_the_references_sequence(lens, align):
    rng = np.random.default_rng(sum(lens) + align)
    x = rng.integers(1, 1 << 16, size=(sum(lens), 6), dtype=np.uint16)     # no zero rows among the real ones
    want, padded = _reference_sequence(x, lens, align)
    got, got_lens = o.pad_groups(x, lens, align)
    assert got.shape == want.shape and np.array_equal(got, want)
    assert got_lens.tolist() == padded
    assert np.array_equal(o.unpad_groups(got, lens, align), x)


def test_worst_case_buffer_counts_its_tail_into_the_last_group():
    lens, align = [5, 0, 33, 0], 32
    x = np.arange(1, 38 * 3 + 1, dtype=np.int32).reshape(38, 3)
    exact, exact_lens = o.pad_groups(x, lens, align)
    bound = o.padded_rows_bound(38, 4, align)
    assert bound == (38 + 4 * 31) // 32 * 32 and bound >= exact.shape[0]
    big, big_lens = o.pad_groups(x, lens, align, bound)
    assert np.array_equal(big[: exact.shape[0]], exact) and not big[exact.shape[0]:].any()
    assert big_lens.sum() == bound and big_lens[:-1].tolist() == exact_lens[:-1].tolist()
    assert np.array_equal(o.unpad_groups(big, lens, align), x)
    # the bound is attained: every group one row over a multiple
    assert sum(-(-n // 32) * 32 for n in [33, 1, 65, 1]) == o.padded_rows_bound(100, 4, 32)
    # rows asked for behind the counts come back as zeros
    assert not o.unpad_groups(big, lens, align, rows=40)[38:].any()
