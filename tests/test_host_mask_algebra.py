"""Product-side block-mask algebra (ultraattn_amd.masks: complicate, simplify, merge_blocks,
BsaRepr) against the numpy oracle and the reference-held mask strings: bit-exact."""
import json
import os

import numpy as np
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from oracle import tilelist_oracle as to
from tests.conftest import GOLDEN
from ultraattn_amd import masks


def oracle_simplify(table):
    """The reference's schedule (search_algo/bsa_config.py:162-175) on top of the oracle's
    single coarsening step: prime factors of gcd(rows, cols) ascending, each as often as it
    divides, a factor is dropped at its first failure."""
    t = np.array(table, dtype=np.uint8)
    g = int(np.gcd(*t.shape))
    p = 2
    while g > 1 and p <= g:
        if g % p == 0:
            e = 0
            while g % p == 0:
                g //= p
                e += 1
            for _ in range(e):
                c = to.simplify_once(t, p)
                if c is None:
                    break
                t = c
        p += 1
    return t


tables = st.integers(1, 6).flatmap(lambda r: st.integers(1, 6).flatmap(lambda c: st.lists(
    st.integers(0, 2), min_size=r * c, max_size=r * c).map(lambda v: np.array(v, np.uint8).reshape(r, c))))


@settings(max_examples=120, deadline=None)
@given(tables, st.integers(1, 4))
def test_complicate_equals_oracle_and_simplify_inverts_it(t, rate):
    fine = masks.complicate(t, rate)
    assert fine.dtype == np.uint8 and np.array_equal(fine, to.complicate(t, rate))
    coarse = masks.simplify(fine)
    assert np.array_equal(coarse, oracle_simplify(fine))
    if t.shape[0] == t.shape[1]:
        # the coarsest form of a refined square table is the coarsest form of the table itself
        # (rectangular tables coarsen by the gcd's factors only, which the refinement enlarges)
        assert np.array_equal(coarse, masks.simplify(t))
    # refining the coarsest form back gives the fine table again
    assert np.array_equal(masks.complicate(coarse, fine.shape[0] // coarse.shape[0]), fine)


@settings(max_examples=80, deadline=None)
@given(tables)
def test_simplify_equals_oracle_on_raw_tables(t):
    assert np.array_equal(masks.simplify(t), oracle_simplify(t))


@pytest.mark.parametrize("k", [1, 2, 3, 4])
def test_merge_blocks(k):
    for ty in (masks.EMPTY, masks.FULL, masks.CAUSAL):
        sub = to.complicate_block(ty, k)
        want = ty if (k > 1 or ty != masks.CAUSAL) else masks.CAUSAL
        assert masks.merge_blocks(sub) == want
    if k > 1:
        bad = to.complicate_block(masks.FULL, k)
        bad[0, k - 1] = masks.EMPTY
        assert masks.merge_blocks(bad) is None
        ok, succeeded = masks.simplify_by_k(bad, k)
        assert not succeeded and np.array_equal(ok, bad)


def test_reference_strings_are_their_own_coarsest_form():
    """The strings the reference plots with (plot/e2e_pick.py:65-72) are BSA_Repr.__str__ output,
    i.e. block_table_raw: parsing, refining and coarsening must reproduce them exactly."""
    ref = json.load(open(os.path.join(GOLDEN, "reference_data.json")))["bsa_reprs"]["strings"]
    for s in ref:
        t = to.parse_bsa_repr(s)
        assert str(masks.BsaRepr(t)) == s
        for rate in (2, 3, 4):
            assert str(masks.BsaRepr(masks.complicate(t, rate))) == s


def test_sub_repr_names_the_tile_type():
    """search_algo/dependent_graph.py:253-258: at the kernel level the sub-representation of one
    (row, column) chunk is [[1]] FULL or [[2]] CAUSAL (or empty), whatever the split."""
    t = masks.config_strided(16, 4, 8)
    r = masks.BsaRepr(t)
    assert r.check_causal() and not r.check_full() and not r.check_empty()
    fine = to.complicate(r.block_table_raw, 4)
    n = r.block_table_raw.shape[0]
    for k in range(0, 4 * n, 5):
        for l in range(0, 4 * n, 3):
            sub = r.create_sub_bsa_repr([4 * n, 4 * n], [[k], [l]])
            assert sub.block_table_raw.shape == (1, 1) and int(sub.block_table_raw[0, 0]) == int(fine[k, l])
            assert sub.check_empty() == (fine[k, l] == 0) and sub.check_full() == (fine[k, l] == 1)
            assert sub.check_causal() == (fine[k, l] == 2)
    # a split coarser than the raw table selects groups of raw rows / columns
    half = r.create_sub_bsa_repr([n // 2, n // 2], [[1], [0, 1]])
    assert np.array_equal(half.block_table, r.block_table_raw[np.ix_([2, 3], [0, 1, 2, 3])])
    # a dense causal table of any size coarsens to [[2]]; dense full to [[1]]
    assert str(masks.BsaRepr(masks.config_causal(12))) == "[[2]]"
    assert str(masks.BsaRepr(np.ones((6, 9), np.uint8))) == "[[111][111]]"        # gcd 3: 6x9 -> 2x3
    assert masks.BsaRepr(np.ones((4, 4), np.uint8)).check_full()
    assert masks.BsaRepr(np.zeros((4, 2), np.uint8)).check_empty()
    assert masks.BsaRepr(masks.config_causal(8)) == masks.BsaRepr(masks.config_causal(2))
    subs = masks.BsaRepr(masks.config_causal(4)).split_n(2)
    assert [str(x) for x in subs] == ["[[2]]", "[[0]]", "[[1]]"]
