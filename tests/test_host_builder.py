"""The C-ABI tile-list builder (host entry points) against the numpy oracle: bit-exact.  No GPU."""
import ctypes
import json
import os

import numpy as np
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

from oracle import tilelist_oracle as to
from ultraattn_amd import _lib, masks
from ultraattn_amd.tilelist import build_tile_list

FIELDS = ("row_ptr", "col_idx", "flag", "col_ptr", "row_idx", "cflag", "q_order", "k_order")


def assert_same(tl, ref):
    assert tl.n_qtiles == ref["n_qtiles"] and tl.n_ktiles == ref["n_ktiles"]
    for f in FIELDS:
        a, b = getattr(tl, f), ref[f]
        assert a.dtype == b.dtype and np.array_equal(a, b), f


@pytest.mark.parametrize("make,rate", [
    (lambda: masks.config_causal(16), 4), (lambda: masks.config_strided(48), 4),
    (lambda: masks.config_global_local(40), 2), (lambda: masks.config_streaming_shard(8, 64, 5), 4),
    (lambda: masks.canonical_block_table(0), 1), (lambda: masks.canonical_block_table(3), 8),
    (lambda: np.zeros((3, 4), np.uint8), 2), (lambda: np.full((1, 1), 2, np.uint8), 5),
])
def test_builder_bit_exact(make, rate, lib):
    m = make()
    assert_same(build_tile_list(m, block=128 * rate), to.build_tile_list(m, rate))


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 9), st.integers(1, 9), st.integers(1, 4), st.integers(0, 2 ** 31 - 1))
def test_builder_bit_exact_random(nq, nk, rate, seed):
    m = np.random.RandomState(seed).randint(0, 3, size=(nq, nk)).astype(np.uint8)
    assert_same(build_tile_list(m, block=128 * rate), to.build_tile_list(m, rate))


def test_full_size_digests(golden_dir, lib):
    gold = json.load(open(os.path.join(golden_dir, "tilelists.json")))
    cfgs = {"c1": masks.config_causal(16), "c2": masks.config_causal(64), "c3": masks.config_strided(),
            "c4": masks.config_global_local(), "c5": masks.config_streaming_shard()}
    for k, m in cfgs.items():
        tl = build_tile_list(m, block=512)
        assert tl.nnz == gold[k]["tiles"] and tl.n_causal == gold[k]["causal_tiles"]
        assert tl.sha256() == gold[k]["sha256"]
        # CSC is the transpose of the CSR
        pairs = sorted((int(c), r) for r in range(tl.n_qtiles) for c in tl.col_idx[tl.row_ptr[r]:tl.row_ptr[r + 1]])
        csc = [(c, int(r)) for c in range(tl.n_ktiles) for r in tl.row_idx[tl.col_ptr[c]:tl.col_ptr[c + 1]]]
        assert pairs == csc
        # launch orders are permutations; rows much longer than average lead, longest first
        assert sorted(tl.q_order.tolist()) == list(range(tl.n_qtiles))
        assert sorted(tl.k_order.tolist()) == list(range(tl.n_ktiles))
        ql = np.diff(tl.row_ptr)
        n_long = int((ql * tl.n_qtiles > 2 * tl.nnz).sum())
        head = tl.q_order[:n_long]
        assert all(ql[r] * tl.n_qtiles > 2 * tl.nnz for r in head)
        assert all(ql[a] >= ql[b] for a, b in zip(head[:-1], head[1:]))


def test_launch_order_groups_rows_with_common_tiles(lib):
    """Independent statement of the order: plain Python sort of (first tile, -length of the block
    row, rest of the list padded so that a prefix sorts last, row)."""
    m = masks.config_strided(32)
    rate = 2
    tl = build_tile_list(m, block=128 * rate)
    lists = [tuple(tl.col_idx[tl.row_ptr[r]:tl.row_ptr[r + 1]]) for r in range(tl.n_qtiles)]
    assert not any(len(l) * tl.n_qtiles > 2 * tl.nnz for l in lists) and all(lists)
    block_len = lambda r: len(lists[r // rate * rate + rate - 1])
    want = sorted(range(tl.n_qtiles), key=lambda r: ((lists[r][0], -block_len(r)) + lists[r][1:] + (10 ** 9,), r))
    order = tl.q_order.tolist()
    assert order == want
    # the two query tiles of one strided block sit next to each other
    pos = {r: i for i, r in enumerate(order)}
    assert all(abs(pos[2 * b] - pos[2 * b + 1]) == 1 for b in range(32))
    # rows that start on the same tile: the longer block rows come first
    for a, b in zip(order[:-1], order[1:]):
        if lists[a][0] == lists[b][0]:
            assert block_len(a) >= block_len(b)
    # the key side of the same mask: every column starts at its own diagonal tile, while the columns of
    # one residue class end on the same query tiles, so the order is anchored at the END of the lists
    cols = [tuple(tl.row_idx[tl.col_ptr[c]:tl.col_ptr[c + 1]]) for c in range(tl.n_ktiles)]
    assert len({c[-1] for c in cols}) < len({c[0] for c in cols})
    col_len = lambda c: len(cols[c // rate * rate])
    want_k = sorted(range(tl.n_ktiles), key=lambda c: ((cols[c][-1], -col_len(c)) + cols[c][-2::-1] + (10 ** 9,), c))
    assert tl.k_order.tolist() == want_k
    ends = [cols[c][-1] for c in tl.k_order.tolist()]
    assert ends == sorted(ends)
    # a plain causal mask: all columns end on the last query tile; the longest column (0) comes first
    tc = build_tile_list(masks.config_causal(8), block=256)
    assert tc.k_order.tolist() == list(range(tc.n_ktiles))
    # global rows of the global+local mask are the long ones and come first
    tg = build_tile_list(masks.config_global_local(64, 2, 4), block=128)
    assert sorted(tg.q_order[:2].tolist()) == [0, 1]


def test_causal_flag_and_offset(lib):
    ones = np.ones((2, 4), np.uint8)
    tl = build_tile_list(ones, block=256, causal=True, q_block_offset=2)
    ref = to.build_tile_list(to.apply_causal_rule(ones, True, 2), 2)
    assert_same(tl, ref)
    assert tl.n_causal == 4
    tl0 = build_tile_list(ones, block=256, causal=False)
    assert tl0.n_causal == 0 and tl0.nnz == 32
    boolean = build_tile_list(np.ones((2, 2), bool), block=128, causal=True)
    assert boolean.flag.tolist() == [1, 1, 1, 0] or boolean.n_causal == 2


def test_error_codes(lib):
    m = np.array([[1, 3]], np.uint8)
    n = (ctypes.c_int64 * 3)()
    p = lambda i: ctypes.byref(n, 8 * i)
    sz = lambda mask, a, b, r: lib.ua_tilelist_size(mask, a, b, r, ctypes.cast(p(0), _lib._i64p),
                                                     ctypes.cast(p(1), _lib._i64p), ctypes.cast(p(2), _lib._i64p))
    assert sz(m.ctypes.data, 1, 2, 1) == -5                     # UA_ERR_MASK
    assert sz(None, 1, 2, 1) == -1                               # UA_ERR_NULL
    ok = np.ones((1, 2), np.uint8)
    assert sz(ok.ctypes.data, 0, 2, 1) == -2                     # UA_ERR_SHAPE
    assert sz(ok.ctypes.data, 1, 2, 0) == -2
    assert sz(ok.ctypes.data, 1, 2, 3) == 0 and list(n) == [3, 6, 18]
    assert b"EMPTY" in lib.ua_strerror(-5) and lib.ua_strerror(0) == b"ok"
    with pytest.raises(RuntimeError, match="mask"):
        build_tile_list(m, block=128)
    with pytest.raises(ValueError):
        build_tile_list(ok, block=100)
    with pytest.raises(ValueError):
        build_tile_list(np.ones(3, np.uint8), block=128)
