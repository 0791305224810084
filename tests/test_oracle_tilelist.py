"""Pins the tile-list oracle (oracle/tilelist_oracle.py) and the mask builders against the
data the reference holds, brute-force element masks and independently derived counts.  No GPU."""
import json
import os

import numpy as np
import pytest

from oracle import tilelist_oracle as to
from ultraattn_amd import masks


@pytest.fixture(scope="module")
def refdata(golden_dir):
    return json.load(open(os.path.join(golden_dir, "reference_data.json")))


def test_canonical_tables_equal_reference_strings(refdata):
    """create_bsa_block_table cases (search_algo/bsa_utils.py:115-150) against the block-table
    strings the reference plots with (plot/e2e_pick.py:65-72)."""
    strings = refdata["bsa_reprs"]["strings"]
    for case_id, s in zip((0, 1, 4, 5, 2, 3), strings):
        assert np.array_equal(masks.canonical_block_table(case_id), to.parse_bsa_repr(s)), case_id


def test_total_sparsity_matches_reference_log(refdata):
    sp = refdata["sparsity"]
    table = next(a["block_table"] for a in refdata["allocations"] if a["source"] == sp["block_table_source"])
    assert to.total_sparsity(np.array(table)) == sp["total_sparsity"] == 28 / 64
    assert masks.total_sparsity(np.array(table, np.uint8)) == sp["total_sparsity"]
    # CAUSAL weighs one half (search_algo/utils.py:145-149)
    assert to.total_sparsity(masks.canonical_block_table(5)) == 0.5
    assert to.total_sparsity(masks.canonical_block_table(2)) == (3 + 0.5 * 4) / 16


def test_allocation_matrices_cover_exactly_the_block_table(refdata):
    """The reference's ILP results: every non-empty block is owned by exactly one GPU, empty
    ones by none; the per-GPU lists (row-major) partition the full list."""
    assert len(refdata["allocations"]) == 17
    for a in refdata["allocations"]:
        table, alloc = np.array(a["block_table"]), np.array(a["allocation"])
        assert np.array_equal(alloc >= 0, table != 0), a["source"]
        full = [(k, l) for k, l, _ in to.enumerate_tiles(table)]
        per_gpu = []
        for g in range(alloc.max() + 1):
            sub = np.where(alloc == g, table, 0)
            per_gpu += [(k, l) for k, l, _ in to.enumerate_tiles(sub)]
        assert sorted(per_gpu) == full


def test_complicate_rule():
    c = to.complicate_block(to.CAUSAL, 3)
    assert c.tolist() == [[2, 0, 0], [1, 2, 0], [1, 1, 2]]
    assert (to.complicate_block(to.FULL, 3) == 1).all() and (to.complicate_block(to.EMPTY, 3) == 0).all()
    with pytest.raises(Exception):
        to.complicate_block(3, 2)
    t = np.array([[2, 0], [1, 2]], np.uint8)
    assert to.complicate(t, 2).tolist() == [[2, 0, 0, 0], [1, 2, 0, 0], [1, 1, 2, 0], [1, 1, 1, 2]]
    # refining a causal table keeps it causal (search_algo/bsa_config.py:44-53) and round-trips
    for rate in (2, 4):
        assert np.array_equal(to.simplify_once(to.complicate(t, rate), rate), t)
    rs = np.random.RandomState(0)
    r = rs.randint(0, 2, size=(5, 7)).astype(np.uint8)
    assert np.array_equal(to.simplify_once(to.complicate(r, 4), 4), r)
    # composition: refining by 2 twice equals refining by 4
    assert np.array_equal(to.complicate(to.complicate(t, 2), 2), to.complicate(t, 4))


def test_refinement_preserves_the_element_mask():
    """A block table and its refinement describe the same S x S visibility."""
    rs = np.random.RandomState(1)
    t = rs.randint(0, 2, size=(4, 4)).astype(np.uint8)
    t[np.arange(4), np.arange(4)] = 2
    coarse = to.tiles_to_element_mask(to.build_tile_list(t, 1), 8)
    fine = to.tiles_to_element_mask(to.build_tile_list(t, 4), 2)
    assert np.array_equal(coarse, fine)


PREDICATES = {
    "causal": (lambda n: masks.config_causal(n), lambda i, j, n: j <= i, True, 0),
    "strided": (lambda n: masks.config_strided(n, 4, 8), lambda i, j, n: j <= i and (i - j < 4 or (i - j) % 8 == 0), True, 0),
    "global_local": (lambda n: masks.config_global_local(n, 2, 8), lambda i, j, n: abs(i - j) < 8 or i < 2 or j < 2, False, 0),
}


@pytest.mark.parametrize("name", list(PREDICATES))
def test_tile_list_expands_to_the_elementwise_predicate(name):
    make, pred, causal, _ = PREDICATES[name]
    n, blk, tile = 24, 8, 2
    tl = to.build_tile_list(make(n), blk // tile)
    keep = to.tiles_to_element_mask(tl, tile)
    for i in range(n * blk):
        for j in range(n * blk):
            bi, bj = i // blk, j // blk
            want = pred(bi, bj, n) and (not (causal and bi == bj) or j <= i)
            assert keep[i, j] == want, (i, j)


def test_streaming_shard_predicate():
    nq, nk, win, blk, tile = 4, 16, 3, 8, 2
    tl = to.build_tile_list(masks.config_streaming_shard(nq, nk, win), blk // tile)
    keep = to.tiles_to_element_mask(tl, tile)
    off = (nk - nq) * blk
    for i in range(nq * blk):
        for j in range(nk * blk):
            gi = (i + off) // blk
            bj = j // blk
            want = ((bj <= gi and gi - bj < win) or bj == 0) and (bj != gi or j <= i + off)
            assert keep[i, j] == want


def test_full_size_counts(golden_dir):
    """Counts derived independently (by formula) for the five benchmark configurations."""
    gold = json.load(open(os.path.join(golden_dir, "tilelists.json")))
    want = {"c1": (136, 16, 2080, 64), "c2": (2080, 64, 32896, 256), "c3": (4986, 256, 78240, 1024),
            "c4": (4774, 0, 76384, 0), "c5": (2176, 128, 34048, 512)}
    for k, (nb, nc, nt, ntc) in want.items():
        g = gold[k]
        assert (g["blocks"], g["causal_blocks"], g["tiles"], g["causal_tiles"]) == (nb, nc, nt, ntc)
        # full block -> 16 tiles, causal block -> 6 full + 4 causal
        assert nt == 16 * (nb - nc) + 10 * nc and ntc == 4 * nc
    # closed forms
    assert 2080 == 64 * 65 // 2 and 136 == 16 * 17 // 2
    strided = sum(1 for i in range(256) for j in range(i + 1) if i - j < 4 or (i - j) % 8 == 0)
    assert strided == 4986
    gl = sum(1 for i in range(256) for j in range(256) if abs(i - j) < 8 or i < 2 or j < 2)
    assert gl == 4774
    m5 = masks.config_streaming_shard()
    assert sorted(set(np.nonzero(m5.any(0))[0])) == [0] + list(range(881, 1024))


def test_causal_rule_table():
    """kernel_causal = causal and rid == cid (orchestrated_attn_impl.py:91), on global ids."""
    ones = np.ones((3, 5), np.uint8)
    for causal in (False, True):
        for off in (0, 2):
            t = to.apply_causal_rule(ones, causal, off)
            t2 = masks.apply_causal_rule(ones, causal, off)
            assert np.array_equal(t, t2)
            for i in range(3):
                for j in range(5):
                    assert t[i, j] == (2 if (causal and i + off == j) else 1)
    z = np.zeros((2, 2), np.uint8)
    assert (to.apply_causal_rule(z, True) == 0).all()       # empty diagonal blocks stay empty


def test_flops_convention():
    """search_algo/utils.py:92-103 and the figures quoted for the benchmark configurations."""
    m, h = to.calc_flops(1, (131072, 131072), 32, 128, fob=0, total_sparsity=to.total_sparsity(masks.config_strided()))
    assert m == h and abs(h - 2.0865e13) / 2.0865e13 < 1e-4
    m, h = to.calc_flops(1, (131072, 131072), 32, 128, fob=2, total_sparsity=to.total_sparsity(masks.config_strided()))
    assert abs(h - 7.3027e13) / 7.3027e13 < 1e-4 and abs(m - 6.2595e13) / 6.2595e13 < 1e-4
    m, h = to.calc_flops(1, (8192, 8192), 8, 128, 0, to.total_sparsity(masks.config_causal(16)))
    assert abs(h - 1.3744e11) / 1.3744e11 < 1e-4
    m, h = to.calc_flops(1, (65536, 524288), 32, 128, 0, to.total_sparsity(masks.config_streaming_shard()))
    assert abs(h - 9.0710e12) / 9.0710e12 < 1e-4
    assert masks.calc_flops(1, (4096, 4096), 2, 128, 1, 0.5) == to.calc_flops(1, (4096, 4096), 2, 128, 1, 0.5)
    assert to.calc_flops(1, (64, 64), 1, 8, 1)[1] == 2.5 * to.calc_flops(1, (64, 64), 1, 8, 0)[1]
