"""numpy restatement of the block-mask algebra and of the active-tile enumeration.

Test infrastructure (see oracle/__init__.py).  Block types are the reference's
``Block_Type`` values (``search_algo/utils.py:140-143``): 0 EMPTY, 1 FULL, 2 CAUSAL;
``Block_Comp_Volume`` (``search_algo/utils.py:145-149``): 0, 1, 0.5.
"""
from typing import Dict, List, Tuple

import numpy as np

EMPTY, FULL, CAUSAL = 0, 1, 2
COMP_VOLUME = {EMPTY: 0.0, FULL: 1.0, CAUSAL: 0.5}


def complicate_block(block_type: int, rate: int) -> np.ndarray:
    """``search_algo/bsa_config.py:177-194``: EMPTY -> all EMPTY, FULL -> all FULL,
    CAUSAL -> CAUSAL on i == j, FULL for i > j, EMPTY for i < j."""
    sub = np.zeros((rate, rate), dtype=np.uint8)
    for i in range(rate):
        for j in range(rate):
            if block_type == EMPTY:
                sub[i, j] = EMPTY
            elif block_type == FULL:
                sub[i, j] = FULL
            elif block_type == CAUSAL:
                sub[i, j] = CAUSAL if i == j else (FULL if i > j else EMPTY)
            else:
                raise Exception(f"[ERROR]: Unknown block_type: {block_type}")
    return sub


def complicate(block_table: np.ndarray, rate: int) -> np.ndarray:
    """``search_algo/bsa_config.py:196-213`` without the cmap (rectangular tables allowed)."""
    nr, nc = block_table.shape
    out = np.empty((nr * rate, nc * rate), dtype=np.uint8)
    for i in range(nr):
        for j in range(nc):
            out[i * rate:(i + 1) * rate, j * rate:(j + 1) * rate] = complicate_block(int(block_table[i, j]), rate)
    return out


def simplify_once(block_table: np.ndarray, k: int):
    """Inverse of ``complicate`` by factor k when every k x k group is uniformly EMPTY, FULL
    or the refined-CAUSAL pattern (``search_algo/bsa_config.py:69-92, 125-175``).
    Returns the coarse table or None."""
    nr, nc = block_table.shape
    if nr % k or nc % k:
        return None
    out = np.empty((nr // k, nc // k), dtype=np.uint8)
    pats = {t: complicate_block(t, k) for t in (EMPTY, FULL, CAUSAL)}
    for i in range(nr // k):
        for j in range(nc // k):
            g = block_table[i * k:(i + 1) * k, j * k:(j + 1) * k]
            for t in (EMPTY, FULL, CAUSAL):
                if np.array_equal(g, pats[t]):
                    out[i, j] = t
                    break
            else:
                return None
    return out


def apply_causal_rule(block_mask: np.ndarray, causal: bool, q_block_offset: int = 0) -> np.ndarray:
    """``orchestrated_attn/orchestrated_attn_impl.py:91``: a tile is causal iff the global
    mask is causal and its row-chunk id equals its column-chunk id.  Row-chunk ids of a q
    shard are offset by ``q_block_offset`` in the global grid."""
    t = np.array(block_mask, dtype=np.uint8, copy=True)
    if causal:
        for i in range(t.shape[0]):
            j = i + q_block_offset
            if 0 <= j < t.shape[1] and t[i, j] != EMPTY:
                t[i, j] = CAUSAL
    return t


def total_sparsity(block_table: np.ndarray) -> float:
    """``search_algo/bsa_config.py:364-371``."""
    blk = 0.0
    for i in range(block_table.shape[0]):
        for j in range(block_table.shape[1]):
            blk += COMP_VOLUME[int(block_table[i, j])]
    return blk / (block_table.shape[0] * block_table.shape[1])


def calc_flops(mbs, S: Tuple[int, int], Nh, D, fob=0, total_sparsity=1.0):
    """``search_algo/utils.py:92-103``: (model flops, hardware flops)."""
    flops = 2 * 2 * mbs * S[0] * S[1] * Nh * D * total_sparsity
    if fob == 0:
        return flops, flops
    if fob == 1:
        return 2 * flops, 2.5 * flops
    return 3 * flops, 3.5 * flops


def enumerate_tiles(tile_table: np.ndarray) -> List[Tuple[int, int, int]]:
    """Active tiles (k, l, type) in the order of ``search_algo/dependent_graph.py:235-240``:
    k (rows) outer, l (columns) inner, every entry that is not EMPTY."""
    out = []
    for k in range(tile_table.shape[0]):
        for l in range(tile_table.shape[1]):
            if tile_table[k, l] != EMPTY:
                out.append((k, l, int(tile_table[k, l])))
    return out


def build_tile_list(block_table: np.ndarray, rate: int) -> Dict[str, np.ndarray]:
    """Refine by ``rate`` and compact: CSR over q tiles (row-major order), the transposed CSC
    over key tiles, and longest-first stable work orders.  flag: 0 = FULL tile, 1 = CAUSAL."""
    tt = complicate(np.asarray(block_table, dtype=np.uint8), rate)
    nqt, nkt = tt.shape
    tiles = enumerate_tiles(tt)
    row_ptr = np.zeros(nqt + 1, dtype=np.int32)
    col_idx = np.zeros(len(tiles), dtype=np.int32)
    flag = np.zeros(len(tiles), dtype=np.uint8)
    for n, (k, l, t) in enumerate(tiles):
        row_ptr[k + 1] += 1
        col_idx[n] = l
        flag[n] = 1 if t == CAUSAL else 0
    row_ptr = np.cumsum(row_ptr, dtype=np.int64).astype(np.int32)
    col_ptr = np.zeros(nkt + 1, dtype=np.int32)
    by_col = sorted(tiles, key=lambda x: (x[1], x[0]))
    row_idx = np.array([k for k, _, _ in by_col], dtype=np.int32).reshape(-1)
    cflag = np.array([1 if t == CAUSAL else 0 for _, _, t in by_col], dtype=np.uint8).reshape(-1)
    for _, l, _ in by_col:
        col_ptr[l + 1] += 1
    col_ptr = np.cumsum(col_ptr, dtype=np.int64).astype(np.int32)
    q_order = launch_order(row_ptr, col_idx, rate, rate - 1)
    k_order = launch_order(col_ptr, row_idx, rate, 0)
    return dict(row_ptr=row_ptr, col_idx=col_idx, flag=flag, col_ptr=col_ptr, row_idx=row_idx,
                cflag=cflag, q_order=q_order, k_order=k_order, n_qtiles=nqt, n_ktiles=nkt)


def launch_order(ptr: np.ndarray, idx: np.ndarray, rate: int, longest_sub: int) -> np.ndarray:
    """Launch order of the rows of a CSR (``longest_sub = rate - 1``) or the columns of a CSC
    (``longest_sub = 0``).  Rows much longer than average (length * n_rows > 2 * nnz) come first,
    so that they cannot end up as the tail of the launch, longest block line first and then
    lexicographically from the anchor as below.  The others are ordered by
    their anchor index: the first index of the list, or the last one if the last indices take
    fewer distinct values than the first ones over these rows (the lists are then read backwards
    below); then by the length of their block line, longest first (measured as the list length of
    the block's longest tile, sub-tile ``longest_sub``); then lexicographically by the rest of
    their index lists (a list that is a prefix of another sorts after it); ties by row number.
    Rows without tiles come last."""
    n = len(ptr) - 1
    nnz = int(ptr[-1])
    inf = 1 << 40
    lists = [tuple(int(x) for x in idx[ptr[i]:ptr[i + 1]]) for i in range(n)]
    ruled = [l for l in lists if l and not len(l) * n > 2 * nnz]
    from_end = len({l[-1] for l in ruled}) < len({l[0] for l in ruled})

    def key(i):
        lst = lists[i]
        if not lst:
            return (2, (), i)
        ref = i // rate * rate + longest_sub
        block_len = int(ptr[ref + 1] - ptr[ref])
        if from_end:
            lst = lst[::-1]
        if len(lst) * n > 2 * nnz:
            return (0, (-block_len,) + lst + (inf,), i)
        return (1, (lst[0], -block_len) + lst[1:] + (inf,), i)
    return np.array(sorted(range(n), key=key), dtype=np.int32).reshape(-1)


def tiles_to_element_mask(tl: Dict[str, np.ndarray], tile: int) -> np.ndarray:
    """Expand a tile list back to keep[Sq, Skv] for brute-force comparison."""
    nqt, nkt = int(tl["n_qtiles"]), int(tl["n_ktiles"])
    keep = np.zeros((nqt * tile, nkt * tile), dtype=bool)
    tri = np.tril(np.ones((tile, tile), dtype=bool))
    for r in range(nqt):
        for e in range(tl["row_ptr"][r], tl["row_ptr"][r + 1]):
            c = int(tl["col_idx"][e])
            keep[r * tile:(r + 1) * tile, c * tile:(c + 1) * tile] = tri if tl["flag"][e] else True
    return keep


def parse_bsa_repr(s: str) -> np.ndarray:
    """Parse the reference's block-table strings, e.g. '[[2000][1200][1020][1002]]'
    (``plot/e2e_pick.py:65-72``), digits are Block_Type values."""
    rows = [r for r in s.strip().strip("[]").split("][")]
    return np.array([[int(ch) for ch in r] for r in rows], dtype=np.uint8)
