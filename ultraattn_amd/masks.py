"""Block masks of the block-sparse attention path (host logic, integer only).

Block types are ``Block_Type`` of the reference (``search_algo/utils.py:140-143``):
0 EMPTY, 1 FULL, 2 CAUSAL, stored as uint8.  ``canonical_block_table`` mirrors
``create_bsa_block_table`` (``search_algo/bsa_utils.py:115-150``); the ``config_*`` builders
are the five benchmark masks, given as predicates on 512-token block indices.
"""
import math
from typing import Tuple

import numpy as np

EMPTY, FULL, CAUSAL = 0, 1, 2
BLOCK_COMP_VOLUME = (0.0, 1.0, 0.5)          # search_algo/utils.py:145-149


def canonical_block_table(case_id: int) -> np.ndarray:
    """The reference's canonical patterns (``search_algo/bsa_utils.py:115-150``)."""
    if case_id == 0:                                   # stride(1/16, 4, 3) after remapping
        t = np.zeros((16, 16), np.uint8)
        for r in range(4):
            t[4 * r:4 * r + 4, 4 * r:4 * r + 4] = FULL
            t[4 * r, 4 * r + 3] = t[4 * r + 3, 4 * r] = EMPTY
    elif case_id == 1:                                 # local+global(1/16, 1, 1)
        t = np.zeros((16, 16), np.uint8)
        t[:, 0] = t[0, :] = FULL
        np.fill_diagonal(t, FULL)
    elif case_id == 2:                                 # star(1/4)
        t = np.zeros((4, 4), np.uint8)
        t[:, 0] = FULL
        np.fill_diagonal(t, CAUSAL)
    elif case_id == 3:                                 # stream(1/8, 3)
        t = np.zeros((8, 8), np.uint8)
        for i in range(8):
            t[i, max(0, i - 2):i] = FULL
            t[i, 0] = FULL
            t[i, i] = CAUSAL
    elif case_id == 4:
        t = np.full((1, 1), FULL, np.uint8)
    elif case_id == 5:
        t = np.full((1, 1), CAUSAL, np.uint8)
    else:
        raise Exception(f"Not support bsa_block_table case_id={case_id}")
    return t


def from_predicate(nqb: int, nkb: int, pred, causal: bool, q_block_offset: int = 0) -> np.ndarray:
    """uint8 table from ``pred(gi, j)`` on global block indices; the diagonal block
    (``gi == j``) is CAUSAL when the mask is causal (``orchestrated_attn_impl.py:91``)."""
    gi = np.arange(nqb)[:, None] + q_block_offset
    j = np.arange(nkb)[None, :]
    t = np.where(pred(gi, j), FULL, EMPTY).astype(np.uint8)
    if causal:
        t[(gi == j) & (t != EMPTY)] = CAUSAL
    return t


def config_causal(n_blocks: int) -> np.ndarray:
    """Configs 1 and 2: query block i attends key blocks j <= i, causal on the diagonal."""
    return from_predicate(n_blocks, n_blocks, lambda i, j: j <= i, causal=True)


def config_strided(n_blocks: int = 256, local: int = 4, stride: int = 8) -> np.ndarray:
    """Config 3: j <= i and (i - j < local or (i - j) % stride == 0), causal."""
    return from_predicate(n_blocks, n_blocks,
                          lambda i, j: (j <= i) & ((i - j < local) | ((i - j) % stride == 0)), causal=True)


def config_global_local(n_blocks: int = 256, n_global: int = 2, band: int = 8) -> np.ndarray:
    """Config 4: blocks < n_global attend and are attended by all, plus |i - j| < band; not causal."""
    return from_predicate(n_blocks, n_blocks,
                          lambda i, j: (np.abs(i - j) < band) | (i < n_global) | (j < n_global), causal=False)


def config_streaming_shard(n_q_blocks: int = 128, n_k_blocks: int = 1024, window: int = 16) -> np.ndarray:
    """Config 5: the last ``n_q_blocks`` query blocks of an ``n_k_blocks`` context; sink
    block 0 plus a causal sliding window of ``window`` blocks."""
    off = n_k_blocks - n_q_blocks
    return from_predicate(n_q_blocks, n_k_blocks,
                          lambda gi, j: ((j <= gi) & (gi - j < window)) | (j == 0), causal=True, q_block_offset=off)


def apply_causal_rule(block_mask: np.ndarray, causal: bool, q_block_offset: int = 0) -> np.ndarray:
    """Turn the diagonal's non-empty blocks into CAUSAL when ``causal`` is set
    (``kernel_causal = causal and rid == cid``, ``orchestrated_attn_impl.py:91``)."""
    t = np.ascontiguousarray(block_mask, dtype=np.uint8).copy()
    if causal:
        i = np.arange(t.shape[0])
        j = i + q_block_offset
        ok = (j >= 0) & (j < t.shape[1])
        i, j = i[ok], j[ok]
        sel = t[i, j] != EMPTY
        t[i[sel], j[sel]] = CAUSAL
    return t


def block_counts(block_table: np.ndarray) -> Tuple[int, int]:
    """(number of FULL blocks, number of CAUSAL blocks)."""
    return int((block_table == FULL).sum()), int((block_table == CAUSAL).sum())


def total_sparsity(block_table: np.ndarray) -> float:
    """Density with CAUSAL blocks weighted 0.5 (``search_algo/bsa_config.py:364-371``)."""
    nf, nc = block_counts(block_table)
    return (nf + 0.5 * nc) / block_table.size


def calc_flops(mbs: int, S: Tuple[int, int], Nh: int, D: int, fob: int = 0, total_sparsity: float = 1.0):
    """(model flops, hardware flops) by the reference's convention
    (``search_algo/utils.py:92-103``): fwd 4*B*Sq*Skv*Nh*D*density; bwd x2 / x2.5;
    fwd+bwd x3 / x3.5."""
    flops = 2 * 2 * mbs * S[0] * S[1] * Nh * D * total_sparsity
    if fob == 0:
        return flops, flops
    if fob == 1:
        return 2 * flops, 2.5 * flops
    if fob == 2:
        return 3 * flops, 3.5 * flops
    raise ValueError(f"fob must be 0, 1 or 2, got {fob}")


# ---- block-mask algebra: refinement, its inverse and sub-selection ---------------------------
# Host counterpart of ``BSA_Repr`` (``search_algo/bsa_config.py:10-263``) on uint8 tables.  The
# refinement is the rule the tile-list builder applies on the device; the inverse and the
# sub-selection are what the reference's planner uses to name a tile's type
# (``search_algo/dependent_graph.py:253-258``).

def _causal_pattern(rate: int) -> np.ndarray:
    i, j = np.indices((rate, rate))
    return np.where(i == j, CAUSAL, np.where(i > j, FULL, EMPTY)).astype(np.uint8)


def complicate(block_table: np.ndarray, rate: int) -> np.ndarray:
    """Refine every block into ``rate x rate`` sub-blocks: EMPTY -> all EMPTY, FULL -> all FULL,
    CAUSAL -> CAUSAL on the sub-diagonal, FULL below it, EMPTY above
    (``complicate_block`` / ``complicate``, ``search_algo/bsa_config.py:177-213``).  Rectangular
    tables are allowed."""
    t = np.ascontiguousarray(block_table, dtype=np.uint8)
    if t.ndim != 2 or rate < 1:
        raise ValueError("complicate needs a 2-D table and rate >= 1")
    if t.size and t.max() > CAUSAL:
        raise Exception(f"[ERROR]: Unknown block_type: {int(t.max())}")
    up = np.kron(t, np.ones((rate, rate), np.uint8))
    causal = np.kron((t == CAUSAL).astype(np.uint8), np.ones((rate, rate), np.uint8)).astype(bool)
    pat = np.tile(_causal_pattern(rate), t.shape)
    return np.where(causal, pat, up).astype(np.uint8)


def complicate_to(block_table: np.ndarray, r_tar: int) -> np.ndarray:
    """Refine so that the table has ``r_tar`` rows (``search_algo/bsa_config.py:215-217``)."""
    n = block_table.shape[0]
    assert n < r_tar and r_tar % n == 0
    return complicate(block_table, r_tar // n)


def merge_blocks(sub_table: np.ndarray):
    """Type of the block that refines to the square ``sub_table``, or None
    (``search_algo/bsa_config.py:69-92``)."""
    s = np.asarray(sub_table)
    if (s == EMPTY).all():
        return EMPTY
    if (s == FULL).all():
        return FULL
    if s.shape[0] == s.shape[1] and np.array_equal(s, _causal_pattern(s.shape[0])):
        return CAUSAL
    return None


def simplify_by_k(block_table: np.ndarray, k: int):
    """One coarsening step by factor ``k`` -> (table, succeeded); the table is returned unchanged
    when some ``k x k`` group is not a refined block (``search_algo/bsa_config.py:125-160``)."""
    t = np.ascontiguousarray(block_table, dtype=np.uint8)
    nq, nk = t.shape
    if k <= 1 or math.gcd(nq, nk) % k != 0:
        return t, False
    g = t.reshape(nq // k, k, nk // k, k).transpose(0, 2, 1, 3)          # [i, j, a, b]
    is_e = (g == EMPTY).all(axis=(2, 3))
    is_f = (g == FULL).all(axis=(2, 3))
    is_c = (g == _causal_pattern(k)).all(axis=(2, 3))
    if not (is_e | is_f | is_c).all():
        return t, False
    # the reference tests EMPTY, then FULL, then CAUSAL (for k >= 2 the three are exclusive)
    return np.where(is_e, EMPTY, np.where(is_f, FULL, CAUSAL)).astype(np.uint8), True


def _prime_factors(n: int):
    out, p = [], 2
    while p * p <= n:
        e = 0
        while n % p == 0:
            n //= p
            e += 1
        if e:
            out.append((p, e))
        p += 1
    if n > 1:
        out.append((n, 1))
    return out


def simplify(block_table: np.ndarray) -> np.ndarray:
    """Coarsest table that refines to ``block_table``: for every prime factor of
    gcd(rows, columns), ascending, coarsen by it as many times as it divides, stopping that
    factor at the first failure (``search_algo/bsa_config.py:162-175``)."""
    t = np.ascontiguousarray(block_table, dtype=np.uint8)
    for alpha, beta in _prime_factors(math.gcd(*t.shape)):
        for _ in range(beta):
            t, ok = simplify_by_k(t, alpha)
            if not ok:
                break
    return t


class BsaRepr:
    """``BSA_Repr`` without the device colour map (``search_algo/bsa_config.py:10-22``): keeps the
    table it was given and its coarsest form ``block_table_raw``."""

    def __init__(self, block_table: np.ndarray, cmap=None):
        if cmap is not None:
            raise NotImplementedError("the colour map belongs to the planner, not to this path")
        t = np.ascontiguousarray(block_table, dtype=np.uint8)
        assert t.ndim == 2
        self.block_table = t
        self.block_table_raw = simplify(t)
        self.minimum_Par_D = self.block_table_raw.shape[0]

    def create_sub_bsa_repr(self, split_degrees, select_ids) -> "BsaRepr":
        """The sub-table of the given row and column ids at granularity ``split_degrees``
        (``search_algo/bsa_config.py:24-42``): refine when the split is finer than the raw table,
        otherwise map every id to its group of raw rows / columns; then ``np.ix_``."""
        raw = self.block_table_raw
        assert len(split_degrees) == len(select_ids) == 2
        assert split_degrees[0] == split_degrees[1]
        if split_degrees[0] > raw.shape[0]:
            cur = complicate_to(raw, split_degrees[0])
        else:
            assert raw.shape[0] % split_degrees[0] == 0
            cur = raw
            factor = raw.shape[0] // split_degrees[0]
            select_ids = [[n for i in ids for n in range(i * factor, (i + 1) * factor)] for ids in select_ids]
        return BsaRepr(cur[np.ix_(*select_ids)])

    def check_causal(self) -> bool:
        """Raw table is EMPTY above the diagonal, CAUSAL on it, EMPTY or FULL below
        (``search_algo/bsa_config.py:44-53``)."""
        t = self.block_table_raw
        i, j = np.indices(t.shape)
        return bool(((i >= j) | (t == EMPTY)).all() and ((i != j) | (t == CAUSAL)).all()
                    and ((i <= j) | (t == EMPTY) | (t == FULL)).all())

    def check_empty(self) -> bool:
        return bool((self.block_table_raw == EMPTY).all())        # bsa_config.py:55-60

    def check_full(self) -> bool:
        return bool((self.block_table_raw == FULL).all())         # bsa_config.py:62-67

    def split_n(self, n: int):
        """The distinct sub-tables of an n x n split (``search_algo/bsa_config.py:226-247``)."""
        cur = self.block_table_raw.shape[0]
        if cur >= n:
            assert cur % n == 0
            size, table = cur // n, self.block_table_raw
        else:
            assert n % cur == 0
            size, table = 1, complicate(self.block_table_raw, n // cur)
        out = []
        for i in range(n):
            for j in range(n):
                r = BsaRepr(table[i * size:(i + 1) * size, j * size:(j + 1) * size])
                if r not in out:
                    out.append(r)
        return out

    def __str__(self) -> str:                                      # bsa_config.py:249-258
        return "[" + "".join("[" + "".join(str(int(v)) for v in row) + "]" for row in self.block_table_raw) + "]"

    def __eq__(self, other) -> bool:
        return isinstance(other, BsaRepr) and np.array_equal(self.block_table_raw, other.block_table_raw)

    __hash__ = None
