"""Block masks of the block-sparse attention path (host logic, integer only).

Block types are ``Block_Type`` of the reference (``search_algo/utils.py:140-143``):
0 EMPTY, 1 FULL, 2 CAUSAL, stored as uint8.  ``canonical_block_table`` mirrors
``create_bsa_block_table`` (``search_algo/bsa_utils.py:115-150``); the ``config_*`` builders
are the five benchmark masks, given as predicates on 512-token block indices.
"""
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
