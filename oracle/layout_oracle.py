"""CPU restatement of the column-buffer layout changes around a fused rectangle of Y column
chunks (test infrastructure only: the product never imports this).

Follows ``orchestrated_attn/orchestrated_attn_impl.py:264-272`` (forward), ``:507-515``
(backward input) and ``:546-549`` (backward column output).  Pure data movement, so results are
bit-exact; pinned in ``tests/test_oracle_layout.py`` by an explicit index loop, by the round trip
and by torch's own ``view / transpose / contiguous`` chain (the reference's expression).
"""
import numpy as np


def cols_gather(buf: np.ndarray, n_chunks: int, k_shape) -> np.ndarray:
    """[Y, 2, B, Skv, Nh, D] -> [2, B, Y*Skv, Nh, D] (orchestrated_attn_impl.py:269)."""
    B, S, Nh, D = k_shape
    x = np.asarray(buf).reshape(n_chunks, 2, B, S, Nh, D)
    return np.ascontiguousarray(x.transpose(1, 2, 0, 3, 4, 5)).reshape(2, B, n_chunks * S, Nh, D)


def cols_scatter(buf: np.ndarray, n_chunks: int, k_shape) -> np.ndarray:
    """[2, B, Y*Skv, Nh, D] -> [Y, 2, B, Skv, Nh, D]; with B = 1 this is the reference's
    ``oc.view(2, Y, K_nelem).transpose(0, 1).contiguous()`` (orchestrated_attn_impl.py:548)."""
    B, S, Nh, D = k_shape
    x = np.asarray(buf).reshape(2, B, n_chunks, S, Nh, D)
    return np.ascontiguousarray(x.transpose(2, 0, 1, 3, 4, 5))
