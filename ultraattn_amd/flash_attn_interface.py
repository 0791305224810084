"""Drop-in for the two functions the reference's executors import from the flash-attention
fork: ``from flash_attn.flash_attn_interface import _flash_attn_forward, _flash_attn_backward``
(``orchestrated_attn/orchestrated_attn_impl.py:7-8``, ``hierarchy_attn/hierarchy_attn_impl.py:3``).

Same positional/keyword arguments, including the fork's ``out=`` (forward) and ``softmax_d=``
(backward).  A dense rectangle is the degenerate block mask (all tiles full, or causal on the
diagonal), so both functions run the block-sparse kernels.
"""
from functools import lru_cache
from typing import Optional

import numpy as np
import torch

from .ops import bsa_bwd, bsa_fwd
from .tilelist import TILE, TileList, build_tile_list


@lru_cache(maxsize=64)
def _dense_tiles(n_qtiles: int, n_ktiles: int, causal: bool) -> TileList:
    m = np.ones((n_qtiles, n_ktiles), np.uint8)
    if causal:
        # flash-attn (2.1 and later) aligns the causal diagonal to the bottom-right corner when
        # Sq != Skv: query i sees key j iff j <= i + Skv - Sq; rows above the first key see nothing
        off = n_ktiles - n_qtiles
        i = np.arange(n_qtiles)[:, None] + off
        j = np.arange(n_ktiles)[None, :]
        m = np.where(j < i, 1, np.where(j == i, 2, 0)).astype(np.uint8)
    return build_tile_list(m, block=TILE)


def _check_unsupported(dropout_p, window_size, alibi_slopes, return_softmax=False):
    if dropout_p != 0:
        raise NotImplementedError("dropout_p must be 0")
    if tuple(window_size) != (-1, -1):
        raise NotImplementedError("window_size must be (-1, -1)")
    if alibi_slopes is not None:
        raise NotImplementedError("alibi_slopes must be None")
    if return_softmax:
        raise NotImplementedError("return_softmax needs dropout_p > 0, which is unsupported")


def _flash_attn_forward(q, k, v, dropout_p, softmax_scale, causal, window_size=(-1, -1),
                        alibi_slopes=None, return_softmax=False, out=None):
    """-> (out, q, k, v, out_padded, softmax_lse, S_dmask, rng_state); callers use [0] and [5]
    (``orchestrated_attn_impl.py:326``, ``hierarchy_attn_impl.py:41``)."""
    _check_unsupported(dropout_p, window_size, alibi_slopes, return_softmax)
    if causal and (k.shape[1] - q.shape[1]) % TILE != 0:
        raise NotImplementedError("causal with Skv - Sq not a multiple of 128")
    tiles = _dense_tiles(q.shape[1] // TILE, k.shape[1] // TILE, bool(causal))
    out, lse = bsa_fwd(q, k, v, tiles, softmax_scale, out=out)
    return out, q, k, v, out, lse, None, None


def _flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, dropout_p, softmax_scale, causal,
                         window_size=(-1, -1), alibi_slopes=None, deterministic=False, rng_state=None,
                         softmax_d: Optional[torch.Tensor] = None):
    """Writes dq, dk, dv in place (allocates the ones passed as None); returns (dq, dk, dv, softmax_d).  With ``softmax_d`` given
    ``out`` is ignored (the reference passes a dummy, ``orchestrated_attn_impl.py:583``).
    The kernels are deterministic regardless of ``deterministic``."""
    _check_unsupported(dropout_p, window_size, alibi_slopes)
    if causal and (k.shape[1] - q.shape[1]) % TILE != 0:
        raise NotImplementedError("causal with Skv - Sq not a multiple of 128")
    tiles = _dense_tiles(q.shape[1] // TILE, k.shape[1] // TILE, bool(causal))
    if softmax_d is None:
        from .ops import softmax_delta
        softmax_d = softmax_delta(out, dout)
    dq, dk, dv = bsa_bwd(dout, q, k, v, None, softmax_lse, tiles, softmax_scale, dq=dq, dk=dk, dv=dv,
                         softmax_d=softmax_d)
    return dq, dk, dv, softmax_d
