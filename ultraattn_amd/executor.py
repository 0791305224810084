"""One-GPU counterpart of the reference's plan-driven loop over ``Comp_Kernel``s
(``intra_attn_forward`` / ``intra_attn_backward``,
``orchestrated_attn/orchestrated_attn_impl.py:300-363, 554-620``).

The reference walks ``execution_plan.gpu_kernel_lists[rank]`` and launches one dense
flash-attention call per ``Comp_Kernel`` key ``(b, h, r_id | r_ids, c_id | c_ids, gpu)``
(``search_algo/dependent_graph.py:51-72``; fused rectangles carry tuples of ids,
``search_algo/graph_transformation_engine.py:83``).  Here the same list becomes ONE block mask,
hence one tile list and one kernel launch per direction, and the ``reduce`` steps the reference
leaves as stubs (``orchestrated_attn/utils.py:119-134, 260-262, 296-298``) are the merge kernel
and an fp32 sum.
"""
from typing import Iterable, List, Optional, Sequence, Tuple, Union

import numpy as np
import torch

from .masks import CAUSAL, EMPTY, FULL
from .ops import bsa_bwd, bsa_fwd, grad_sum, merge_partials, softmax_delta
from .tilelist import TileList, build_tile_list

Ids = Union[int, Tuple[int, ...]]
CompKey = Tuple[int, int, Ids, Ids, int]


def _ids(x: Ids) -> Tuple[int, ...]:
    return tuple(int(i) for i in x) if isinstance(x, (tuple, list, np.ndarray)) else (int(x),)


def mask_from_comp_kernels(keys: Iterable[CompKey], n_row_chunks: int, n_col_chunks: int, causal: bool,
                           rank: Optional[int] = None) -> np.ndarray:
    """Block mask (0/1/2) covered by a list of ``Comp_Kernel`` keys.  A kernel is causal iff the
    mask is causal and its row id is a plain int equal to its column id
    (``kernel_causal = causal and isinstance(rid, int) and rid == cid``,
    ``orchestrated_attn_impl.py:91``); a fused rectangle (tuple ids) is a dense block of chunks.
    ``rank`` keeps only the keys assigned to that GPU (key[4])."""
    m = np.zeros((n_row_chunks, n_col_chunks), np.uint8)
    for key in keys:
        _, _, rid, cid, gpu = key
        if rank is not None and int(gpu) != rank:
            continue
        kernel_causal = bool(causal) and isinstance(rid, (int, np.integer)) and isinstance(cid, (int, np.integer)) \
            and int(rid) == int(cid)
        for r in _ids(rid):
            for c in _ids(cid):
                if m[r, c] != EMPTY:
                    raise ValueError(f"chunk ({r}, {c}) is covered by two kernels")
                m[r, c] = CAUSAL if kernel_causal else FULL
    return m


def comp_kernels_from_schedule(schedule_table: np.ndarray, rank: Optional[int] = None) -> List[CompKey]:
    """Keys in the reference's enumeration order (``search_algo/dependent_graph.py:235-240``):
    batch, head, then row chunk k outer / column chunk l inner, every entry >= 0
    (-1 = empty, ``search_algo/search_engine.py:363-370``)."""
    st = np.asarray(schedule_table)
    if st.ndim == 2:
        st = st[None, None]
    out = []
    for i in range(st.shape[0]):
        for j in range(st.shape[1]):
            for k in range(st.shape[2]):
                for l in range(st.shape[3]):
                    g = int(st[i, j, k, l])
                    if g >= 0 and (rank is None or g == rank):
                        out.append((i, j, k, l, g))
    return out


class BlockSparseExecutor:
    """Runs one device's share of a block-sparse attention on one GPU.

    ``block_mask``: uint8 [row chunks, column chunks] of 0 EMPTY / 1 FULL / 2 CAUSAL for the
    chunks this device computes; ``chunk`` = tokens per chunk (``S_per_partition``).
    ``kernel_tiles`` > 1 splits the key range into that many kernel tiles whose partial
    (O, LSE) are merged, as the streaming configuration does."""

    def __init__(self, block_mask: np.ndarray, chunk: int, softmax_scale: Optional[float] = None,
                 kernel_tiles: int = 1):
        self.mask = np.ascontiguousarray(block_mask, dtype=np.uint8)
        self.chunk = int(chunk)
        self.softmax_scale = softmax_scale
        self.tiles: TileList = build_tile_list(self.mask, block=self.chunk)
        self.kernel_tiles: List[TileList] = []
        self._parts, self._part_key = None, None
        if kernel_tiles > 1:
            cols = np.nonzero(self.mask.any(0))[0]
            for part in np.array_split(cols, min(kernel_tiles, max(1, len(cols)))):
                sub = np.zeros_like(self.mask)
                sub[:, part] = self.mask[:, part]
                self.kernel_tiles.append(build_tile_list(sub, block=self.chunk))

    @classmethod
    def from_comp_kernels(cls, keys: Iterable[CompKey], n_row_chunks: int, n_col_chunks: int, chunk: int,
                          causal: bool, rank: Optional[int] = None, **kw) -> "BlockSparseExecutor":
        return cls(mask_from_comp_kernels(keys, n_row_chunks, n_col_chunks, causal, rank), chunk, **kw)

    @classmethod
    def from_schedule_table(cls, schedule_table: np.ndarray, block_table: np.ndarray, rank: int, chunk: int,
                            **kw) -> "BlockSparseExecutor":
        """``schedule_table[k, l] == rank`` selects this device's chunks; their types come from the
        block table (``Block_Type`` values)."""
        st = np.asarray(schedule_table)
        st = st.reshape(st.shape[-2:])
        return cls(np.where(st == rank, np.asarray(block_table, np.uint8), EMPTY).astype(np.uint8), chunk, **kw)

    def _partials(self, q):
        """The partial (O, LSE) buffers of the kernel tiles, allocated on the first call for a shape
        and device and reused afterwards (a serving loop then allocates nothing per step)."""
        key = (tuple(q.shape), q.device)
        if self._part_key != key:
            B, Sq, Nh, _ = q.shape
            self._parts = [(torch.empty(q.shape, dtype=q.dtype, device=q.device),
                            torch.empty(B, Nh, Sq, dtype=torch.float32, device=q.device)) for _ in self.kernel_tiles]
            self._part_key = key
        return self._parts

    def forward(self, q, k, v, out=None, lse=None):
        """-> (out, lse); one launch, or ``kernel_tiles`` launches into partial buffers that the
        executor keeps + one merge.  The partials are overwritten by the next call with kernel
        tiles, so calls on different streams must not overlap."""
        if not self.kernel_tiles:
            return bsa_fwd(q, k, v, self.tiles, self.softmax_scale, out=out, lse=lse)
        parts = [bsa_fwd(q, k, v, t, self.softmax_scale, out=po, lse=pl)
                 for t, (po, pl) in zip(self.kernel_tiles, self._partials(q))]
        return merge_partials([p[0] for p in parts], [p[1] for p in parts], out=out, lse=lse)

    def forward_per_rectangle(self, q, k, v, fold: bool = True):
        """-> (out, lse) computed the way the reference's executors do it: one dense tile call per
        non-empty chunk pair, in the row-major order of the kernel list
        (``intra_attn_forward``'s loop, ``orchestrated_attn/orchestrated_attn_impl.py:348-349``; a
        chunk is causal iff its type is CAUSAL, ``:91``), each partial ``(O, LSE)`` folded into the
        row chunk's running result with ``update_out_and_lse(..., slice_=)``
        (``ring_flash_attn/utils.py:78-99``, as ``hierarchy_attn/hierarchy_attn_impl.py:64-81`` does),
        running output in fp32, running LSE ``[B, S, Nh, 1]``.  Same result as ``forward`` to the
        parity bar; it exists to measure what the single launch over a tile list replaces, and as
        a second, independent path through the kernels.  ``fold=False`` leaves the folding out, as
        the reference's harness does (its ``reduce`` is ``pass``, ``orchestrated_attn/utils.py:119-134``):
        every rectangle overwrites its row chunk, the result is the last rectangle's and only the
        time means anything."""
        from .flash_attn_interface import _flash_attn_forward
        from .ops import update_out_and_lse
        B, Sq, Nh, D = q.shape
        c = self.chunk
        scale = self.softmax_scale if self.softmax_scale is not None else D ** -0.5
        out = torch.zeros(B, Sq, Nh, D, dtype=torch.float32, device=q.device)
        lse = torch.full((B, Sq, Nh, 1), float("-inf"), dtype=torch.float32, device=q.device)
        blk = torch.empty(B, c, Nh, D, dtype=q.dtype, device=q.device)
        for r, row in enumerate(self.mask):
            rows = slice(r * c, (r + 1) * c)
            for col in np.nonzero(row)[0]:
                cols = slice(int(col) * c, (int(col) + 1) * c)
                res = _flash_attn_forward(q[:, rows], k[:, cols], v[:, cols], 0.0, scale, causal=bool(row[col] == CAUSAL), out=blk)
                if fold:
                    update_out_and_lse(out, lse, res[0], res[5], slice_=(slice(None), rows))
        return out.to(q.dtype), lse.squeeze(-1).transpose(1, 2).contiguous()

    def backward_per_rectangle(self, dout, q, k, v, lse, softmax_d):
        """-> (dq, dk, dv) the reference's way: one dense backward call per non-empty chunk pair
        (``intra_attn_backward``'s loop, ``orchestrated_attn/orchestrated_attn_impl.py:554-620``) with
        the rows' global ``lse`` and ``softmax_d``, every partial gradient added into an fp32 running
        sum per row chunk (dQ) or column chunk (dK, dV) and cast once at the end
        (``ring_flash_attn/ring_flash_attn.py:110-118, 135``), one ``ua_grad_accumulate`` per partial."""
        from .flash_attn_interface import _flash_attn_backward
        from .ops import grad_accumulate
        B, Sq, Nh, D = q.shape
        c = self.chunk
        scale = self.softmax_scale if self.softmax_scale is not None else D ** -0.5
        f32 = dict(dtype=torch.float32, device=q.device)
        acc_q = [torch.zeros(B, c, Nh, D, **f32) for _ in range(self.mask.shape[0])]
        acc_k = [torch.zeros(B, c, Nh, D, **f32) for _ in range(self.mask.shape[1])]
        acc_v = [torch.zeros(B, c, Nh, D, **f32) for _ in range(self.mask.shape[1])]
        gq, gk, gv = (torch.empty(B, c, Nh, D, dtype=q.dtype, device=q.device) for _ in range(3))
        for r, row in enumerate(self.mask):
            rows = slice(r * c, (r + 1) * c)
            lse_r, d_r = lse[:, :, rows].contiguous(), softmax_d[:, :, rows].contiguous()
            for col in np.nonzero(row)[0]:
                cols = slice(int(col) * c, (int(col) + 1) * c)
                _flash_attn_backward(dout[:, rows], q[:, rows], k[:, cols], v[:, cols], None, lse_r, gq, gk, gv, 0.0, scale,
                                     bool(row[col] == CAUSAL), softmax_d=d_r)
                grad_accumulate(gq, None, acc=acc_q[r])
                grad_accumulate(gk, None, acc=acc_k[int(col)])
                grad_accumulate(gv, None, acc=acc_v[int(col)])
        cat = lambda parts: torch.cat([a.to(q.dtype) for a in parts], dim=1)
        return cat(acc_q), cat(acc_k), cat(acc_v)

    def backward(self, dout, q, k, v, out, lse, dq=None, dk=None, dv=None, softmax_d=None):
        """-> (dq, dk, dv).  ``lse`` (and ``softmax_d``) are the rows' GLOBAL statistics: when this
        device holds only part of a row's keys they are those of the merged result."""
        if softmax_d is None:
            softmax_d = softmax_delta(out, dout)
        return bsa_bwd(dout, q, k, v, None, lse, self.tiles, self.softmax_scale, dq=dq, dk=dk, dv=dv,
                       softmax_d=softmax_d)

    @staticmethod
    def reduce_fwd(parts: Sequence[Tuple[torch.Tensor, torch.Tensor]], out=None, lse=None):
        """``Output_Row_Fwd.reduce`` for any number of partial (O, LSE) pairs."""
        return merge_partials([p[0] for p in parts], [p[1] for p in parts], out=out, lse=lse)

    @staticmethod
    def reduce_bwd(parts: Sequence[torch.Tensor]) -> torch.Tensor:
        """``Output_Row_Bwd.reduce`` / ``Output_Col_Bwd.reduce``: fp32 sum of partial gradients
        (``ring_flash_attn/ring_flash_attn.py:110-118`` accumulates in fp32), returned in bf16; one
        pass over up to 16 partials (``ua_grad_sum``)."""
        return grad_sum([p if p.is_contiguous() else p.contiguous() for p in parts])
