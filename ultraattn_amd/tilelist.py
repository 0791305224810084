"""Active-tile lists: the compacted 128x128 form of a block mask that the kernels walk."""
import ctypes
import hashlib
from ctypes import c_int64
from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np

from . import _lib
from .masks import apply_causal_rule

TILE = 128

_HOST_FIELDS = ("row_ptr", "col_idx", "flag", "col_ptr", "row_idx", "cflag", "q_order", "k_order")


@dataclass
class TileList:
    """CSR over query tiles (``row_ptr, col_idx, flag``), CSC over key tiles
    (``col_ptr, row_idx, cflag``) and the launch orders (rows that share tiles adjacent, very long rows first), as host numpy arrays;
    ``on(device)`` gives (and caches) device copies."""
    n_qtiles: int
    n_ktiles: int
    row_ptr: np.ndarray
    col_idx: np.ndarray
    flag: np.ndarray
    col_ptr: np.ndarray
    row_idx: np.ndarray
    cflag: np.ndarray
    q_order: np.ndarray
    k_order: np.ndarray
    _dev: Dict = field(default_factory=dict, repr=False)

    @property
    def nnz(self) -> int:
        return int(self.col_idx.shape[0])

    @property
    def n_causal(self) -> int:
        return int(self.flag.sum())

    def sha256(self) -> str:
        """Digest of the row-major active-tile list (row_ptr, col_idx, flag)."""
        hsh = hashlib.sha256()
        for a in (self.row_ptr, self.col_idx, self.flag):
            hsh.update(np.ascontiguousarray(a).tobytes())
        return hsh.hexdigest()

    def on(self, device):
        """Device copies of all arrays as torch tensors (cached per device)."""
        import torch
        key = str(torch.device(device))
        if key not in self._dev:
            if torch.cuda.is_current_stream_capturing():
                # the staging buffers are released once the copies are done: a graph must not replay them
                raise RuntimeError("TileList.on(device) must be called once before the stream is captured into a graph")
            # staged through pinned host memory and copied on the current stream without a host
            # synchronisation; the flag arrays are padded to a multiple of 4 bytes (the kernels read
            # them one aligned 32-bit word at a time)
            dev, pinned = {}, []
            for n in _HOST_FIELDS:
                a = np.ascontiguousarray(getattr(self, n))
                size = -(-max(a.shape[0], 1) // 4) * 4
                host = torch.zeros(size, dtype=torch.from_numpy(a).dtype, pin_memory=True)
                host[:a.shape[0]].copy_(torch.from_numpy(a))
                full = host.to(device, non_blocking=True)
                dev[n] = full[:a.shape[0]] if a.shape[0] else full[:0]
                pinned.append(host)
            dev["_pinned"] = pinned         # kept alive: the copies may still be in flight
            dev["_ready"] = torch.cuda.Event()
            dev["_ready"].record()
            self._dev[key] = dev
            return dev
        dev = self._dev[key]
        ready = dev.get("_ready")
        if ready is not None and not torch.cuda.is_current_stream_capturing():
            if ready.query():
                dev["_ready"] = None
                dev["_pinned"] = None
            else:                           # a later use on another stream orders itself behind the copies
                torch.cuda.current_stream().wait_event(ready)
        return dev


def build_tile_list(block_mask, block: int = 512, tile: int = TILE, causal: bool = False,
                    q_block_offset: int = 0) -> TileList:
    """Block mask [n_qblocks, n_kblocks] (0 EMPTY / 1 FULL / 2 CAUSAL, or bool) -> TileList.

    ``causal`` applies the executor's rule (a non-empty block is causal iff the mask is causal
    and its global row-block id equals its column-block id,
    ``orchestrated_attn/orchestrated_attn_impl.py:91``); ``q_block_offset`` is the global
    block index of the first query block of this shard.  Each block is refined to
    (block/tile)^2 tiles by the rule of ``search_algo/bsa_config.py:177-194`` and emitted in
    the row-major order of ``search_algo/dependent_graph.py:235-240``."""
    if tile != TILE:
        raise ValueError(f"kernel tile is {TILE}, got {tile}")
    if block % tile != 0 or block <= 0:
        raise ValueError(f"block ({block}) must be a positive multiple of {tile}")
    m = np.asarray(block_mask)
    if m.ndim != 2:
        raise ValueError("block_mask must be 2-D [n_qblocks, n_kblocks]")
    m = apply_causal_rule(m.astype(np.uint8), causal, q_block_offset)
    rate = block // tile
    lib = _lib.load()
    nqb, nkb = m.shape
    mp = m.ctypes.data_as(ctypes.c_void_p)
    nqt, nkt, nnz = c_int64(), c_int64(), c_int64()
    _lib.check(lib.ua_tilelist_size(mp, nqb, nkb, rate, ctypes.byref(nqt), ctypes.byref(nkt), ctypes.byref(nnz)),
               "ua_tilelist_size")
    nqt, nkt, nnz = nqt.value, nkt.value, nnz.value
    arrs = dict(row_ptr=np.zeros(nqt + 1, np.int32), col_idx=np.zeros(nnz, np.int32), flag=np.zeros(nnz, np.uint8),
                col_ptr=np.zeros(nkt + 1, np.int32), row_idx=np.zeros(nnz, np.int32), cflag=np.zeros(nnz, np.uint8),
                q_order=np.zeros(nqt, np.int32), k_order=np.zeros(nkt, np.int32))
    ptrs = [arrs[n].ctypes.data_as(ctypes.c_void_p) for n in _HOST_FIELDS]
    _lib.check(lib.ua_tilelist_build(mp, nqb, nkb, rate, *ptrs), "ua_tilelist_build")
    return TileList(n_qtiles=nqt, n_ktiles=nkt, **arrs)


def build_tile_list_device(block_mask_dev, block: int = 512, nnz: Optional[int] = None, check: bool = False):
    """Device-side builder: ``block_mask_dev`` is a uint8 CUDA tensor [n_qblocks, n_kblocks]
    (values 0/1/2, causal rule already applied).  Returns a dict of device tensors with the
    same contents as ``build_tile_list(...).on(device)``.  ``nnz`` (from a host-side size
    query) trims the arrays; without it they are sized to the upper bound.  ``check`` reads back
    the builder's count of invalid mask entries (this synchronises) and raises if it is not 0."""
    import torch
    m = block_mask_dev
    if m.dtype != torch.uint8 or m.dim() != 2 or not m.is_cuda or not m.is_contiguous():
        raise ValueError("block_mask_dev must be a contiguous 2-D uint8 CUDA tensor")
    rate = block // TILE
    nqb, nkb = m.shape
    nqt, nkt = nqb * rate, nkb * rate
    cap = nnz if nnz is not None else nqt * nkt
    alloc = -(-max(cap, 1) // 4) * 4   # non-NULL for an empty list; flag arrays padded to whole 32-bit words
    dev = m.device
    i32 = dict(dtype=torch.int32, device=dev)
    u8 = dict(dtype=torch.uint8, device=dev)
    out = dict(row_ptr=torch.empty(nqt + 1, **i32), col_idx=torch.empty(alloc, **i32), flag=torch.empty(alloc, **u8),
               col_ptr=torch.empty(nkt + 1, **i32), row_idx=torch.empty(alloc, **i32), cflag=torch.empty(alloc, **u8),
               q_order=torch.empty(nqt, **i32), k_order=torch.empty(nkt, **i32))
    work = torch.empty(nqt + nkt + 7, **i32)
    lib = _lib.load()
    with torch.cuda.device(dev):
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.ua_tilelist_build_device(m.data_ptr(), nqb, nkb, rate,
                                                *[out[n].data_ptr() for n in _HOST_FIELDS],
                                                work.data_ptr(), st), "ua_tilelist_build_device")
    if check and int(work[nqt + nkt + 2].item()) != 0:
        raise ValueError(f"block mask holds {int(work[nqt + nkt + 2].item())} entries other than 0 (EMPTY), 1 (FULL), 2 (CAUSAL)")
    for n in ("col_idx", "flag", "row_idx", "cflag"):
        out[n] = out[n][:cap]
    return out
