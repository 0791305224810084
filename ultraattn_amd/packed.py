"""Zero-copy packed row / column buffers: views carved out of one flat bf16 tensor, in the
layout of the reference's ``Integrated_Data`` family (``orchestrated_attn/utils.py:25-298``) and
of ``create_buf_dict`` (``search_algo/benchmark.py:231-283``).  These are what travels between
devices in the reference, so they are also what the kernels must read and write in place: every
view below can be handed to ``bsa_fwd`` / ``bsa_bwd`` / ``softmax_delta`` directly.

Forward:  row in  = [Q]          col in = [K | V]      row out = [O]
Backward: row in  = [Q | dO | D (fp32) | lse]          col in = [K | V]
          row out = [dQ]                               col out = [dK | dV]
"""
import math
from typing import Iterable, Optional, Tuple

import torch

FULL_DTYPE = torch.float32          # orchestrated_attn/global_vars.py:4


def _take(buf: torch.Tensor, start: int, numel: int) -> torch.Tensor:
    if buf.dim() != 1 or buf.dtype != torch.bfloat16:
        raise ValueError("the backing buffer must be a flat bfloat16 tensor")
    if start + numel > buf.numel():
        raise ValueError(f"buffer too small: need {start + numel} elements, have {buf.numel()}")
    return buf[start:start + numel]


class InputRowFwd:
    """``Input_Row_Fwd`` (``orchestrated_attn/utils.py:38-54``): data = Q."""

    def __init__(self, buf: torch.Tensor, q_shape: Tuple[int, int, int, int]):
        self.data = _take(buf, 0, math.prod(q_shape))
        self.Q = self.data.view(q_shape)

    @staticmethod
    def numel(q_shape) -> int:
        return math.prod(q_shape)


class InputColFwd:
    """``Input_Col_Fwd`` / ``Input_Col_Bwd`` (``orchestrated_attn/utils.py:57-82, 210-235``):
    data = [K | V]."""

    def __init__(self, buf: torch.Tensor, k_shape: Tuple[int, int, int, int]):
        n = math.prod(k_shape)
        self.data = _take(buf, 0, 2 * n)
        self.K = self.data[:n].view(k_shape)
        self.V = self.data[n:].view(k_shape)

    @staticmethod
    def numel(k_shape) -> int:
        return 2 * math.prod(k_shape)


InputColBwd = InputColFwd


class OutputRowFwd:
    """``Output_Row_Fwd`` (``orchestrated_attn/utils.py:84-134``): data = O.  The reference
    carries no LSE here and leaves ``reduce`` empty; this one keeps the fp32 LSE beside the
    view and implements the commented formula (``:120-133``) with the merge kernel."""

    def __init__(self, buf: torch.Tensor, q_shape: Tuple[int, int, int, int], lse: torch.Tensor = None):
        self.data = _take(buf, 0, math.prod(q_shape))
        self.O = self.data.view(q_shape)
        self._lse = lse

    @property
    def lse(self) -> torch.Tensor:
        """fp32 [B, Nh, S]; allocated (as "no keys seen", -inf) on first use when none was given."""
        if self._lse is None:
            B, S, Nh, _ = self.O.shape
            self._lse = torch.full((B, Nh, S), float("-inf"), dtype=FULL_DTYPE, device=self.data.device)
        return self._lse

    @lse.setter
    def lse(self, value: torch.Tensor) -> None:
        self._lse = value

    def reduce(self, other: "OutputRowFwd") -> None:
        from .ops import merge_partials
        merge_partials([self.O, other.O], [self.lse, other.lse], out=self.O, lse=self.lse)


class OutputColFwd:
    """``Output_Col_Fwd`` (``orchestrated_attn/utils.py:137-146``): the forward produces nothing
    per column; the class exists so that the buffer dictionary has all four corners."""

    def __init__(self, buf: torch.Tensor = None, k_shape=None):
        self.data = None

    @staticmethod
    def numel(k_shape) -> int:
        return 0


class InputRowBwd:
    """``Input_Row_Bwd`` (``orchestrated_attn/utils.py:148-188``): data = [Q | dO | D | lse] with
    D stored as fp32 in two bf16 slots per element (``:173-188``; offsets
    ``[0, Qn, 2Qn, 2Qn+2L, ...]`` as at ``orchestrated_attn_impl.py:490``).

    The reference gives ``lse`` ONE bf16 slot per element (``tot_numel = 2Qn + 3L``), an
    artefact of a harness that never reads it back; the kernels produce and need fp32 LSE, so
    the default here is two slots (``lse_slots=2``, ``2Qn + 4L`` elements).  ``lse_slots=1``
    reproduces the reference's footprint with a bf16 ``lse`` view (layout checks only)."""

    def __init__(self, buf: torch.Tensor, q_shape: Tuple[int, int, int, int], lse_slots: int = 2):
        if lse_slots not in (1, 2):
            raise ValueError("lse_slots must be 1 or 2")
        B, S, Nh, _ = q_shape
        qn, ln = math.prod(q_shape), B * Nh * S
        self.offsets = (0, qn, 2 * qn, 2 * qn + 2 * ln, 2 * qn + (2 + lse_slots) * ln)
        self.data = _take(buf, 0, self.offsets[-1])
        self.Q = self.data[:qn].view(q_shape)
        self.dO = self.data[qn:2 * qn].view(q_shape)
        self.D = self.data[2 * qn:2 * qn + 2 * ln].view(FULL_DTYPE).view(B, Nh, S)
        tail = self.data[2 * qn + 2 * ln:]
        self.lse = tail.view(FULL_DTYPE).view(B, Nh, S) if lse_slots == 2 else tail.view(B, Nh, S)

    @staticmethod
    def numel(q_shape, lse_slots: int = 2) -> int:
        B, S, Nh, _ = q_shape
        return 2 * math.prod(q_shape) + (2 + lse_slots) * B * Nh * S

    def fill_delta(self, out: torch.Tensor) -> torch.Tensor:
        """D = rowsum(dO * O) written straight into the pack (one HBM-bound kernel)."""
        from .ops import softmax_delta
        return softmax_delta(out, self.dO, delta=self.D)


class _Fp32Accumulated:
    """``reduce`` for gradient packs, the accumulation the reference specifies
    (``ring_flash_attn/ring_flash_attn.py:110-118``: partial gradients are added into fp32 buffers
    and cast once) and leaves commented out in its packs.

    The pack is a view into a persistent buffer that kernels and receives rewrite in place, so no
    fp32 state outlives a reduction chain: ``begin_reduce()`` opens one (the running sum then
    lives in fp32, in ``acc`` when the caller supplies the buffer), every ``reduce(other)`` adds
    one partial and leaves the bf16 rounding of the sum in ``data``, ``end_reduce()`` drops the
    fp32 sum.  Outside a chain ``reduce`` is stateless: ``data = bf16(float(data) + other)``,
    which costs about half a bit per partial but can never mix in a stale sum."""
    data: torch.Tensor
    _acc = None
    _acc_live = False

    def begin_reduce(self, acc: torch.Tensor = None) -> None:
        n = self.data.numel()
        if acc is None:
            acc = torch.empty(n, dtype=FULL_DTYPE, device=self.data.device)
        if acc.dtype != FULL_DTYPE or acc.numel() < n or not acc.is_contiguous() or acc.device != self.data.device:
            raise ValueError(f"acc must be a contiguous float32 tensor of at least {n} elements on the pack's device")
        self._acc = acc.view(-1)[:n]
        self._acc_live = False            # the first reduce() initialises it from data

    def end_reduce(self) -> None:
        self._acc = None
        self._acc_live = False

    def reduce(self, other) -> None:
        from .ops import grad_accumulate
        if self._acc is None:
            grad_accumulate(other.data, self.data)
        else:
            grad_accumulate(other.data, self.data, acc=self._acc, init_from_out=not self._acc_live)
            self._acc_live = True


class OutputRowBwd(_Fp32Accumulated):
    """``Output_Row_Bwd`` (``orchestrated_attn/utils.py:237-262``): data = dQ; ``reduce`` is the
    accumulation the reference leaves commented out (``:262``), done in fp32."""

    def __init__(self, buf: torch.Tensor, q_shape: Tuple[int, int, int, int]):
        self.data = _take(buf, 0, math.prod(q_shape))
        self.dQ = self.data.view(q_shape)


class OutputColBwd(_Fp32Accumulated):
    """``Output_Col_Bwd`` (``orchestrated_attn/utils.py:264-298``): data = [dK | dV]; ``reduce``
    (``:296-298``) accumulates in fp32."""

    def __init__(self, buf: torch.Tensor, k_shape: Tuple[int, int, int, int]):
        n = math.prod(k_shape)
        self.data = _take(buf, 0, 2 * n)
        self.dK = self.data[:n].view(k_shape)
        self.dV = self.data[n:].view(k_shape)


def _permute_cols(entry: str, src: torch.Tensor, n_chunks: int, k_shape, out: torch.Tensor = None) -> torch.Tensor:
    from . import _lib
    B, S, Nh, D = k_shape
    inner = S * Nh * D
    n = 2 * n_chunks * B * inner
    if src.dim() != 1 or src.dtype != torch.bfloat16 or not src.is_cuda or src.numel() < n:
        raise ValueError(f"the column buffer must be a flat bfloat16 CUDA tensor of at least {n} elements")
    out = torch.empty(n, dtype=torch.bfloat16, device=src.device) if out is None else out
    if out.dim() != 1 or out.dtype != torch.bfloat16 or out.device != src.device or out.numel() < n:
        raise ValueError(f"out must be a flat bfloat16 tensor of at least {n} elements on the source's device")
    lib = _lib.load()
    with torch.cuda.device(src.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = getattr(lib, entry)(src.data_ptr(), out.data_ptr(), n_chunks, B, inner, st)
    _lib.check(rc, entry)
    return out


def gather_cols(buf: torch.Tensor, n_chunks: int, k_shape, out: torch.Tensor = None) -> InputColFwd:
    """Fused-rectangle column input: ``buf`` holds ``n_chunks`` received column chunks, each
    ``[K | V]`` of shape ``k_shape`` (B, Skv, Nh, D): ``[Y, 2, B, Skv, Nh, D]``.  Returns the
    ``InputColFwd`` over ``[2, B, Y*Skv, Nh, D]`` — one K and one V across all chunks — produced
    by one HBM-bound copy kernel in place of
    ``view(Y,2,B,Skv,Nh,D).transpose(0,1).transpose(1,2).flatten(2,3).contiguous()``
    (``orchestrated_attn/orchestrated_attn_impl.py:269, 512``)."""
    B, S, Nh, D = k_shape
    data = _permute_cols("ua_cols_gather", buf, n_chunks, k_shape, out)
    return InputColFwd(data, (B, n_chunks * S, Nh, D))


def scatter_cols(col_out: OutputColBwd, n_chunks: int, k_shape, out: torch.Tensor = None) -> torch.Tensor:
    """Inverse for the column output of a fused rectangle: ``col_out.data`` is ``[dK | dV]`` over
    ``Y*Skv`` keys (``[2, B, Y*Skv, Nh, D]``); returns the flat ``[Y, 2, B, Skv, Nh, D]`` buffer
    of per-chunk ``[dK | dV]`` that the column reduce-scatter sends
    (``oc.view(2, Y, K_nelem).transpose(0,1).contiguous()``,
    ``orchestrated_attn/orchestrated_attn_impl.py:548``)."""
    return _permute_cols("ua_cols_scatter", col_out.data, n_chunks, k_shape, out)


def _scaled(shape: Tuple[int, int, int, int], n_chunks: int) -> Tuple[int, int, int, int]:
    """Shape of ``n_chunks`` partitions side by side (``get_Q_shape_from_da_config`` /
    ``get_K_shape_from_da_config``, ``orchestrated_attn/utils.py:25-29``)."""
    return (shape[0], shape[1] * n_chunks, shape[2], shape[3])


def create_buf_dict(q_shape, k_shape, fob: int, tensor_buf: torch.Tensor, comp_keys: Iterable = (),
                    fused_xy: Optional[Tuple[int, int]] = None, level_rank: int = 0,
                    batch_degrees: Tuple[int, int] = (1, 1), lse_slots: int = 1) -> dict:
    """Carves the packs of one execution plan out of ``tensor_buf`` (flat bf16), with the keys and
    offsets of the reference's ``create_buf_dict`` (``search_algo/benchmark.py:231-334``).

    ``q_shape`` / ``k_shape``: ``(bs, S_per_partition, Nh, D)`` of one row / column partition;
    ``fob`` 0 forward, 1 backward; ``batch_degrees`` the (row, column) partitions per kernel of
    the level above.

    General graph (``fused_xy=None``): ``(('i'|'o', 'r'|'c'), n) -> pack`` over ``n`` partitions
    for ``n = 1`` and for every ``low_bds`` that the ``Comp_Kernel`` keys ``(b, h, rid, cid, gpu)``
    in ``comp_keys`` need (ids may be tuples, the fused rectangles of
    ``search_algo/graph_transformation_engine.py:83``); as in the reference every pack starts at
    offset 0 of the same buffer (``:254-283``: the harness times kernels, the addresses are
    dummies), plus ``graph_type``, ``tensor_buf``, ``inp_row``, ``inp_col``, ``out_row``, ``out_col``.

    Fused X x Y graph (``fused_xy=(X, Y)``): the flat slices ``ir | ic | or | oc`` with
    ``ir_nelems = bs*Sq*Nh*D`` (forward) or ``bs*Sq*Nh*(2D + 2 + lse_slots)`` (backward: Q, dO, D, lse),
    ``ic_nelems = bs*Skv*Nh*2D``, ``or_nelems = bs*Sq*Nh*D``, ``oc_nelems = 0 | bs*Skv*Nh*2D``, the
    totals ``*_tot = *_nelems * X`` (rows) or ``* Y`` (columns), for the backward the second row
    buffer (``ir`` = the extra one, ``ir_`` = the first, ``:318-323``), and ``inp_row`` / ``inp_col`` =
    this rank's pack inside ``ir`` / ``ic`` (x = rank % X, y = rank // X, ``:326-329``).

    ``lse_slots=1`` is the reference's footprint (its ``lse`` view is bf16, an artefact of a harness
    that never reads it back); ``lse_slots=2`` keeps a usable fp32 ``lse`` in every backward row pack."""
    if fob not in (0, 1):
        raise ValueError("fob must be 0 (forward) or 1 (backward)")
    if len(batch_degrees) != 2:
        raise ValueError(f"Invalid batch_degrees: {batch_degrees}")
    bs, Sq, Nh, D = q_shape
    Skv, Nhg = k_shape[1], k_shape[2]          # the reference sizes the column packs with the K/V head count (Nhg)
    row_in = (lambda buf, n: InputRowFwd(buf, _scaled(q_shape, n))) if fob == 0 else \
        (lambda buf, n: InputRowBwd(buf, _scaled(q_shape, n), lse_slots=lse_slots))
    col_in = lambda buf, n: InputColFwd(buf, _scaled(k_shape, n))
    row_out = (lambda buf, n: OutputRowFwd(buf, _scaled(q_shape, n))) if fob == 0 else \
        (lambda buf, n: OutputRowBwd(buf, _scaled(q_shape, n)))
    col_out = (lambda buf, n: OutputColFwd()) if fob == 0 else (lambda buf, n: OutputColBwd(buf, _scaled(k_shape, n)))
    if fused_xy is None:
        d = {}

        def add_rows(n):
            if (("i", "r"), n) not in d:
                d[(("i", "r"), n)] = row_in(tensor_buf, batch_degrees[0] * n)
                d[(("o", "r"), n)] = row_out(tensor_buf, batch_degrees[0] * n)

        def add_cols(n):
            if (("i", "c"), n) not in d:
                d[(("i", "c"), n)] = col_in(tensor_buf, batch_degrees[1] * n)
                d[(("o", "c"), n)] = col_out(tensor_buf, batch_degrees[1] * n)
        add_rows(1)
        add_cols(1)
        for key in comp_keys:
            rid, cid = key[2], key[3]
            add_rows(len(rid) if isinstance(rid, tuple) else 1)
            add_cols(len(cid) if isinstance(cid, tuple) else 1)
        d.update(graph_type="general", tensor_buf=tensor_buf, inp_row=d[(("i", "r"), 1)], inp_col=d[(("i", "c"), 1)],
                 out_row=d[(("o", "r"), 1)], out_col=d[(("o", "c"), 1)])
        return d
    X, Y = fused_xy
    sq, skv = Sq * batch_degrees[0], Skv * batch_degrees[1]
    ir_nelems = bs * sq * Nh * (D if fob == 0 else 2 * D + 2 + lse_slots)
    ic_nelems = bs * skv * Nhg * 2 * D
    or_nelems = bs * sq * Nh * D
    oc_nelems = 0 if fob == 0 else bs * skv * Nhg * 2 * D
    ir_tot, ic_tot, or_tot, oc_tot = ir_nelems * X, ic_nelems * Y, or_nelems * X, oc_nelems * Y
    end = ir_tot + ic_tot + or_tot + oc_tot
    buf = _take(tensor_buf, 0, end + (ir_tot if fob == 1 else 0))
    d = {"ir": buf[:ir_tot], "ic": buf[ir_tot:ir_tot + ic_tot], "or": buf[ir_tot + ic_tot:ir_tot + ic_tot + or_tot],
         "oc": buf[ir_tot + ic_tot + or_tot:end],
         "ir_nelems": ir_nelems, "ic_nelems": ic_nelems, "or_nelems": or_nelems, "oc_nelems": oc_nelems,
         "ir_tot": ir_tot, "ic_tot": ic_tot, "or_tot": or_tot, "oc_tot": oc_tot, "graph_type": "fused"}
    if fob == 1:
        d["ir_"] = d["ir"]
        d["ir"] = buf[end:end + ir_tot]
    x, y = level_rank % X, level_rank // X
    d["inp_row"] = row_in(d["ir"][ir_nelems * x:ir_nelems * (x + 1)], batch_degrees[0])
    d["inp_col"] = col_in(d["ic"][ic_nelems * y:ic_nelems * (y + 1)], batch_degrees[1])
    return d
