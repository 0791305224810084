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
from typing import Tuple

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
        B, S, Nh, _ = q_shape
        self.lse = lse if lse is not None else torch.full((B, Nh, S), float("-inf"), dtype=FULL_DTYPE, device=buf.device)

    def reduce(self, other: "OutputRowFwd") -> None:
        from .ops import merge_partials
        merge_partials([self.O, other.O], [self.lse, other.lse], out=self.O, lse=self.lse)


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
    """``reduce`` for gradient packs: the running sum is kept in fp32 beside the bf16 pack (the
    accumulation the reference specifies, ``ring_flash_attn/ring_flash_attn.py:110-118``: partial
    gradients are added into fp32 buffers and cast once), and ``data`` always holds its bf16
    rounding.  Summing in bf16 instead loses about half a bit per partial."""
    data: torch.Tensor
    _acc = None

    def reduce(self, other) -> None:
        if self._acc is None:
            self._acc = self.data.to(FULL_DTYPE)
        self._acc.add_(other.data)            # bf16 -> fp32 promotion happens inside the add
        self.data.copy_(self._acc)


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
