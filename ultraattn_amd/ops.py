"""Block-sparse attention operators on one MI355X: forward, backward, merge of partials.

Host side of the C ABI in ``include/ultraattn.h``.  Tensors follow the reference's tile
kernel (``orchestrated_attn/orchestrated_attn_impl.py:326`` comment): q, o, do, dq
``[B, Sq, Nh, 128]`` bf16; k, v, dk, dv ``[B, Skv, Nh, 128]`` bf16; lse, delta ``[B, Nh, Sq]``
fp32.  Everything runs on the current CUDA(HIP) stream; nothing synchronises.
"""
import ctypes
from typing import Optional, Sequence, Tuple, Union

import numpy as np
import torch

from . import _lib
from .tilelist import TILE, TileList, build_tile_list

HEAD_DIM = 128


def _check_qkv(name: str, t: torch.Tensor, seq_multiple: int = TILE) -> None:
    if not t.is_cuda:
        raise ValueError(f"{name} must be a CUDA (HIP) tensor")
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name} must be bfloat16, got {t.dtype}")
    if t.dim() != 4 or t.shape[-1] != HEAD_DIM:
        raise ValueError(f"{name} must be [B, S, Nh, {HEAD_DIM}], got {tuple(t.shape)}")
    if t.stride(-1) != 1:
        raise ValueError(f"{name}: head_dim axis must be contiguous")
    if t.shape[1] % seq_multiple != 0:
        raise ValueError(f"{name}: sequence length {t.shape[1]} is not a multiple of {seq_multiple}")


def _tiles_for(tiles: Union[TileList, np.ndarray, torch.Tensor], q, k, block, causal, q_block_offset) -> TileList:
    if isinstance(tiles, TileList):
        tl = tiles
    else:
        if isinstance(tiles, torch.Tensor):
            tiles = tiles.cpu().numpy()
        m = np.asarray(tiles)
        if block is None:
            if q.shape[1] % m.shape[0] != 0:
                raise ValueError("cannot infer block size: Sq is not a multiple of the mask's rows")
            block = q.shape[1] // m.shape[0]
        tl = build_tile_list(m, block=block, causal=causal, q_block_offset=q_block_offset)
    if tl.n_qtiles * TILE != q.shape[1] or tl.n_ktiles * TILE != k.shape[1]:
        raise ValueError(f"tile list is {tl.n_qtiles}x{tl.n_ktiles} tiles but Sq={q.shape[1]}, Skv={k.shape[1]}")
    return tl


def bsa_fwd(q, k, v, tiles, softmax_scale: Optional[float] = None, causal: bool = False,
            q_block_offset: int = 0, out: Optional[torch.Tensor] = None, block: Optional[int] = None,
            lse: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Block-sparse flash-attention forward -> (out, lse).

    ``tiles`` is a ``TileList`` or a block mask (0/1/2 or bool; ``causal`` and
    ``q_block_offset`` then apply the executor's diagonal rule).  One launch replaces the
    per-rectangle ``_flash_attn_forward`` calls of ``fwd_comp_func``
    (``orchestrated_attn/orchestrated_attn_impl.py:320-338``).  ``out`` is written in place
    when given (the fork's ``out=`` argument)."""
    for n, t in (("q", q), ("k", k), ("v", v)):
        _check_qkv(n, t)
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    tl = _tiles_for(tiles, q, k, block, causal, q_block_offset)
    B, Sq, Nh, D = q.shape
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if out is None:
        out = torch.empty_like(q)
    else:
        _check_qkv("out", out)
        if out.shape != q.shape:
            raise ValueError("out must have q's shape")
    if lse is None:
        lse = torch.empty(B, Nh, Sq, dtype=torch.float32, device=q.device)
    elif lse.shape != (B, Nh, Sq) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("lse must be a contiguous fp32 [B, Nh, Sq] tensor")
    d = tl.on(q.device)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.ua_bsa_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                            d["row_ptr"].data_ptr(), d["col_idx"].data_ptr(), d["flag"].data_ptr(),
                            d["q_order"].data_ptr(), B, Nh, tl.n_qtiles, tl.n_ktiles, tl.nnz, D,
                            _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(out),
                            float(softmax_scale), st)
    _lib.check(rc, "ua_bsa_fwd")
    return out, lse


def softmax_delta(out, dout, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
    """delta = rowsum(dout * out) as fp32 [B, Nh, Sq]: the ``softmax_d`` input of the fork's
    backward (``orchestrated_attn/orchestrated_attn_impl.py:595``)."""
    _check_qkv("out", out, 1)
    _check_qkv("dout", dout, 1)
    if out.shape != dout.shape:
        raise ValueError("out and dout must have the same shape")
    B, Sq, Nh, D = out.shape
    if delta is None:
        delta = torch.empty(B, Nh, Sq, dtype=torch.float32, device=out.device)
    lib = _lib.load()
    with torch.cuda.device(out.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.ua_bsa_bwd_delta(out.data_ptr(), dout.data_ptr(), delta.data_ptr(), B, Sq, Nh, D,
                                  _lib.strides3(out), _lib.strides3(dout), st)
    _lib.check(rc, "ua_bsa_bwd_delta")
    return delta


def bsa_bwd(dout, q, k, v, out, lse, tiles, softmax_scale: Optional[float] = None, causal: bool = False,
            dq=None, dk=None, dv=None, softmax_d: Optional[torch.Tensor] = None, q_block_offset: int = 0,
            block: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Block-sparse backward -> (dq, dk, dv), written in place when the buffers are given
    (as ``_flash_attn_backward`` does, ``orchestrated_attn/orchestrated_attn_impl.py:578-596``).
    ``lse`` (and ``softmax_d`` when given; then ``out`` is ignored and may be None, the
    reference passes a dummy) are the rows' global statistics."""
    for n, t in (("dout", dout), ("q", q), ("k", k), ("v", v)):
        _check_qkv(n, t)
    tl = _tiles_for(tiles, q, k, block, causal, q_block_offset)
    B, Sq, Nh, D = q.shape
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if lse.shape != (B, Nh, Sq) or lse.dtype != torch.float32 or not lse.is_contiguous():
        raise ValueError("lse must be a contiguous fp32 [B, Nh, Sq] tensor")
    if softmax_d is None:
        if out is None:
            raise ValueError("either out or softmax_d is required")
        softmax_d = softmax_delta(out, dout)
    elif softmax_d.shape != (B, Nh, Sq) or softmax_d.dtype != torch.float32 or not softmax_d.is_contiguous():
        raise ValueError("softmax_d must be a contiguous fp32 [B, Nh, Sq] tensor")
    dq = torch.empty_like(q) if dq is None else dq
    dk = torch.empty_like(k) if dk is None else dk
    dv = torch.empty_like(v) if dv is None else dv
    for n, t, ref in (("dq", dq, q), ("dk", dk, k), ("dv", dv, v)):
        _check_qkv(n, t)
        if t.shape != ref.shape:
            raise ValueError(f"{n} has shape {tuple(t.shape)}, expected {tuple(ref.shape)}")
    d = tl.on(q.device)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.ua_bsa_bwd_dkdv(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(),
                                 softmax_d.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                                 d["col_ptr"].data_ptr(), d["row_idx"].data_ptr(), d["cflag"].data_ptr(),
                                 d["k_order"].data_ptr(), B, Nh, tl.n_qtiles, tl.n_ktiles, tl.nnz, D,
                                 _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(dout),
                                 _lib.strides3(dk), _lib.strides3(dv), float(softmax_scale), st)
        _lib.check(rc, "ua_bsa_bwd_dkdv")
        rc = lib.ua_bsa_bwd_dq(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), lse.data_ptr(),
                               softmax_d.data_ptr(), dq.data_ptr(),
                               d["row_ptr"].data_ptr(), d["col_idx"].data_ptr(), d["flag"].data_ptr(),
                               d["q_order"].data_ptr(), B, Nh, tl.n_qtiles, tl.n_ktiles, tl.nnz, D,
                               _lib.strides3(q), _lib.strides3(k), _lib.strides3(v), _lib.strides3(dout),
                               _lib.strides3(dq), float(softmax_scale), st)
        _lib.check(rc, "ua_bsa_bwd_dq")
    return dq, dk, dv


def merge_partials(outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor],
                   out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None):
    """LSE-weighted merge of partial outputs -> (out, lse): one pass in place of the chain of
    ``update_out_and_lse`` calls (``ring_flash_attn/utils.py:38-52, 78-99``).
    outs[p]: contiguous [B, S, Nh, 128] bf16; lses[p]: contiguous [B, Nh, S] fp32."""
    P = len(outs)
    if P == 0 or P != len(lses):
        raise ValueError("need as many lses as outs, at least one")
    B, S, Nh, D = outs[0].shape
    for o_, l_ in zip(outs, lses):
        _check_qkv("partial out", o_, 1)
        if o_.shape != outs[0].shape or not o_.is_contiguous():
            raise ValueError("partial outs must be contiguous and of equal shape")
        if l_.shape != (B, Nh, S) or l_.dtype != torch.float32 or not l_.is_contiguous():
            raise ValueError("partial lses must be contiguous fp32 [B, Nh, S]")
    out = torch.empty_like(outs[0]) if out is None else out
    lse = torch.empty_like(lses[0]) if lse is None else lse
    if out.shape != outs[0].shape or not out.is_contiguous() or out.dtype != torch.bfloat16:
        raise ValueError("out must be a contiguous bf16 tensor of the partials' shape")
    if lse.shape != (B, Nh, S) or not lse.is_contiguous() or lse.dtype != torch.float32:
        raise ValueError("lse must be a contiguous fp32 [B, Nh, S] tensor")
    op = (ctypes.c_void_p * P)(*[t.data_ptr() for t in outs])
    lp = (ctypes.c_void_p * P)(*[t.data_ptr() for t in lses])
    lib = _lib.load()
    with torch.cuda.device(out.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.ua_merge(op, lp, P, out.data_ptr(), lse.data_ptr(), B, S, Nh, D, st)
    _lib.check(rc, "ua_merge")
    return out, lse


def grad_accumulate(partial: torch.Tensor, out: Optional[torch.Tensor], acc: Optional[torch.Tensor] = None,
                    init_from_out: bool = False) -> None:
    """One step of the gradient accumulation that the reference specifies
    (``ring_flash_attn/ring_flash_attn.py:110-118``) and its packs leave as stubs
    (``orchestrated_attn/utils.py:260-262, 296-298``), as one kernel (``ua_grad_accumulate``):

    * ``acc`` (fp32) given: ``acc += partial`` and ``out = bf16(acc)`` (``out`` may be None);
      with ``init_from_out`` the sum starts from ``out``: ``acc = float(out) + partial``;
    * no ``acc``: ``out = bf16(float(out) + partial)``.
    ``partial`` and ``out`` are contiguous bf16 tensors of equal size, ``acc`` contiguous fp32."""
    n = partial.numel()
    for name, t, dt in (("partial", partial, torch.bfloat16), ("out", out, torch.bfloat16), ("acc", acc, torch.float32)):
        if t is None:
            continue
        if not t.is_cuda or t.dtype != dt or not t.is_contiguous() or t.numel() != n:
            raise ValueError(f"{name} must be a contiguous {dt} CUDA tensor of {n} elements")
    lib = _lib.load()
    with torch.cuda.device(partial.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.ua_grad_accumulate(acc.data_ptr() if acc is not None else None, partial.data_ptr(),
                                    out.data_ptr() if out is not None else None, n, int(init_from_out), st)
    _lib.check(rc, "ua_grad_accumulate")


def grad_sum(parts: Sequence[torch.Tensor], out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """``out = bf16(scale * sum(parts))`` with the sum carried in fp32, one pass (``ua_grad_sum``).
    parts: 1..16 contiguous ``[B, S, Nh, 128]`` tensors, all bf16 or all fp32; ``out`` bf16, may be a
    strided view (head_dim contiguous)."""
    if not parts:
        raise ValueError("need at least one partial gradient")
    dt = parts[0].dtype
    if dt not in (torch.bfloat16, torch.float32):
        raise TypeError("partial gradients must be bfloat16 or float32")
    for t in parts:
        if not t.is_cuda or t.dtype != dt or t.shape != parts[0].shape or not t.is_contiguous() or t.dim() != 4 \
                or t.shape[-1] != HEAD_DIM:
            raise ValueError("partial gradients must be contiguous [B, S, Nh, 128] CUDA tensors of one dtype and shape")
    B, S, Nh, D = parts[0].shape
    if out is None:
        out = torch.empty(parts[0].shape, dtype=torch.bfloat16, device=parts[0].device)
    _check_qkv("out", out, 1)
    if out.shape != parts[0].shape:
        raise ValueError("out must have the partials' shape")
    pp = (ctypes.c_void_p * len(parts))(*[t.data_ptr() for t in parts])
    lib = _lib.load()
    with torch.cuda.device(out.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.ua_grad_sum(pp, len(parts), int(dt == torch.float32), out.data_ptr(), B, S, Nh, D,
                             _lib.strides3(out), float(scale), st)
    _lib.check(rc, "ua_grad_sum")
    return out


def _strides_bsh(t: torch.Tensor, layout: str):
    """(batch, token, head) element strides of a statistics tensor given as [B, S, Nh, 1]
    ('bsh1') or [B, Nh, S] ('bhs'), or of a [B, S, Nh, D] row tensor ('rows')."""
    if layout == "bhs":
        return (ctypes.c_int64 * 3)(t.stride(0), t.stride(2), t.stride(1))
    return (ctypes.c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))


def _stat_layout(t: torch.Tensor, B: int, S: int, Nh: int, name: str) -> str:
    if t.dtype != torch.float32 or not t.is_cuda:
        raise TypeError(f"{name} must be a float32 CUDA tensor")
    if t.dim() == 4 and tuple(t.shape) == (B, S, Nh, 1):
        return "bsh1"
    if t.dim() == 3 and tuple(t.shape) == (B, Nh, S):
        return "bhs"
    raise ValueError(f"{name} must be [B, S, Nh, 1] or [B, Nh, S] = ({B}, {S}, {Nh}), got {tuple(t.shape)}")


def _check_rows(name: str, t: torch.Tensor):
    if not t.is_cuda or t.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"{name} must be a bfloat16 or float32 CUDA tensor")
    if t.dim() != 4 or t.shape[-1] != HEAD_DIM or t.stride(-1) != 1:
        raise ValueError(f"{name} must be [B, S, Nh, {HEAD_DIM}] with a contiguous last axis, got {tuple(t.shape)}")


def update_out_and_lse(out: Optional[torch.Tensor], lse: Optional[torch.Tensor], block_out: torch.Tensor,
                       block_lse: torch.Tensor, slice_=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Drop-in for ``update_out_and_lse`` of the ring / hierarchy executors
    (``ring_flash_attn/utils.py:78-99``; call sites ``hierarchy_attn/hierarchy_attn_impl.py:64-81``):
    folds one more partial ``(block_out [B,Sb,Nh,D], block_lse [B,Nh,Sb])`` into the running
    ``(out [B,S,Nh,D], lse [B,S,Nh,1])`` and returns the pair.

    * first call (``out is None``): returns ``block_out`` and ``block_lse`` as ``[B,S,Nh,1]``, as the
      reference does (``slice_`` is then an error);
    * ``slice_`` (an index for both ``out`` and ``lse``, e.g. ``(slice(None), slice(S//2, None))``):
      the rows it selects are updated in place, in ``out``'s dtype;
    * otherwise new tensors are returned and ``out`` is fp32, which is what the reference's
      expression yields (fp32 statistics times bf16 rows).
    One kernel (``ua_merge_update``) in place of the reference's eight element-wise launches; the
    arithmetic is max-stabilised and treats ``lse = -inf`` as "no keys", which the literal formula
    does not (it agrees with it on every input where that one is finite).  ``block_lse`` may also
    come as ``[B,Sb,Nh,1]`` (the hierarchy executor's ``forward`` closure, ``:40-53``)."""
    if out is None:
        if slice_ is not None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        if block_lse.dim() == 3:
            block_lse = block_lse.transpose(-2, -1).unsqueeze(dim=-1)
        return block_out, block_lse
    _check_rows("out", out)
    _check_rows("block_out", block_out)
    if slice_ is not None:
        tgt_out, tgt_lse = out[slice_], lse[slice_]
        if tgt_out.untyped_storage().data_ptr() != out.untyped_storage().data_ptr() or \
                tgt_lse.untyped_storage().data_ptr() != lse.untyped_storage().data_ptr():
            # the reference assigns `out[slice_] = ...`, which writes through any index; a kernel can
            # only write through a view
            raise ValueError("slice_ must select a view of out and lse (slices, not index lists or tensors)")
        new_out, new_lse = tgt_out, tgt_lse                    # views: written in place
    else:
        tgt_out, tgt_lse = out, lse
        new_out = torch.empty(out.shape, dtype=torch.float32, device=out.device)
        new_lse = torch.empty(lse.shape, dtype=torch.float32, device=out.device)
    _check_rows("out[slice_]", tgt_out)
    B, S, Nh, D = tgt_out.shape
    if tuple(block_out.shape) != (B, S, Nh, D):
        raise ValueError(f"block_out is {tuple(block_out.shape)}, the rows to update are {(B, S, Nh, D)}")
    l_lay = _stat_layout(tgt_lse, B, S, Nh, "lse")
    b_lay = _stat_layout(block_lse, B, S, Nh, "block_lse")
    lib = _lib.load()
    with torch.cuda.device(out.device):
        st = torch.cuda.current_stream().cuda_stream
        rc = lib.ua_merge_update(tgt_out.data_ptr(), tgt_lse.data_ptr(), block_out.data_ptr(), block_lse.data_ptr(),
                                 new_out.data_ptr(), new_lse.data_ptr(), B, S, Nh, D,
                                 int(tgt_out.dtype == torch.float32), int(block_out.dtype == torch.float32),
                                 int(new_out.dtype == torch.float32),
                                 _strides_bsh(tgt_out, "rows"), _strides_bsh(tgt_lse, l_lay),
                                 _strides_bsh(block_out, "rows"), _strides_bsh(block_lse, b_lay),
                                 _strides_bsh(new_out, "rows"), _strides_bsh(new_lse, l_lay), st)
    _lib.check(rc, "ua_merge_update")
    return (out, lse) if slice_ is not None else (new_out, new_lse)
