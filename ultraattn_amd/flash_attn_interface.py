"""Drop-in for the two functions the reference's executors import from the flash-attention
fork: ``from flash_attn.flash_attn_interface import _flash_attn_forward, _flash_attn_backward``
(``orchestrated_attn/orchestrated_attn_impl.py:7-8``, ``hierarchy_attn/hierarchy_attn_impl.py:3``).

Same positional/keyword arguments, including the fork's ``out=`` (forward) and ``softmax_d=``
(backward).  A call is one dense rectangle: it goes to ``ua_dense_fwd`` / ``ua_dense_bwd``, which
enumerate the tiles themselves (no tile list is built, copied or cached) and cut rectangles with
few tile lines into parts that fill the device.  Nothing here synchronises or copies from the
host, so a call (a first call at a new shape included) can be captured into a HIP graph.
"""
from typing import Dict, Optional, Tuple

import torch

from . import _lib
from .ops import HEAD_DIM, _check_qkv, softmax_delta
from .tilelist import TILE

# (device index, stream handle) -> uint8 tensor holding the partial results of split calls.  Calls
# on one stream run in order, so they can share it; it only ever grows.  At most _MAX_WORKSPACES are
# kept (least recently used first out: stream handles come and go).
_workspaces: Dict[Tuple[int, int], torch.Tensor] = {}
_MAX_WORKSPACES = 16
_captured = []             # workspaces that a captured graph may replay into: never released
_initialised = set()


def _check_unsupported(dropout_p, window_size, alibi_slopes, return_softmax=False):
    if dropout_p != 0:
        raise NotImplementedError("dropout_p must be 0")
    if tuple(window_size) != (-1, -1):
        raise NotImplementedError("window_size must be (-1, -1)")
    if alibi_slopes is not None:
        raise NotImplementedError("alibi_slopes must be None")
    if return_softmax:
        raise NotImplementedError("return_softmax needs dropout_p > 0, which is unsupported")


def _workspace(lib, q, k, backward: bool, stream: int):
    """(pointer, bytes) of this stream's workspace, grown to what the shape needs to split;
    (None, 0) for shapes that never split."""
    need = lib.ua_dense_workspace_bytes(q.shape[0], q.shape[2], q.shape[1], k.shape[1], int(backward))
    if need <= 0:
        return None, 0
    key = (q.device.index, stream)
    ws = _workspaces.pop(key, None)
    if ws is None or ws.numel() < need:
        ws = torch.empty(need, dtype=torch.uint8, device=q.device)
    _workspaces[key] = ws                      # most recently used last
    while len(_workspaces) > _MAX_WORKSPACES:
        _workspaces.pop(next(iter(_workspaces)))
    if torch.cuda.is_current_stream_capturing() and not any(w is ws for w in _captured):
        _captured.append(ws)                   # outlives its cache entry: the graph keeps writing to it
    return ws.data_ptr(), ws.numel()


def _prepare(q):
    lib = _lib.load()
    if q.device.index not in _initialised:
        with torch.cuda.device(q.device):
            _lib.check(lib.ua_init(), "ua_init")      # per-device lookups, done once and outside any capture
        _initialised.add(q.device.index)
    return lib


def _check_shapes(q, k, v, causal):
    for n, t in (("q", q), ("k", k), ("v", v)):
        _check_qkv(n, t)
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2]:
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
    if causal and (k.shape[1] - q.shape[1]) % TILE != 0:
        raise NotImplementedError("causal with Skv - Sq not a multiple of 128")


def _flash_attn_forward(q, k, v, dropout_p, softmax_scale, causal, window_size=(-1, -1),
                        alibi_slopes=None, return_softmax=False, out=None):
    """-> (out, q, k, v, out_padded, softmax_lse, S_dmask, rng_state); callers use [0] and [5]
    (``orchestrated_attn_impl.py:326``, ``hierarchy_attn_impl.py:41``).  With ``causal`` and
    Sq != Skv the diagonal is aligned to the bottom-right corner, as flash-attn (2.1 and later)
    does: query i sees key j iff j <= i + Skv - Sq."""
    _check_unsupported(dropout_p, window_size, alibi_slopes, return_softmax)
    _check_shapes(q, k, v, causal)
    B, Sq, Nh, D = q.shape
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if out is None:
        out = torch.empty_like(q)
    else:
        _check_qkv("out", out)
        if out.shape != q.shape:
            raise ValueError("out must have q's shape")
    lse = torch.empty(B, Nh, Sq, dtype=torch.float32, device=q.device)
    lib = _prepare(q)
    with torch.cuda.device(q.device):
        st = torch.cuda.current_stream().cuda_stream
        ws, ws_bytes = _workspace(lib, q, k, False, st)
        rc = lib.ua_dense_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                              B, Nh, Sq, k.shape[1], D, _lib.strides3(q), _lib.strides3(k), _lib.strides3(v),
                              _lib.strides3(out), float(softmax_scale), int(bool(causal)), ws, ws_bytes, st)
    _lib.check(rc, "ua_dense_fwd")
    return out, q, k, v, out, lse, None, None


def _flash_attn_backward(dout, q, k, v, out, softmax_lse, dq, dk, dv, dropout_p, softmax_scale, causal,
                         window_size=(-1, -1), alibi_slopes=None, deterministic=False, rng_state=None,
                         softmax_d: Optional[torch.Tensor] = None):
    """Writes dq, dk, dv in place (allocates the ones passed as None); returns (dq, dk, dv, softmax_d).  With ``softmax_d`` given
    ``out`` is ignored (the reference passes a dummy, ``orchestrated_attn_impl.py:583``).
    The kernels are deterministic regardless of ``deterministic``."""
    _check_unsupported(dropout_p, window_size, alibi_slopes)
    _check_shapes(q, k, v, causal)
    _check_qkv("dout", dout)
    B, Sq, Nh, D = q.shape
    if dout.shape != q.shape:
        raise ValueError("dout must have q's shape")
    if softmax_scale is None:
        softmax_scale = D ** -0.5
    if softmax_lse.shape != (B, Nh, Sq) or softmax_lse.dtype != torch.float32 or not softmax_lse.is_contiguous():
        raise ValueError("softmax_lse must be a contiguous fp32 [B, Nh, Sq] tensor")
    if softmax_d is None:
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
    lib = _prepare(q)
    with torch.cuda.device(q.device):
        st = torch.cuda.current_stream().cuda_stream
        ws, ws_bytes = _workspace(lib, q, k, True, st)
        rc = lib.ua_dense_bwd(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), softmax_lse.data_ptr(),
                              softmax_d.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                              B, Nh, Sq, k.shape[1], D, _lib.strides3(q), _lib.strides3(k), _lib.strides3(v),
                              _lib.strides3(dout), _lib.strides3(dq), _lib.strides3(dk), _lib.strides3(dv),
                              float(softmax_scale), int(bool(causal)), ws, ws_bytes, st)
    _lib.check(rc, "ua_dense_bwd")
    return dq, dk, dv, softmax_d
