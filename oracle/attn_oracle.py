"""fp32/fp64 CPU restatement of the attention tile, its backward and the LSE merge.

Test infrastructure (see oracle/__init__.py).  Shapes follow the reference's call sites:
q, o, do, dq: [B, Sq, Nh, D]; k, v, dk, dv: [B, Skv, Nh, D]; lse, delta: [B, Nh, Sq].
"""
import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

NEG_INF = float("-inf")


def tile_fwd(q, k, v, scale: float, causal: bool = False, dtype=torch.float32):
    """One dense rectangular tile: O = softmax(scale*Q K^T [+ causal]) V, LSE = logsumexp.

    Stands in for ``_flash_attn_forward`` as called at
    ``orchestrated_attn/orchestrated_attn_impl.py:326-337`` and
    ``hierarchy_attn/hierarchy_attn_impl.py:41-51`` (returns [0]=O and [5]=lse of the 8-tuple).
    ``causal`` masks key j > query i on local indices: the reference only sets it for
    row-chunk id == column-chunk id tiles (``orchestrated_attn_impl.py:91``), which are square.
    Rows with no visible key give O = 0 and LSE = -inf.
    """
    q_, k_, v_ = (t.to(dtype) for t in (q, k, v))
    s = torch.einsum("bqhd,bkhd->bhqk", q_, k_) * scale
    if causal:
        sq, sk = s.shape[-2:]
        keep = torch.arange(sk)[None, :] <= torch.arange(sq)[:, None]
        s = s.masked_fill(~keep, NEG_INF)
    lse = torch.logsumexp(s, dim=-1)                              # [B, Nh, Sq]
    p = torch.exp(s - lse.masked_fill(lse == NEG_INF, 0.0)[..., None])
    o = torch.einsum("bhqk,bkhd->bqhd", p, v_)
    return o, lse


def dense_fwd(q, k, v, scale: float, keep: torch.Tensor, dtype=torch.float32):
    """Attention under an explicit element mask keep[Sq, Skv] (True = visible).

    Independent cross-check of the block loop: no tiling, no merge."""
    q_, k_, v_ = (t.to(dtype) for t in (q, k, v))
    s = torch.einsum("bqhd,bkhd->bhqk", q_, k_) * scale
    s = s.masked_fill(~keep[None, None], NEG_INF)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse.masked_fill(lse == NEG_INF, 0.0)[..., None])
    o = torch.einsum("bhqk,bkhd->bqhd", p, v_)
    return o, lse


def dense_bwd_autograd(q, k, v, do, scale: float, keep: torch.Tensor, dtype=torch.float64):
    """dQ, dK, dV of ``dense_fwd`` by torch.autograd (the reference checks its baselines the
    same way, ``easy_context/dist_flash_attn/lightseq_async_attn.py:489-492``)."""
    q_, k_, v_ = (t.detach().to(dtype).requires_grad_(True) for t in (q, k, v))
    o, _ = dense_fwd(q_, k_, v_, scale, keep, dtype=dtype)
    o.backward(do.to(dtype))
    return q_.grad, k_.grad, v_.grad


def softmax_delta(o, do, dtype=torch.float32):
    """D = rowsum(dO * O) as [B, Nh, Sq]: the ``softmax_d`` the reference precomputes and
    passes to the fork's backward (``orchestrated_attn_impl.py:595``)."""
    return (o.to(dtype) * do.to(dtype)).sum(-1).permute(0, 2, 1).contiguous()


def tile_bwd(do, q, k, v, lse, delta, scale: float, causal: bool = False, dtype=torch.float32):
    """Backward of one dense tile with recompute from the row statistics.

    Stands in for ``_flash_attn_backward(..., softmax_d=D)`` at
    ``orchestrated_attn/orchestrated_attn_impl.py:578-596``.  ``lse`` and ``delta`` are the
    GLOBAL (post-merge) statistics of the rows, identical for every tile of a row, as in
    ``ring_flash_attn/ring_flash_attn.py:91-108``:
        P = exp(scale*QK^T - lse);  dV = P^T dO;  dP = dO V^T;  dS = P*(dP - D);
        dQ = scale*dS K;  dK = scale*dS^T Q.
    """
    q_, k_, v_, do_ = (t.to(dtype) for t in (q, k, v, do))
    lse_, d_ = lse.to(dtype), delta.to(dtype)
    s = torch.einsum("bqhd,bkhd->bhqk", q_, k_) * scale
    if causal:
        sq, sk = s.shape[-2:]
        keep = torch.arange(sk)[None, :] <= torch.arange(sq)[:, None]
        s = s.masked_fill(~keep, NEG_INF)
    p = torch.exp(s - lse_.masked_fill(lse_ == NEG_INF, 0.0)[..., None])
    p = torch.where(torch.isinf(s) & (s < 0), torch.zeros_like(p), p)
    dv = torch.einsum("bhqk,bqhd->bkhd", p, do_)
    dp = torch.einsum("bqhd,bkhd->bhqk", do_, v_)
    ds = p * (dp - d_[..., None])
    dq = torch.einsum("bhqk,bkhd->bqhd", ds, k_) * scale
    dk = torch.einsum("bhqk,bqhd->bkhd", ds, q_) * scale
    return dq, dk, dv


# --------------------------------------------------------------------------------------
# merge  (ring_flash_attn/utils.py:38-52 and 78-99; twin copy hierarchy_attn/utils.py:16-56)
# --------------------------------------------------------------------------------------

def _update_out_and_lse(out, lse, block_out, block_lse):
    """``ring_flash_attn/utils.py:38-52``: lse is [B, S, Nh, 1], block_lse arrives [B, Nh, S].

    new_lse = lse + log(1 + exp(block_lse - lse))
    out     = exp(lse - new_lse) * out + exp(block_lse - new_lse) * block_out
    Literal form: not max-stabilised (overflows for block_lse - lse > ~88 in fp32, NaN for
    -inf partials).  ``merge_partials`` below is the stabilised definition the kernel follows;
    the two agree on all finite, non-overflowing inputs (tested)."""
    block_lse = block_lse.transpose(-2, -1).unsqueeze(dim=-1)
    new_lse = lse + torch.log(1 + torch.exp(block_lse - lse))
    out = torch.exp(lse - new_lse) * out + torch.exp(block_lse - new_lse) * block_out
    return out, new_lse


def update_out_and_lse(out, lse, block_out, block_lse, slice_=None):
    """``ring_flash_attn/utils.py:78-99``: first partial initialises, ``slice_`` updates a
    sub-range of rows in place."""
    if out is None:
        if slice_ is not None:
            raise RuntimeError("first update_out_and_lse should not pass slice_ args")
        out = block_out
        lse = block_lse.transpose(-2, -1).unsqueeze(dim=-1)
    elif slice_ is not None:
        slice_out, slice_lse = out[slice_], lse[slice_]
        slice_out, slice_lse = _update_out_and_lse(slice_out, slice_lse, block_out, block_lse)
        out[slice_], lse[slice_] = slice_out, slice_lse
    else:
        out, lse = _update_out_and_lse(out, lse, block_out, block_lse)
    return out, lse


def merge_partials(outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor], dtype=torch.float32):
    """All-at-once, max-stabilised form of the recurrence above.

    outs[p]: [B, S, Nh, D]; lses[p]: [B, Nh, S].  m = max_p lse_p;
    LSE = m + log(sum_p exp(lse_p - m));  O = sum_p exp(lse_p - LSE) * O_p.
    A partial with lse = -inf (no visible key) is the identity; all -inf gives O = 0, LSE = -inf.
    """
    L = torch.stack([l.to(dtype) for l in lses])                     # [P, B, Nh, S]
    m = L.max(dim=0).values
    m_safe = m.masked_fill(m == NEG_INF, 0.0)
    w = torch.exp(L - m_safe)                                        # [P, B, Nh, S]
    den = w.sum(0)
    lse = m_safe + torch.log(den)
    lse = torch.where(den == 0, torch.full_like(lse, NEG_INF), lse)
    wn = w / den.masked_fill(den == 0, 1.0)
    o = sum(wn[p].permute(0, 2, 1)[..., None] * outs[p].to(dtype) for p in range(len(outs)))
    return o, lse


# --------------------------------------------------------------------------------------
# the block loop: what orchestrated_attn / hierarchy_attn execute on one device
# --------------------------------------------------------------------------------------

def accumulate_gradients(parts: Sequence[torch.Tensor]):
    """The gradient accumulation of ``ring_flash_attn/ring_flash_attn.py:110-118``: the first
    partial is converted to fp32 (``dq = block_dq_buffer.to(torch.float32)``), every later one is
    added into that fp32 buffer (``dq += block_dq_buffer``), and the result is cast to the
    partials' dtype once (``:135``).  Returns (fp32 sum, its cast)."""
    acc = parts[0].to(torch.float32)
    for p in parts[1:]:
        acc = acc + p            # bf16 -> fp32 promotion, as `dq += block` does
    return acc, acc.to(parts[0].dtype)


def block_loop_fwd(q, k, v, block_table: np.ndarray, block: int, scale: float,
                   dtype=torch.float32, q_block_offset: int = 0):
    """Forward over a block table with values 0 EMPTY / 1 FULL / 2 CAUSAL
    (``search_algo/utils.py:140-143``).

    For every active block (i, j) in row-major order (``search_algo/dependent_graph.py:235-240``;
    executed like ``orchestrated_attn/orchestrated_attn_impl.py:348-349`` and
    ``hierarchy_attn/hierarchy_attn_impl.py:86-98``) run one dense tile
    (causal inside the block iff it is CAUSAL, ``orchestrated_attn_impl.py:91``) and fold its
    (O_ij, LSE_ij) into row-block i's accumulator with ``update_out_and_lse``.
    ``q_block_offset`` only documents where the q shard sits in the global grid; the table
    already carries the diagonal as CAUSAL entries.  Returns O [B,Sq,Nh,D], LSE [B,Nh,Sq].
    """
    del q_block_offset
    nqb, nkb = block_table.shape
    B, Sq, Nh, D = q.shape
    assert Sq == nqb * block and k.shape[1] == nkb * block
    o_out = torch.zeros(B, Sq, Nh, D, dtype=dtype)
    lse_out = torch.full((B, Nh, Sq), NEG_INF, dtype=dtype)
    for i in range(nqb):
        rs = slice(i * block, (i + 1) * block)
        out, lse = None, None
        for j in range(nkb):
            t = int(block_table[i, j])
            if t == 0:
                continue
            cs = slice(j * block, (j + 1) * block)
            bo, bl = tile_fwd(q[:, rs], k[:, cs], v[:, cs], scale, causal=(t == 2), dtype=dtype)
            out, lse = update_out_and_lse(out, lse, bo, bl)
        if out is not None:
            o_out[:, rs] = out
            lse_out[:, :, rs] = lse.squeeze(-1).transpose(-2, -1)
    return o_out, lse_out


def block_loop_bwd(do, q, k, v, o, lse, block_table: np.ndarray, block: int, scale: float,
                   dtype=torch.float32):
    """Backward over the same block loop: per active block one ``tile_bwd`` with the global
    lse / D of its rows, accumulated with ``+=`` in the working dtype — the accumulation the
    reference specifies (``ring_flash_attn/ring_flash_attn.py:110-118``) and leaves as a
    stub in ``orchestrated_attn/utils.py:260-262, 296-298``."""
    nqb, nkb = block_table.shape
    delta = softmax_delta(o, do, dtype=dtype)
    dq = torch.zeros(q.shape, dtype=dtype)
    dk = torch.zeros(k.shape, dtype=dtype)
    dv = torch.zeros(v.shape, dtype=dtype)
    for i in range(nqb):
        rs = slice(i * block, (i + 1) * block)
        for j in range(nkb):
            t = int(block_table[i, j])
            if t == 0:
                continue
            cs = slice(j * block, (j + 1) * block)
            a, b, c = tile_bwd(do[:, rs], q[:, rs], k[:, cs], v[:, cs], lse[:, :, rs],
                               delta[:, :, rs], scale, causal=(t == 2), dtype=dtype)
            dq[:, rs] += a
            dk[:, cs] += b
            dv[:, cs] += c
    return dq, dk, dv


def element_mask(block_table: np.ndarray, block: int) -> torch.Tensor:
    """Expand a 0/1/2 block table to keep[Sq, Skv] (True = visible); CAUSAL blocks keep
    local key index <= local query index."""
    nqb, nkb = block_table.shape
    bt = torch.from_numpy(np.ascontiguousarray(block_table).astype(np.int64))
    full = (bt == 1).repeat_interleave(block, 0).repeat_interleave(block, 1)
    caus = (bt == 2).repeat_interleave(block, 0).repeat_interleave(block, 1)
    tri = torch.tril(torch.ones(block, block, dtype=torch.bool)).repeat(nqb, nkb)
    return full | (caus & tri)


def brute_force_fwd(q, k, v, scale, keep):
    """Python-loop fp64 attention for tiny inputs: no einsum, no logsumexp."""
    B, Sq, Nh, D = q.shape
    Sk = k.shape[1]
    o = [[[[0.0] * D for _ in range(Nh)] for _ in range(Sq)] for _ in range(B)]
    lse = [[[NEG_INF] * Sq for _ in range(Nh)] for _ in range(B)]
    qa, ka, va = q.double().tolist(), k.double().tolist(), v.double().tolist()
    for b in range(B):
        for h in range(Nh):
            for i in range(Sq):
                vis = [j for j in range(Sk) if bool(keep[i, j])]
                if not vis:
                    continue
                s = [scale * sum(qa[b][i][h][d] * ka[b][j][h][d] for d in range(D)) for j in vis]
                m = max(s)
                e = [math.exp(x - m) for x in s]
                z = sum(e)
                lse[b][h][i] = m + math.log(z)
                for d in range(D):
                    o[b][i][h][d] = sum(e[t] * va[b][j][h][d] for t, j in enumerate(vis)) / z
    return torch.tensor(o, dtype=torch.float64), torch.tensor(lse, dtype=torch.float64)
