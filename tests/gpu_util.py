"""Helpers shared by the GPU parity tests."""
import math

import numpy as np
import torch

from oracle import attn_oracle as ao

# Tolerances of the parity bar: bf16 kernel results against the fp32/fp64 oracle.
ATOL_O = 2e-2         # max-abs on O, dQ, dK, dV
RTOL_LSE = 1e-3       # relative on LSE (denominator max(|lse|, 1) so values near 0 stay meaningful)
SCALE = 1.0 / math.sqrt(128)


def seeded_inputs(mask, block, seed, nh=2, batch=1, d=128, std=1.0):
    """bf16 q, k, v, do from a seeded CPU generator (identical on every machine)."""
    g = torch.Generator().manual_seed(seed)
    nqb, nkb = mask.shape
    mk = lambda n: (torch.randn(batch, n * block, nh, d, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)
    return mk(nqb), mk(nkb), mk(nkb), mk(nqb)


def lse_rel_err(lse, ref):
    lse, ref = lse.detach().cpu().double(), ref.detach().cpu().double()
    fin = torch.isfinite(ref)
    assert torch.equal(torch.isinf(lse) & (lse < 0), ~fin), "-inf pattern of LSE differs"
    if not fin.any():
        return 0.0
    return ((lse[fin] - ref[fin]).abs() / ref[fin].abs().clamp_min(1.0)).max().item()


def max_abs(a, ref):
    return (a.detach().cpu().double() - ref.detach().cpu().double()).abs().max().item()


def oracle_fwd_bwd(q, k, v, do, mask, block, scale=SCALE):
    keep = ao.element_mask(np.asarray(mask), block)
    o, lse = ao.dense_fwd(q, k, v, scale, keep, dtype=torch.float64)
    dq, dk, dv = ao.dense_bwd_autograd(q, k, v, do, scale, keep)
    return o, lse, dq, dk, dv


def visible_keys_of_row(mask, block, row):
    """Boolean [Skv] visibility of one query row under a 0/1/2 block table."""
    bi, li = divmod(row, block)
    types = torch.from_numpy(np.asarray(mask[bi]).astype(np.int64))
    keep = (types == 1).repeat_interleave(block)
    diag = (types == 2).repeat_interleave(block)
    local = torch.arange(block).repeat(mask.shape[1])
    return keep | (diag & (local <= li))


def visible_rows_of_key(mask, block, key):
    bj, lj = divmod(key, block)
    types = torch.from_numpy(np.asarray(mask[:, bj]).astype(np.int64))
    keep = (types == 1).repeat_interleave(block)
    diag = (types == 2).repeat_interleave(block)
    local = torch.arange(block).repeat(mask.shape[0])
    return keep | (diag & (local >= lj))


def head_reference_on_device(q, k, v, do, mask, block, head, scale=SCALE, batch=0):
    """One whole head of a block-sparse attention, forward and backward, by the oracle's tile
    formula (oracle.attn_oracle.tile_fwd / tile_bwd: S = scale Q K^T, causal inside CAUSAL blocks,
    LSE = logsumexp, P = exp(S - LSE), O = P V; dV = P^T dO, dP = dO V^T, dS = P (dP - D),
    dQ = scale dS K, dK = scale dS^T Q with D = rowsum(dO O)) evaluated block row by block row in
    fp32 torch on the tensors' device.  A block row's visible key blocks are concatenated, so no
    merge is involved.  Returns fp32 O [Sq,D], LSE [Sq], dQ [Sq,D], dK [Skv,D], dV [Skv,D].
    Pinned against the CPU oracle on a small mask by tests/test_gpu_fullsize.py."""
    mask = np.asarray(mask)
    nqb, nkb = mask.shape
    dev = q.device
    old = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        Q, K, V, DO = (t[batch, :, head].float() for t in (q, k, v, do))
        O = torch.zeros_like(Q)
        LSE = torch.full((Q.shape[0],), float("-inf"), device=dev)
        dQ, dK, dV = torch.zeros_like(Q), torch.zeros_like(K), torch.zeros_like(V)
        loc = torch.arange(block, device=dev)
        for i in range(nqb):
            cols = np.nonzero(mask[i])[0]
            if len(cols) == 0:
                continue
            rs = slice(i * block, (i + 1) * block)
            kidx = torch.cat([torch.arange(j * block, (j + 1) * block, device=dev) for j in cols])
            Ks, Vs = K[kidx], V[kidx]
            s = (Q[rs] @ Ks.T) * scale
            hide = torch.zeros(block, len(cols) * block, dtype=torch.bool, device=dev)
            for n, j in enumerate(cols):
                if mask[i, j] == 2:
                    hide[:, n * block:(n + 1) * block] = loc[None, :] > loc[:, None]
            s = s.masked_fill(hide, float("-inf"))
            lse = torch.logsumexp(s, dim=-1)
            p = torch.exp(s - lse[:, None])
            o = p @ Vs
            O[rs], LSE[rs] = o, lse
            delta = (DO[rs] * o).sum(-1)
            dp = DO[rs] @ Vs.T
            ds = p * (dp - delta[:, None])
            dQ[rs] = (ds @ Ks) * scale
            dK.index_add_(0, kidx, (ds.T @ Q[rs]) * scale)
            dV.index_add_(0, kidx, p.T @ DO[rs])
    finally:
        torch.backends.cuda.matmul.allow_tf32 = old
    return O, LSE, dQ, dK, dV
