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
