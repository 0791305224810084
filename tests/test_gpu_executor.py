"""Executor and packed buffers on the GPU: the reference's per-GPU shares, computed one after the
other on this GPU and reduced, reproduce the whole block-sparse attention."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import attn_oracle as ao
from tests.gpu_util import ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs, oracle_fwd_bwd, seeded_inputs
from ultraattn_amd import masks, packed
from ultraattn_amd.executor import BlockSparseExecutor, comp_kernels_from_schedule

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("which", [0, 9, 13])
def test_all_gpu_shares_reduce_to_the_whole(which, golden_dir):
    ref = json.load(open(os.path.join(golden_dir, "reference_data.json")))
    a = ref["allocations"][which]
    table, alloc = np.array(a["block_table"], np.uint8), np.array(a["allocation"])
    chunk, nh = 128, 2
    q, k, v, do = seeded_inputs(table, chunk, seed=which, nh=nh)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    keys = comp_kernels_from_schedule(alloc)
    execs = [BlockSparseExecutor.from_comp_kernels(keys, *table.shape, chunk, causal=False, rank=g, softmax_scale=SCALE)
             for g in range(alloc.max() + 1)]
    parts = [e.forward(qd, kd, vd) for e in execs]
    out, lse = BlockSparseExecutor.reduce_fwd(parts)
    ro, rl, rq, rk, rv = oracle_fwd_bwd(q, k, v, do, table, chunk)
    assert max_abs(out, ro) <= ATOL_O and lse_rel_err(lse, rl) <= RTOL_LSE
    grads = [e.backward(dod, qd, kd, vd, out, lse) for e in execs]       # global out / lse for every share
    dq = BlockSparseExecutor.reduce_bwd([g[0] for g in grads])
    dk = BlockSparseExecutor.reduce_bwd([g[1] for g in grads])
    dv = BlockSparseExecutor.reduce_bwd([g[2] for g in grads])
    assert max_abs(dq, rq) <= ATOL_O and max_abs(dk, rk) <= ATOL_O and max_abs(dv, rv) <= ATOL_O


def test_schedule_table_and_kernel_tiles():
    table = masks.config_streaming_shard(4, 16, 3)
    sched = np.where(table != 0, 5, -1)
    chunk = 128
    q, k, v, _ = seeded_inputs(table, chunk, seed=3)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    one = BlockSparseExecutor.from_schedule_table(sched, table, rank=5, chunk=chunk, softmax_scale=SCALE)
    four = BlockSparseExecutor.from_schedule_table(sched, table, rank=5, chunk=chunk, softmax_scale=SCALE, kernel_tiles=4)
    none = BlockSparseExecutor.from_schedule_table(sched, table, rank=1, chunk=chunk, softmax_scale=SCALE)
    assert len(four.kernel_tiles) == 4 and none.tiles.nnz == 0
    o1, l1 = one.forward(qd, kd, vd)
    o4, l4 = four.forward(qd, kd, vd)
    ro, rl = ao.dense_fwd(q, k, v, SCALE, ao.element_mask(table, chunk))
    assert max_abs(o1, ro) <= ATOL_O and max_abs(o4, ro) <= ATOL_O
    assert lse_rel_err(l1, rl) <= RTOL_LSE and lse_rel_err(l4, rl) <= RTOL_LSE
    o0, l0 = none.forward(qd, kd, vd)
    assert (o0 == 0).all() and torch.isinf(l0).all()


def test_kernels_run_in_place_on_packed_buffers():
    """Forward and backward straight on the packed row / column views, D filled in the pack."""
    table = masks.config_causal(2)
    chunk, nh = 128, 2
    q, k, v, do = seeded_inputs(table, chunk, seed=11, nh=nh)
    qs = tuple(q.shape)
    flat = lambda n: torch.zeros(n, dtype=torch.bfloat16, device=DEV)
    row = packed.InputRowBwd(flat(packed.InputRowBwd.numel(qs)), qs)
    col = packed.InputColBwd(flat(packed.InputColBwd.numel(qs)), qs)
    orow = packed.OutputRowFwd(flat(packed.InputRowFwd.numel(qs)), qs)
    gq = packed.OutputRowBwd(flat(packed.InputRowFwd.numel(qs)), qs)
    gc = packed.OutputColBwd(flat(packed.InputColBwd.numel(qs)), qs)
    row.Q.copy_(q); row.dO.copy_(do); col.K.copy_(k); col.V.copy_(v)
    ex = BlockSparseExecutor(table, chunk, softmax_scale=SCALE)
    ex.forward(row.Q, col.K, col.V, out=orow.O, lse=row.lse)
    row.fill_delta(orow.O)
    ex.backward(row.dO, row.Q, col.K, col.V, None, row.lse, dq=gq.dQ, dk=gc.dK, dv=gc.dV, softmax_d=row.D)
    torch.cuda.synchronize()
    ro, rl, rq, rk, rv = oracle_fwd_bwd(q, k, v, do, table, chunk)
    assert max_abs(orow.O, ro) <= ATOL_O and lse_rel_err(row.lse, rl) <= RTOL_LSE
    assert (row.D.cpu() - ao.softmax_delta(orow.O.cpu(), do)).abs().max() < 1e-3
    assert max_abs(gq.dQ, rq) <= ATOL_O and max_abs(gc.dK, rk) <= ATOL_O and max_abs(gc.dV, rv) <= ATOL_O
    # reduce() of the output packs: merge for O, sum for gradients
    other = packed.OutputRowFwd(flat(packed.InputRowFwd.numel(qs)), qs)
    other.O.copy_(orow.O); other.lse.copy_(row.lse); orow.lse = row.lse.clone()
    orow.reduce(other)                                     # two equal partials: O unchanged, LSE + log 2
    assert max_abs(orow.O, ro) <= ATOL_O
    assert (orow.lse - row.lse - np.log(2.0)).abs().max().item() < 1e-4
    g2 = packed.OutputRowBwd(gq.data.clone(), qs)
    gq.reduce(g2)
    assert max_abs(gq.dQ, 2 * rq) <= 2 * ATOL_O
