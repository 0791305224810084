"""Executor and packed buffers on the GPU: the reference's per-GPU shares, computed one after the
other on this GPU and reduced, reproduce the whole block-sparse attention."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import attn_oracle as ao
from tests.gpu_util import ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs, oracle_fwd_bwd, seeded_inputs
from ultraattn_amd import masks, ops, packed
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


@pytest.mark.parametrize("make,chunk", [(lambda: masks.config_strided(8, 2, 4), 256), (lambda: masks.config_global_local(6, 1, 2), 128),
                                        (lambda: masks.canonical_block_table(3), 128)])
def test_one_dense_call_per_rectangle_equals_the_single_launch(make, chunk):
    """The reference's way of running a device's share (a dense tile call per chunk pair, partials
    folded with update_out_and_lse) and the single launch over the tile list give the same result."""
    table = make()
    q, k, v, do = seeded_inputs(table, chunk, seed=21, nh=3)
    qd, kd, vd = (t.to(DEV) for t in (q, k, v))
    ex = BlockSparseExecutor(table, chunk, softmax_scale=SCALE)
    o1, l1 = ex.forward(qd, kd, vd)
    o2, l2 = ex.forward_per_rectangle(qd, kd, vd)
    torch.cuda.synchronize()
    keep = ao.element_mask(table, chunk)
    ro, rl = ao.dense_fwd(q, k, v, SCALE, keep)
    assert max_abs(o2, ro) <= ATOL_O and lse_rel_err(l2, rl) <= RTOL_LSE
    assert max_abs(o2, o1.cpu()) <= 8e-3 and lse_rel_err(l2, l1.cpu()) <= 1e-5
    # backward: a dense call per rectangle with the rows' global statistics, fp32 running sums
    dod = do.to(DEV)
    delta = ops.softmax_delta(o1, dod)
    g1 = ex.backward(dod, qd, kd, vd, None, l1, softmax_d=delta)
    g2 = ex.backward_per_rectangle(dod, qd, kd, vd, l1, delta)
    torch.cuda.synchronize()
    want = ao.dense_bwd_autograd(q, k, v, do, SCALE, keep)
    for a, b, w in zip(g1, g2, want):
        # every partial is rounded to bf16 before it is added (as in the reference): the bar scales with
        # the size of the gradients, which on these short rows reach several units
        bar = ATOL_O * max(1.0, float(w.abs().max()))
        assert max_abs(a, w) <= ATOL_O and max_abs(b, w) <= bar and max_abs(b, a.cpu()) <= bar


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


@pytest.mark.parametrize("Y,ks", [(2, (1, 128, 2, 128)), (3, (2, 40, 3, 8)), (1, (1, 8, 1, 8)), (4, (1, 2048, 8, 128))])
def test_column_gather_and_scatter_are_bit_exact(Y, ks):
    from oracle import layout_oracle as lo
    B, S, Nh, D = ks
    n = 2 * Y * B * S * Nh * D
    g = torch.Generator().manual_seed(Y)
    raw = torch.randint(-2 ** 15, 2 ** 15, (n,), generator=g, dtype=torch.int16)
    buf = raw.view(torch.bfloat16).to(DEV)
    col = packed.gather_cols(buf, Y, ks)
    want = lo.cols_gather(raw.numpy(), Y, ks)
    assert col.K.shape == (B, Y * S, Nh, D)
    assert np.array_equal(col.K.cpu().view(torch.int16).numpy(), want[0])
    assert np.array_equal(col.V.cpu().view(torch.int16).numpy(), want[1])
    back = packed.scatter_cols(packed.OutputColBwd(col.data, (B, Y * S, Nh, D)), Y, ks)
    assert np.array_equal(back.cpu().view(torch.int16).numpy(), raw.numpy())
    want_s = lo.cols_scatter(raw.numpy(), Y, ks).reshape(-1)
    got_s = packed.scatter_cols(packed.OutputColBwd(buf, (B, Y * S, Nh, D)), Y, ks)
    assert np.array_equal(got_s.cpu().view(torch.int16).numpy(), want_s)


def test_column_gather_rejects_bad_arguments():
    buf = torch.zeros(4096, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError):       # inner not a multiple of 8 elements
        packed.gather_cols(buf, 2, (1, 3, 1, 4))
    with pytest.raises(RuntimeError):       # source and destination overlap
        packed.gather_cols(buf, 2, (1, 8, 1, 8), out=buf[8:])
    with pytest.raises(ValueError):         # buffer too small
        packed.gather_cols(buf, 2, (1, 128, 2, 128))


def test_fused_rectangle_reads_gathered_columns():
    """Y received column chunks -> gather -> one forward launch over Y*Skv keys equals the oracle on
    the concatenated keys (the X x Y step of orchestrated_attn_impl.py:255-279)."""
    Y, Nh, S = 3, 2, 256
    g = torch.Generator().manual_seed(5)
    q = torch.randn(1, S, Nh, 128, generator=g).to(torch.bfloat16)
    chunks = [torch.randn(2, 1, S, Nh, 128, generator=g).to(torch.bfloat16) for _ in range(Y)]
    buf = torch.stack(chunks).reshape(-1).to(DEV)
    col = packed.gather_cols(buf, Y, (1, S, Nh, 128))
    mask = np.ones((1, Y), np.uint8)
    o, lse = ops.bsa_fwd(q.to(DEV), col.K, col.V, mask, SCALE, block=S)
    k = torch.cat([c[0] for c in chunks], dim=1)
    v = torch.cat([c[1] for c in chunks], dim=1)
    ro, rl = ao.dense_fwd(q, k, v, SCALE, ao.element_mask(mask, S))
    assert max_abs(o, ro) <= ATOL_O and lse_rel_err(lse, rl) <= RTOL_LSE
