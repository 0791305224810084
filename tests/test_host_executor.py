"""Host logic of the executor and of the packed buffers (no GPU): kernel-key -> mask rules and
the buffer layouts of the reference, checked by pointer arithmetic."""
import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import tilelist_oracle as to
from ultraattn_amd import packed
from ultraattn_amd.executor import comp_kernels_from_schedule, mask_from_comp_kernels


def test_causal_rule_over_all_keys():
    """kernel_causal = causal and isinstance(rid, int) and rid == cid (orchestrated_attn_impl.py:91)."""
    n = 4
    for causal in (False, True):
        for rid in range(n):
            for cid in range(n):
                m = mask_from_comp_kernels([(0, 0, rid, cid, 0)], n, n, causal)
                assert m[rid, cid] == (2 if causal and rid == cid else 1) and (m != 0).sum() == 1
    # fused rectangles (tuple ids) are never causal, even on the diagonal, and may be non-contiguous
    m = mask_from_comp_kernels([(0, 0, (0, 2), (0, 3), 1)], n, n, True)
    assert m.tolist() == [[1, 0, 0, 1], [0, 0, 0, 0], [1, 0, 0, 1], [0, 0, 0, 0]]
    with pytest.raises(ValueError):
        mask_from_comp_kernels([(0, 0, 1, 1, 0), (0, 0, (1,), (1,), 0)], n, n, False)


def test_schedule_table_enumeration_and_reference_allocations(golden_dir):
    """Row-major enumeration (dependent_graph.py:235-240) over the reference's own ILP results."""
    ref = json.load(open(os.path.join(golden_dir, "reference_data.json")))
    for a in ref["allocations"]:
        table, alloc = np.array(a["block_table"], np.uint8), np.array(a["allocation"])
        keys = comp_kernels_from_schedule(alloc)
        assert [(k, l) for _, _, k, l, _ in keys] == [(k, l) for k, l, _ in to.enumerate_tiles(table)]
        assert all(g == alloc[k, l] for _, _, k, l, g in keys)
        total = np.zeros_like(table)
        for g in range(alloc.max() + 1):
            mine = mask_from_comp_kernels(keys, *table.shape, causal=False, rank=g)
            assert np.array_equal(mine != 0, alloc == g)
            assert [k[2:4] for k in comp_kernels_from_schedule(alloc, rank=g)] == \
                   [(k, l) for k, l, _ in to.enumerate_tiles(mine)]
            total += mine
        assert np.array_equal(total, table)


def test_packed_layouts_match_the_reference_offsets():
    B, S, Nh, D = 1, 256, 4, 128
    qs, L = (B, S, Nh, D), B * Nh * S
    qn = B * S * Nh * D
    buf = torch.zeros(packed.InputRowBwd.numel(qs) + 8, dtype=torch.bfloat16)
    base = buf.data_ptr()
    row = packed.InputRowBwd(buf, qs)
    # offsets [0, Qn, 2Qn, 2Qn+2L, ...] in bf16 elements (orchestrated_attn_impl.py:490, utils.py:173-188)
    assert row.offsets[:4] == (0, qn, 2 * qn, 2 * qn + 2 * L)
    assert row.Q.data_ptr() == base and row.dO.data_ptr() == base + 2 * qn
    assert row.D.data_ptr() == base + 4 * qn and row.D.dtype == torch.float32 and row.D.shape == (B, Nh, S)
    assert row.lse.data_ptr() == base + 4 * qn + 4 * L and row.lse.dtype == torch.float32
    assert row.data.numel() == 2 * qn + 4 * L
    ref_sized = packed.InputRowBwd(buf, qs, lse_slots=1)         # the reference's footprint: 2Qn + 3L
    assert ref_sized.data.numel() == 2 * qn + 3 * L and ref_sized.lse.dtype == torch.bfloat16
    col = packed.InputColFwd(buf, qs)
    assert col.K.data_ptr() == base and col.V.data_ptr() == base + 2 * qn and col.data.numel() == 2 * qn
    oc = packed.OutputColBwd(buf, qs)
    assert oc.dK.data_ptr() == base and oc.dV.data_ptr() == base + 2 * qn
    # writes through a view land in the flat buffer
    row.D.fill_(1.0)
    assert buf[2 * qn:2 * qn + 2 * L].view(torch.float32).eq(1.0).all() and buf[:2 * qn].eq(0).all()
    with pytest.raises(ValueError):
        packed.InputRowBwd(buf[:100], qs)
    # a fused rectangle of n chunks is the first n*Sp tokens of the same buffer (benchmark.py:271-276)
    two = packed.InputRowFwd(buf, (B, 2 * S // 2, Nh, D))
    assert two.Q.data_ptr() == base


def test_gradient_accumulation_oracle_is_an_fp32_sum_rounded_once():
    """Pins oracle.accumulate_gradients (ring_flash_attn/ring_flash_attn.py:110-118: partial
    dq/dk/dv are added into fp32 buffers and cast once): on bf16 inputs with small integer
    mantissas the fp32 sum is exact, so it must equal the fp64 sum; on random inputs it equals
    torch's fp32 sum of the stack rounded once, and a bf16 running sum gives other bits."""
    from oracle import attn_oracle as ao
    g = torch.Generator().manual_seed(5)
    exact = [torch.randint(-64, 64, (4096,), generator=g).to(torch.bfloat16) for _ in range(8)]
    acc, cast = ao.accumulate_gradients(exact)
    assert torch.equal(acc.double(), torch.stack([p.double() for p in exact]).sum(0))
    parts = [torch.randn(2 * 128 * 2 * 128, generator=g).to(torch.bfloat16) for _ in range(8)]
    acc, cast = ao.accumulate_gradients(parts)
    seq = parts[0].float()
    for p in parts[1:]:
        seq += p.float()
    assert torch.equal(acc, seq) and torch.equal(cast, seq.to(torch.bfloat16))
    assert (acc.double() - torch.stack([p.double() for p in parts]).sum(0)).abs().max() < 1e-5
    naive = parts[0].clone()
    for p in parts[1:]:
        naive.add_(p)
    assert not torch.equal(naive, cast)


def test_create_buf_dict_general_graph_matches_the_reference_layout():
    """search_algo/benchmark.py:246-283: one pack per corner and per low_bds the plan's kernels
    need, every one of them at offset 0 of the same buffer, sized by the partition shapes."""
    qs, ks = (1, 128, 2, 128), (1, 256, 2, 128)
    buf = torch.zeros(1 << 20, dtype=torch.bfloat16)
    base = buf.data_ptr()
    keys = [(0, 0, 1, 1, 0), (0, 0, (0, 2), 3, 0), (0, 0, (0, 1, 2), (1, 3), 0), (0, 0, 4, 0, 1)]
    for fob in (0, 1):
        d = packed.create_buf_dict(qs, ks, fob, buf, comp_keys=keys, batch_degrees=(2, 1), lse_slots=2)
        pack_keys = sorted(k for k in d if isinstance(k, tuple))
        assert pack_keys == sorted([((io, "r"), n) for io in "io" for n in (1, 2, 3)] +
                                   [((io, "c"), n) for io in "io" for n in (1, 2)])
        assert d["graph_type"] == "general" and d["tensor_buf"] is buf
        assert d["inp_row"] is d[(("i", "r"), 1)] and d["out_col"] is d[(("o", "c"), 1)]
        for n in (1, 2, 3):
            rows = d[(("i", "r"), n)]
            assert rows.Q.shape == (1, 128 * 2 * n, 2, 128) and rows.Q.data_ptr() == base
            assert d[(("o", "r"), n)].data.data_ptr() == base
            qn = math.prod(rows.Q.shape)
            if fob == 1:
                L = 1 * 2 * 128 * 2 * n
                assert rows.dO.data_ptr() == base + 2 * qn and rows.D.data_ptr() == base + 4 * qn
                assert rows.lse.data_ptr() == base + 4 * qn + 4 * L and rows.data.numel() == 2 * qn + 4 * L
                assert d[(("o", "r"), n)].dQ.shape == rows.Q.shape
        for n in (1, 2):
            cols = d[(("i", "c"), n)]
            assert cols.K.shape == (1, 256 * n, 2, 128) and cols.K.data_ptr() == base
            assert cols.V.data_ptr() == base + 2 * math.prod(cols.K.shape)
            if fob == 1:
                assert d[(("o", "c"), n)].dV.data_ptr() == cols.V.data_ptr()
            else:
                assert d[(("o", "c"), n)].data is None


def test_create_buf_dict_fused_graph_matches_the_reference_formulas():
    """search_algo/benchmark.py:284-334: ir | ic | or | oc element counts, totals, slices, the second
    row buffer of the backward, and this rank's packs inside ir / ic."""
    bs, Sq, Skv, Nh, D = 1, 64, 128, 2, 128
    qs, ks = (bs, Sq, Nh, D), (bs, Skv, Nh, D)
    X, Y = 2, 3
    buf = torch.zeros(1 << 21, dtype=torch.bfloat16)
    base = buf.data_ptr()
    for fob, slots in ((0, 1), (1, 1), (1, 2)):
        for rank in (0, 1, 4, 5):
            d = packed.create_buf_dict(qs, ks, fob, buf, fused_xy=(X, Y), level_rank=rank, lse_slots=slots)
            ir = bs * Sq * Nh * (D if fob == 0 else 2 * D + 2 + slots)      # the reference: d*2 + 1*(2+1)
            ic = bs * Skv * Nh * 2 * D
            orr = bs * Sq * Nh * D
            oc = 0 if fob == 0 else bs * Skv * Nh * 2 * D
            assert (d["ir_nelems"], d["ic_nelems"], d["or_nelems"], d["oc_nelems"]) == (ir, ic, orr, oc)
            assert (d["ir_tot"], d["ic_tot"], d["or_tot"], d["oc_tot"]) == (ir * X, ic * Y, orr * X, oc * Y)
            first = "ir_" if fob == 1 else "ir"
            assert d[first].data_ptr() == base and d[first].numel() == ir * X
            assert d["ic"].data_ptr() == base + 2 * ir * X and d["ic"].numel() == ic * Y
            assert d["or"].data_ptr() == base + 2 * (ir * X + ic * Y) and d["or"].numel() == orr * X
            assert d["oc"].numel() == oc * Y
            end = ir * X + ic * Y + orr * X + oc * Y
            if fob == 1:
                assert d["oc"].data_ptr() == base + 2 * (ir * X + ic * Y + orr * X)
                assert d["ir"].data_ptr() == base + 2 * end and d["ir"].numel() == ir * X
            x, y = rank % X, rank // X
            assert d["inp_row"].Q.data_ptr() == d["ir"].data_ptr() + 2 * ir * x and d["inp_row"].Q.shape == qs
            assert d["inp_col"].K.data_ptr() == d["ic"].data_ptr() + 2 * ic * y
            assert d["inp_col"].V.data_ptr() == d["inp_col"].K.data_ptr() + 2 * math.prod(ks)
            if fob == 1:
                qn, L = math.prod(qs), bs * Nh * Sq
                assert d["inp_row"].data.numel() == ir and d["inp_row"].D.data_ptr() == d["inp_row"].Q.data_ptr() + 4 * qn
                assert d["inp_row"].lse.dtype == (torch.float32 if slots == 2 else torch.bfloat16)
                assert d["inp_row"].lse.data_ptr() == d["inp_row"].Q.data_ptr() + 4 * qn + 4 * L
    with pytest.raises(ValueError):
        packed.create_buf_dict(qs, ks, 1, buf[:1000], fused_xy=(X, Y))
    with pytest.raises(ValueError):
        packed.create_buf_dict(qs, ks, 2, buf)
