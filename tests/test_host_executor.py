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


def test_gradient_packs_accumulate_in_fp32():
    """Eight partial gradients reduced one by one equal the fp32 sum rounded once
    (ring_flash_attn/ring_flash_attn.py:110-118 accumulates partial dq/dk/dv in fp32); a bf16
    running sum does not."""
    shape = (1, 128, 2, 128)
    g = torch.Generator().manual_seed(5)
    parts = [torch.randn(2 * 128 * 2 * 128, generator=g).to(torch.bfloat16) for _ in range(8)]
    want = torch.stack([p.float() for p in parts]).sum(0)
    for cls in (packed.OutputRowBwd, packed.OutputColBwd):
        n = math.prod(shape) * (2 if cls is packed.OutputColBwd else 1)
        packs = [cls(p.clone(), shape) for p in parts]
        for other in packs[1:]:
            packs[0].reduce(other)
        assert torch.equal(packs[0].data, want[:n].to(torch.bfloat16))
        naive = parts[0][:n].clone()
        for p in parts[1:]:
            naive.add_(p[:n])
        assert not torch.equal(naive, packs[0].data)
