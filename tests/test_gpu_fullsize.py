"""Full-size parity on the GPU: configuration 1's exact workload against the CPU block loop, and
one WHOLE head (every row of O, LSE, dQ, dK, dV) of the 128k configurations against the oracle's
tile formula evaluated on the device."""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as ao
from tests.gpu_util import (ATOL_O, RTOL_LSE, SCALE, head_reference_on_device, lse_rel_err, max_abs,
                            oracle_fwd_bwd, seeded_inputs)
from ultraattn_amd import masks, ops
from ultraattn_amd.tilelist import build_tile_list

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.mark.parametrize("mask,block", [(masks.config_strided(8, 2, 4), 128), (masks.config_global_local(6, 1, 2), 256),
                                        (masks.config_streaming_shard(3, 8, 2), 128)])
def test_device_head_reference_equals_the_cpu_oracle(mask, block):
    """Pins the checker used at full size: on small masks it must reproduce the CPU oracle
    (dense fp64 formula + autograd) to fp32 rounding."""
    q, k, v, do = seeded_inputs(mask, block, 11, nh=3)
    ro, rl, rq, rk, rv = oracle_fwd_bwd(q, k, v, do, mask, block)
    for h in range(3):
        O, LSE, dQ, dK, dV = head_reference_on_device(q.to(DEV), k.to(DEV), v.to(DEV), do.to(DEV), mask, block, h)
        assert max_abs(O, ro[0, :, h]) <= 2e-5 and lse_rel_err(LSE, rl[0, h]) <= 1e-5
        assert max_abs(dQ, rq[0, :, h]) <= 1e-4 and max_abs(dK, rk[0, :, h]) <= 1e-4 and max_abs(dV, rv[0, :, h]) <= 1e-4


def test_config1_exact_workload_vs_cpu_block_loop():
    """Configuration 1 as stated: B=1, S=8192, Nh=8, d=128, 16x16 causal grid of 512-token blocks,
    Q/K/V ~ N(0,1) from a seed, scale 1/sqrt(128).  The CPU side is the reference's block loop
    (oracle.block_loop_fwd / block_loop_bwd, fp32) on the same bf16-rounded values."""
    mask, block, nh = masks.config_causal(16), 512, 8
    q, k, v, do = seeded_inputs(mask, block, 0, nh=nh)
    ro, rl = ao.block_loop_fwd(q, k, v, mask, block, SCALE)
    rq, rk, rv = ao.block_loop_bwd(do, q, k, v, ro, rl, mask, block, SCALE)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    tl = build_tile_list(mask, block)
    assert tl.nnz == 2080 and tl.n_causal == 64
    o, lse = ops.bsa_fwd(qd, kd, vd, tl, SCALE)
    dq, dk, dv = ops.bsa_bwd(dod, qd, kd, vd, o, lse, tl, SCALE)
    torch.cuda.synchronize()
    assert max_abs(o, ro) <= ATOL_O and lse_rel_err(lse, rl) <= RTOL_LSE
    assert max_abs(dq, rq) <= ATOL_O and max_abs(dk, rk) <= ATOL_O and max_abs(dv, rv) <= ATOL_O


@pytest.mark.parametrize("cfg,head", [("c2", 17), ("c3", 5), ("c4", 26), ("c5", 9)])
def test_whole_head_at_full_size(cfg, head):
    """Configurations 2 to 5 at their real shape (Nh=32; S=32768, 131072, 131072 and the streaming
    shard's 65536 query rows against 524288 keys): every row of one head, forward and backward."""
    mask = {"c2": masks.config_causal(64), "c3": masks.config_strided(), "c4": masks.config_global_local(),
            "c5": masks.config_streaming_shard()}[cfg]
    block, nh = 512, 32
    g = torch.Generator(device=DEV).manual_seed(0)
    mk = lambda n: torch.randn(1, n * block, nh, 128, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(mask.shape[0]), mk(mask.shape[1]), mk(mask.shape[1]), mk(mask.shape[0])
    tl = build_tile_list(mask, block)
    o, lse = ops.bsa_fwd(q, k, v, tl, SCALE)
    dq, dk, dv = ops.bsa_bwd(do, q, k, v, o, lse, tl, SCALE)
    torch.cuda.synchronize()
    O, LSE, dQ, dK, dV = head_reference_on_device(q, k, v, do, mask, block, head)
    assert lse_rel_err(lse[0, head], LSE) <= RTOL_LSE
    for name, got, ref in (("o", o, O), ("dq", dq, dQ), ("dk", dk, dK), ("dv", dv, dV)):
        err = (got[0, :, head].float() - ref).abs()
        assert torch.isfinite(err).all(), name
        assert err.max().item() <= ATOL_O, (name, err.max().item(), int(err.argmax()) // 128)
