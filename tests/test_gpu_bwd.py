"""Backward parity on the GPU, through the C ABI."""
import os

import numpy as np
import pytest
import torch

from oracle import attn_oracle as ao
from tests.gpu_util import (ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs, oracle_fwd_bwd, seeded_inputs,
                            visible_keys_of_row, visible_rows_of_key)
from ultraattn_amd import masks, ops
from ultraattn_amd.tilelist import build_tile_list

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run_fwd_bwd(q, k, v, do, mask, block):
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    tl = build_tile_list(mask, block)
    o, lse = ops.bsa_fwd(qd, kd, vd, tl, SCALE)
    dq, dk, dv = ops.bsa_bwd(dod, qd, kd, vd, o, lse, tl, SCALE)
    torch.cuda.synchronize()
    return o, lse, dq, dk, dv


@pytest.mark.parametrize("name", ["c1_causal", "c3_strided", "c4_global_local", "c5_streaming"])
def test_golden_twins(name, golden_dir):
    from tests.golden.make_golden import twin_inputs
    g = np.load(os.path.join(golden_dir, f"twin_{name}.npz"))
    mask, block = g["mask"], int(g["block"])
    q, k, v, do = twin_inputs(mask, block, int(g["seed"]))
    _, _, dq, dk, dv = run_fwd_bwd(q, k, v, do, mask, block)
    qr, kr = torch.from_numpy(g["qrows"]).to(DEV), torch.from_numpy(g["krows"]).to(DEV)
    assert max_abs(dq[:, qr], torch.from_numpy(g["dq"])) <= ATOL_O
    assert max_abs(dk[:, kr], torch.from_numpy(g["dk"])) <= ATOL_O
    assert max_abs(dv[:, kr], torch.from_numpy(g["dv"])) <= ATOL_O


CASES = {
    "causal_4x4_b128": (lambda: masks.config_causal(4), 128, 2, 1),
    "causal_2x2_b512": (lambda: masks.config_causal(2), 512, 2, 1),
    "strided_16_b256": (lambda: masks.config_strided(16), 256, 4, 1),
    "global_local_12": (lambda: masks.config_global_local(12, 1, 2), 128, 3, 1),
    "stream_shard": (lambda: masks.config_streaming_shard(4, 16, 3), 128, 2, 1),
    "batch2_heads5": (lambda: masks.config_causal(3), 128, 5, 2),
    "single_causal_tile": (lambda: np.full((1, 1), 2, np.uint8), 128, 1, 1),
    "rect_6x1": (lambda: np.ones((6, 1), np.uint8), 128, 2, 1),
    # every XCD owns whole heads; 3 / 5 / 6 tile rows and columns leave the last dispatch team short
    "heads16_rows3_cols5": (lambda: np.random.RandomState(1).randint(0, 2, size=(3, 5)).astype(np.uint8), 128, 16, 1),
    "heads8_batch2_rows6": (lambda: masks.config_causal(3), 256, 8, 2),
}


@pytest.mark.parametrize("case", list(CASES))
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_bwd_vs_oracle(case, seed):
    make, block, nh, batch = CASES[case]
    mask = make()
    q, k, v, do = seeded_inputs(mask, block, seed, nh=nh, batch=batch)
    _, _, dq, dk, dv = run_fwd_bwd(q, k, v, do, mask, block)
    _, _, rq, rk, rv = oracle_fwd_bwd(q, k, v, do, mask, block)
    assert max_abs(dq, rq) <= ATOL_O
    assert max_abs(dk, rk) <= ATOL_O
    assert max_abs(dv, rv) <= ATOL_O


def test_delta_kernel_and_softmax_d_argument():
    mask = masks.config_causal(2)
    q, k, v, do = seeded_inputs(mask, 128, 1, nh=3, batch=2)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    o, lse = ops.bsa_fwd(qd, kd, vd, mask, SCALE, block=128)
    delta = ops.softmax_delta(o, dod)
    ref = ao.softmax_delta(o.cpu(), do)
    assert (delta.cpu() - ref).abs().max().item() <= 1e-4 * max(1.0, ref.abs().max().item())
    # with softmax_d the `out` argument is ignored: the reference passes a dummy there
    a = ops.bsa_bwd(dod, qd, kd, vd, o, lse, mask, SCALE, block=128)
    b = ops.bsa_bwd(dod, qd, kd, vd, None, lse, mask, SCALE, block=128, softmax_d=delta)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


def test_rows_and_columns_without_tiles_get_zero_gradients():
    mask = np.zeros((3, 3), np.uint8)
    mask[0, 0] = 2
    mask[2, 0] = 1
    q, k, v, do = seeded_inputs(mask, 128, 0)
    _, _, dq, dk, dv = run_fwd_bwd(q, k, v, do, mask, 128)
    assert (dq[:, 128:256] == 0).all() and (dk[:, 128:] == 0).all() and (dv[:, 128:] == 0).all()
    _, _, rq, rk, rv = oracle_fwd_bwd(q, k, v, do, mask, 128)
    assert max_abs(dq, rq) <= ATOL_O and max_abs(dk, rk) <= ATOL_O and max_abs(dv, rv) <= ATOL_O


def test_key_range_split_gradients_add_up():
    """Per kernel tile the backward uses the rows' global lse / delta; summing the tiles'
    gradients (the reduce() of orchestrated_attn/utils.py:260-262, 296-298) gives the whole."""
    mask = masks.config_strided(8, 2, 4)
    q, k, v, do = seeded_inputs(mask, 128, 2)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    o, lse = ops.bsa_fwd(qd, kd, vd, mask, SCALE, block=128)
    delta = ops.softmax_delta(o, dod)
    whole = ops.bsa_bwd(dod, qd, kd, vd, None, lse, mask, SCALE, block=128, softmax_d=delta)
    acc = [torch.zeros_like(t, dtype=torch.float32) for t in whole]
    for cols in (slice(0, 3), slice(3, 8)):
        sub = np.zeros_like(mask)
        sub[:, cols] = mask[:, cols]
        part = ops.bsa_bwd(dod, qd, kd, vd, None, lse, sub, SCALE, block=128, softmax_d=delta)
        for a, p in zip(acc, part):
            a += p.float()
    for a, w in zip(acc, whole):
        assert (a - w.float()).abs().max().item() <= ATOL_O


@pytest.mark.parametrize("cfg", ["c3", "c4"])
def test_full_size_sampled_rows(cfg):
    """Benchmark shapes: sampled query rows (dQ) and key rows (dK, dV) recomputed densely in
    fp32 on the device with the oracle's tile formula, from the kernel's own lse / delta."""
    mask = {"c3": masks.config_strided(), "c4": masks.config_global_local()}[cfg]
    block, nh = 512, 32
    g = torch.Generator(device=DEV).manual_seed(0)
    mk = lambda n: torch.randn(1, n * block, nh, 128, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(256), mk(256), mk(256), mk(256)
    tl = build_tile_list(mask, block)
    o, lse = ops.bsa_fwd(q, k, v, tl, SCALE)
    delta = ops.softmax_delta(o, do)
    dq, dk, dv = ops.bsa_bwd(do, q, k, v, None, lse, tl, SCALE, softmax_d=delta)
    torch.cuda.synchronize()
    for t in (dq, dk, dv):
        assert torch.isfinite(t).all()
    rs = np.random.RandomState(1)
    for row in list(rs.choice(q.shape[1], 10, replace=False)) + [0, 511, 1024, q.shape[1] - 1]:
        h = int(rs.randint(nh))
        vis = visible_keys_of_row(mask, block, int(row)).to(DEV)
        sl = (slice(None), slice(row, row + 1), slice(h, h + 1))
        rq, _, _ = ao.tile_bwd(do[sl], q[sl], k[:, vis, h:h + 1], v[:, vis, h:h + 1],
                               lse[:, h:h + 1, row:row + 1], delta[:, h:h + 1, row:row + 1], SCALE)
        assert (dq[0, row, h].float() - rq[0, 0, 0]).abs().max().item() <= ATOL_O, (row, h)
    for key in list(rs.choice(k.shape[1], 10, replace=False)) + [0, 600, k.shape[1] - 1]:
        h = int(rs.randint(nh))
        vis = visible_rows_of_key(mask, block, int(key)).to(DEV)
        _, rk, rv = ao.tile_bwd(do[:, vis, h:h + 1], q[:, vis, h:h + 1], k[:, key:key + 1, h:h + 1],
                                v[:, key:key + 1, h:h + 1], lse[:, h:h + 1, vis], delta[:, h:h + 1, vis], SCALE)
        assert (dk[0, key, h].float() - rk[0, 0, 0]).abs().max().item() <= ATOL_O, (key, h)
        assert (dv[0, key, h].float() - rv[0, 0, 0]).abs().max().item() <= ATOL_O, (key, h)


def test_stale_lds_contents_do_not_leak_into_gradients():
    """The kernels stage operands in LDS rings and may touch a stage before its first fill; what an
    earlier launch left there (here: NaN everywhere, from a backward over NaN inputs that fills
    every CU) must not reach any result."""
    big = np.ones((8, 8), np.uint8)
    nan = torch.full((1, 8 * 128, 64, 128), float("nan"), dtype=torch.bfloat16, device=DEV)
    lse_nan = torch.zeros(1, 64, 8 * 128, dtype=torch.float32, device=DEV)
    for _ in range(2):
        ops.bsa_fwd(nan, nan, nan, big, SCALE, block=128)
        ops.bsa_bwd(nan, nan, nan, nan, None, lse_nan, big, SCALE, block=128, softmax_d=lse_nan)
    torch.cuda.synchronize()
    for mask in (np.array([[1, 0], [0, 0]], np.uint8), np.array([[2, 0, 0], [1, 2, 0], [1, 0, 1]], np.uint8),
                 np.zeros((2, 2), np.uint8)):
        q, k, v, do = seeded_inputs(mask, 128, 7, nh=8)
        o, lse, dq, dk, dv = run_fwd_bwd(q, k, v, do, mask, 128)
        ro, rl, rq, rk, rv = oracle_fwd_bwd(q, k, v, do, mask, 128)
        for got, ref in ((o, ro), (dq, rq), (dk, rk), (dv, rv)):
            assert torch.isfinite(got.float()).all()
            assert max_abs(got, ref) <= ATOL_O
