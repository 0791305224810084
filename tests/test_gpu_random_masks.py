"""Forward and backward on seeded random block tables (EMPTY / FULL / CAUSAL anywhere, rectangular
grids, block sizes 128 / 256 / 384, 1..16 heads) against the dense oracle: exercises list lengths,
empty rows and columns, causal tiles off the diagonal and the dispatch order's corner cases."""
import numpy as np
import pytest
import torch

from tests.gpu_util import ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs, oracle_fwd_bwd
from ultraattn_amd import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(seed):
    r = np.random.RandomState(1000 + seed)
    nqb, nkb = int(r.randint(1, 6)), int(r.randint(1, 6))
    block = int(r.choice([128, 128, 256, 384]))
    nh = int(r.choice([1, 2, 3, 8, 16]))
    batch = int(r.choice([1, 1, 2]))
    density = r.choice([0.3, 0.6, 0.9])
    mask = (r.rand(nqb, nkb) < density).astype(np.uint8)
    mask[(r.rand(nqb, nkb) < 0.25) & (mask == 1)] = 2
    return mask, block, nh, batch


@pytest.mark.parametrize("seed", range(16))
def test_random_block_table(seed):
    mask, block, nh, batch = _case(seed)
    g = torch.Generator().manual_seed(seed)
    mk = lambda n: torch.randn(batch, n * block, nh, 128, generator=g, dtype=torch.float32).to(torch.bfloat16)
    q, k, v, do = mk(mask.shape[0]), mk(mask.shape[1]), mk(mask.shape[1]), mk(mask.shape[0])
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    o, lse = ops.bsa_fwd(qd, kd, vd, mask, SCALE, block=block)
    dq, dk, dv = ops.bsa_bwd(dod, qd, kd, vd, o, lse, mask, SCALE, block=block)
    ro, rl, rq, rk, rv = oracle_fwd_bwd(q, k, v, do, mask, block)
    assert max_abs(o, ro) <= ATOL_O
    assert lse_rel_err(lse, rl) <= RTOL_LSE
    assert max_abs(dq, rq) <= ATOL_O
    assert max_abs(dk, rk) <= ATOL_O
    assert max_abs(dv, rv) <= ATOL_O
