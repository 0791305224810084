"""The hierarchy executor's forward loop on one GPU: the call pattern of ``intra_attn_forward``
(``hierarchy_attn/hierarchy_attn_impl.py:14-103``: a ring over zigzag-sharded ranks, one dense
``_flash_attn_forward`` per step on q, on the first half of k/v, or on the second half of q, each
folded into the running (out, lse [B,S,Nh,1]) by ``update_out_and_lse``, the last case through
``slice_``) with the import lines swapped to this package.  Every "rank" is run in turn; its rows
must equal causal attention over the whole sequence."""
import pytest
import torch

from oracle import attn_oracle as ao
from tests.gpu_util import ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs
from ultraattn_amd.flash_attn_interface import _flash_attn_forward
from ultraattn_amd.ops import update_out_and_lse

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _forward(q, k, v, causal):
    block_out, _, _, _, _, block_lse, _, _ = _flash_attn_forward(q, k, v, 0.0, SCALE, causal=causal,
                                                                 window_size=(-1, -1), alibi_slopes=None, return_softmax=False)
    return block_out, block_lse.transpose(-2, -1).contiguous().unsqueeze(dim=-1)      # [B,S,Nh,D], [B,S,Nh,1]


def _rank_forward(rank, world, shards):
    """One rank's loop: at step s it holds the k/v of rank (rank - s) mod world."""
    q = shards[rank][0]
    half = q.shape[1] // 2
    q1 = q[:, half:]
    out = lse = None
    for step in range(world):
        _, k, v = shards[(rank - step) % world]
        if step == 0:
            block_out, block_lse = _forward(q, k, v, causal=True)
            out, lse = update_out_and_lse(out, lse, block_out, block_lse)
        elif step <= rank:
            block_out, block_lse = _forward(q, k[:, :half], v[:, :half], causal=False)
            out, lse = update_out_and_lse(out, lse, block_out, block_lse)
        else:
            block_out, block_lse = _forward(q1, k, v, causal=False)
            out, lse = update_out_and_lse(out, lse, block_out, block_lse,
                                          slice_=(slice(None), slice(half, None)))
    return out, lse


@pytest.mark.parametrize("world,chunk,nh", [(4, 256, 2), (3, 128, 3)])
def test_zigzag_ring_forward_equals_causal_attention(world, chunk, nh):
    g = torch.Generator().manual_seed(7)
    S = 2 * world * chunk
    q, k, v = (torch.randn(1, S, nh, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    ref_o, ref_lse = ao.dense_fwd(q, k, v, SCALE, torch.ones(S, S, dtype=torch.bool).tril())
    # rank r owns chunks r and 2*world-1-r of the sequence
    rows = [torch.cat([torch.arange(r * chunk, (r + 1) * chunk),
                       torch.arange((2 * world - 1 - r) * chunk, (2 * world - r) * chunk)]) for r in range(world)]
    shards = [tuple(t[:, idx].contiguous().to(DEV) for t in (q, k, v)) for idx in rows]
    for r in range(world):
        out, lse = _rank_forward(r, world, shards)
        torch.cuda.synchronize()
        assert lse.shape == (1, 2 * chunk, nh, 1)
        assert max_abs(out, ref_o[:, rows[r]]) <= ATOL_O
        assert lse_rel_err(lse.squeeze(-1).transpose(1, 2), ref_lse[:, :, rows[r]]) <= RTOL_LSE
