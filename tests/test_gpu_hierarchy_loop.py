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


def test_ring_forward_and_backward_equal_causal_attention():
    """The plain ring (``ring_flash_attn/ring_flash_attn.py:16-135``): rank r owns chunk r; forward
    steps 0..r fold one dense call each; the backward calls ``_flash_attn_backward`` once per step with
    the rank's FINAL out and softmax_lse, sums dq in fp32 at the query owner and lets dk/dv travel with
    their k/v chunk (here: summed per chunk in fp32, bf16 blocks as the reference's buffers)."""
    from ultraattn_amd.flash_attn_interface import _flash_attn_backward
    world, chunk, nh = 4, 256, 2
    g = torch.Generator().manual_seed(9)
    S = world * chunk
    q, k, v, do = (torch.randn(1, S, nh, 128, generator=g).to(torch.bfloat16) for _ in range(4))
    keep = torch.ones(S, S, dtype=torch.bool).tril()
    ref_o, ref_lse = ao.dense_fwd(q, k, v, SCALE, keep)
    ref_dq, ref_dk, ref_dv = ao.dense_bwd_autograd(q, k, v, do, SCALE, keep)
    cut = lambda t, r: t[:, r * chunk:(r + 1) * chunk].contiguous().to(DEV)
    Q, K, V, DO = ([cut(t, r) for r in range(world)] for t in (q, k, v, do))
    dK = [torch.zeros(1, chunk, nh, 128, dtype=torch.float32, device=DEV) for _ in range(world)]
    dV = [torch.zeros_like(t) for t in dK]
    for r in range(world):
        out = lse = None
        for step in range(r + 1):                      # forward: k/v of rank r - step
            j = r - step
            block_out, _, _, _, _, block_lse, _, _ = _flash_attn_forward(Q[r], K[j], V[j], 0.0, SCALE, causal=step == 0)
            out, lse = update_out_and_lse(out, lse, block_out, block_lse)
        out_bf16 = out.to(torch.bfloat16)
        softmax_lse = lse.squeeze(dim=-1).transpose(1, 2).contiguous()          # [B, Nh, S], as the reference restores it
        assert max_abs(out, ref_o[:, r * chunk:(r + 1) * chunk]) <= ATOL_O
        assert lse_rel_err(softmax_lse, ref_lse[:, :, r * chunk:(r + 1) * chunk]) <= RTOL_LSE
        dq = None
        bdq, bdk, bdv = (torch.empty_like(Q[r]) for _ in range(3))
        for step in range(r + 1):                      # backward: global out / lse for every block
            j = r - step
            _flash_attn_backward(DO[r], Q[r], K[j], V[j], out_bf16, softmax_lse, bdq, bdk, bdv, 0.0, SCALE,
                                 step == 0, (-1, -1), None, False, rng_state=None)
            dq = bdq.to(torch.float32) if dq is None else dq + bdq
            dK[j] += bdk
            dV[j] += bdv
        torch.cuda.synchronize()
        assert max_abs(dq, ref_dq[:, r * chunk:(r + 1) * chunk]) <= ATOL_O
    for j in range(world):
        assert max_abs(dK[j], ref_dk[:, j * chunk:(j + 1) * chunk]) <= ATOL_O
        assert max_abs(dV[j], ref_dv[:, j * chunk:(j + 1) * chunk]) <= ATOL_O
