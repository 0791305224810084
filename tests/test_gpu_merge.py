"""Merge kernel parity on the GPU, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as ao
from tests.gpu_util import ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs, seeded_inputs
from ultraattn_amd import masks, ops
from ultraattn_amd.tilelist import build_tile_list

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def parts(P, B, S, Nh, seed, lse_std=3.0):
    g = torch.Generator().manual_seed(seed)
    outs = [torch.randn(B, S, Nh, 128, generator=g).to(torch.bfloat16) for _ in range(P)]
    lses = [torch.randn(B, Nh, S, generator=g) * lse_std for _ in range(P)]
    return outs, lses


@pytest.mark.parametrize("P", [1, 2, 3, 4, 7, 16])
@pytest.mark.parametrize("shape", [(1, 512, 4), (2, 48, 3), (1, 16, 32), (2, 37, 5), (1, 3, 2)])
def test_merge_vs_oracle(P, shape):
    B, S, Nh = shape
    outs, lses = parts(P, B, S, Nh, seed=P)
    o, l = ops.merge_partials([t.to(DEV) for t in outs], [t.to(DEV) for t in lses])
    ro, rl = ao.merge_partials(outs, lses)
    assert max_abs(o, ro) <= ATOL_O
    assert lse_rel_err(l, rl) <= RTOL_LSE


def test_merge_edge_values():
    outs, lses = parts(3, 1, 64, 2, seed=9)
    lses[1][0, 0, :5] = float("-inf")                    # partial without keys: identity
    lses[0][0, 1, 7] = lses[1][0, 1, 7] = lses[2][0, 1, 7] = float("-inf")    # row without keys at all
    lses[2][0, 0, 20:30] += 100.0                         # dominating partial
    lses[0][0, 1, 40:50] -= 100.0                         # vanishing partial
    o, l = ops.merge_partials([t.to(DEV) for t in outs], [t.to(DEV) for t in lses])
    ro, rl = ao.merge_partials(outs, lses)
    assert torch.isfinite(o).all()
    assert max_abs(o, ro) <= ATOL_O and lse_rel_err(l, rl) <= RTOL_LSE
    assert (o[0, 7, 1] == 0).all()
    assert torch.equal(o[0, 20:30, 0].cpu(), outs[2][0, 20:30, 0])


def test_merge_single_partial_is_a_copy_and_in_place_alias():
    outs, lses = parts(2, 1, 32, 4, seed=2)
    o, l = ops.merge_partials([outs[0].to(DEV)], [lses[0].to(DEV)])
    assert torch.equal(o.cpu(), outs[0]) and torch.allclose(l.cpu(), lses[0], atol=1e-6)
    d_outs, d_lses = [t.to(DEV) for t in outs], [t.to(DEV) for t in lses]
    ro, rl = ao.merge_partials(outs, lses)
    o, l = ops.merge_partials(d_outs, d_lses, out=d_outs[0], lse=d_lses[0])      # accumulate into partial 0
    assert o.data_ptr() == d_outs[0].data_ptr()
    assert max_abs(o, ro) <= ATOL_O and lse_rel_err(l, rl) <= RTOL_LSE


def test_merge_argument_errors():
    outs, lses = parts(2, 1, 32, 2, seed=1)
    d_outs, d_lses = [t.to(DEV) for t in outs], [t.to(DEV) for t in lses]
    with pytest.raises(ValueError):
        ops.merge_partials(d_outs, d_lses[:1])
    with pytest.raises(ValueError):
        ops.merge_partials([], [])
    with pytest.raises(ValueError):
        ops.merge_partials(d_outs, [d_lses[0], d_lses[1].transpose(1, 2)])
    with pytest.raises(RuntimeError, match="unsupported"):
        ops.merge_partials(d_outs * 9, d_lses * 9)                 # 18 partials
    with pytest.raises(TypeError):
        ops.merge_partials([t.float() for t in d_outs], d_lses)


@pytest.mark.parametrize("cfg", ["twin", "c5_full"])
def test_kernel_tiles_plus_merge_equal_single_launch(cfg):
    """The streaming shard computed as 4 key-range kernel tiles + merge equals one launch over
    the whole tile list (merge of partials over disjoint key sets = single pass over the union)."""
    if cfg == "twin":
        mask, block, nh = masks.config_streaming_shard(4, 16, 3), 128, 2
    else:
        mask, block, nh = masks.config_streaming_shard(), 512, 32
    g = torch.Generator(device=DEV).manual_seed(0)
    mk = lambda n: torch.randn(1, n * block, nh, 128, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v = mk(mask.shape[0]), mk(mask.shape[1]), mk(mask.shape[1])
    whole_o, whole_lse = ops.bsa_fwd(q, k, v, build_tile_list(mask, block), SCALE)
    cols = np.nonzero(mask.any(0))[0]
    cuts = np.array_split(cols, 4)
    p_o, p_l = [], []
    for c in cuts:
        sub = np.zeros_like(mask)
        sub[:, c] = mask[:, c]
        o, l = ops.bsa_fwd(q, k, v, build_tile_list(sub, block), SCALE)
        p_o.append(o)
        p_l.append(l)
    o, l = ops.merge_partials(p_o, p_l)
    torch.cuda.synchronize()
    assert (o.float() - whole_o.float()).abs().max().item() <= ATOL_O
    assert lse_rel_err(l, whole_lse) <= RTOL_LSE
