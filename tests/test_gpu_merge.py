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


# ---- update_out_and_lse drop-in (ring_flash_attn/utils.py:78-99) ---------------------------------

def _ring_inputs(B, S, Nh, seed, n_blocks=3):
    g = torch.Generator().manual_seed(seed)
    outs = [torch.randn(B, S, Nh, 128, generator=g).to(torch.bfloat16) for _ in range(n_blocks)]
    lses = [torch.randn(B, Nh, S, generator=g) * 3.0 for _ in range(n_blocks)]
    return outs, lses


@pytest.mark.parametrize("shape", [(1, 256, 4), (2, 48, 3), (1, 37, 5)])
def test_update_out_and_lse_chain_vs_oracle(shape):
    """The executors' accumulation loop (hierarchy_attn_impl.py:64-81): first partial initialises,
    the second is folded into all rows, the third into the second half of the rows only
    (slice_).  Same calls on the oracle (CPU, the reference's literal formula) and on the GPU."""
    B, S, Nh = shape
    outs, lses = _ring_inputs(B, S, Nh, seed=S)
    half = S // 2
    sl = (slice(None), slice(half, None))
    ro, rl = None, None
    ro, rl = ao.update_out_and_lse(ro, rl, outs[0], lses[0])
    ro, rl = ao.update_out_and_lse(ro, rl, outs[1], lses[1])
    ro, rl = ao.update_out_and_lse(ro, rl, outs[2][:, half:], lses[2][:, :, half:].contiguous(), slice_=sl)
    d = lambda t: t.to(DEV)
    o, l = None, None
    o, l = ops.update_out_and_lse(o, l, d(outs[0]), d(lses[0]))
    assert o.dtype == torch.bfloat16 and l.shape == (B, S, Nh, 1)             # as the reference: block_out itself
    o, l = ops.update_out_and_lse(o, l, d(outs[1]), d(lses[1]))
    assert o.dtype == ro.dtype == torch.float32 and l.shape == rl.shape == (B, S, Nh, 1)
    before = o[:, :half].clone()
    o2, l2 = ops.update_out_and_lse(o, l, d(outs[2][:, half:].contiguous()), d(lses[2][:, :, half:].contiguous()), slice_=sl)
    torch.cuda.synchronize()
    assert o2.data_ptr() == o.data_ptr() and l2.data_ptr() == l.data_ptr()     # slice_ updates in place
    assert torch.equal(o[:, :half], before)                                    # rows outside the slice untouched
    # fp32 rows and statistics on both sides: only the exp2/log2 hardware approximations differ
    assert max_abs(o2, ro) <= 3e-5 and (l2.cpu() - rl).abs().max().item() <= 1e-5


def test_update_out_and_lse_bf16_in_place_and_statistics_layouts():
    """slice_ on a bf16 running output stays bf16 (assignment casts, utils.py:95), block_lse may
    come as [B,S,Nh,1] (hierarchy_attn_impl.py:52) and -inf partials are the identity."""
    B, S, Nh = 1, 64, 4
    outs, lses = _ring_inputs(B, S, Nh, seed=3, n_blocks=2)
    lses[1][0, 1, 5:9] = float("-inf")                    # block without keys on some rows
    lses[0][0, 2, 20:24] = float("-inf")                  # running rows that have seen no key yet
    lses[0][0, 3, 40] = lses[1][0, 3, 40] = float("-inf")  # neither has
    run_o = outs[0].to(DEV)
    run_l = lses[0].transpose(-2, -1).unsqueeze(-1).contiguous().to(DEV)          # [B,S,Nh,1]
    blk_l = lses[1].transpose(-2, -1).unsqueeze(-1).contiguous().to(DEV)          # [B,S,Nh,1] as well
    o, l = ops.update_out_and_lse(run_o, run_l, outs[1].to(DEV), blk_l, slice_=(slice(None), slice(None)))
    torch.cuda.synchronize()
    assert o.dtype == torch.bfloat16 and o.data_ptr() == run_o.data_ptr()
    ro, rl = ao.merge_partials(outs, lses)
    assert torch.isfinite(o).all()
    assert max_abs(o, ro) <= ATOL_O and lse_rel_err(l.squeeze(-1).transpose(1, 2), rl) <= RTOL_LSE
    assert (o[0, 40, 3] == 0).all() and torch.equal(o[0, 5:9, 1].cpu(), outs[0][0, 5:9, 1])
    assert torch.equal(o[0, 20:24, 2].cpu(), outs[1][0, 20:24, 2])
    with pytest.raises(RuntimeError):
        ops.update_out_and_lse(None, None, outs[0].to(DEV), lses[0].to(DEV), slice_=(slice(None),))
    with pytest.raises(ValueError):
        ops.update_out_and_lse(run_o, run_l, outs[1][:, :32].to(DEV), blk_l)


@pytest.mark.parametrize("run_dtype,blk_dtype", [(torch.float32, torch.bfloat16), (torch.bfloat16, torch.float32),
                                                 (torch.float32, torch.float32)])
def test_update_out_and_lse_views_dtypes_and_layouts(run_dtype, blk_dtype):
    """Strided targets (a head range and a row range of a larger running tensor, batch 2), rows in
    bf16 or fp32 on either side, and the running statistics kept in the kernels' [B,Nh,S] layout:
    one ua_merge_update call each, against the stabilised oracle."""
    B, S, Nh = 2, 53, 6
    g = torch.Generator().manual_seed(17)
    run_o = torch.randn(B, S, Nh, 128, generator=g).to(run_dtype)
    blk_o = torch.randn(B, 20, 4, 128, generator=g).to(blk_dtype)
    run_l = torch.randn(B, Nh, S, generator=g) * 2.0
    blk_l = torch.randn(B, 4, 20, generator=g) * 2.0
    sl_rows, sl_heads = slice(30, 50), slice(1, 5)
    ro, rl = ao.merge_partials([run_o[:, sl_rows, sl_heads], blk_o], [run_l[:, sl_heads, sl_rows], blk_l])
    d_o, d_l = run_o.to(DEV), run_l.to(DEV)
    keep_o, keep_l = d_o.clone(), d_l.clone()
    tgt_o = d_o[:, sl_rows, sl_heads]                      # strided view: written in place through slice_
    tgt_l = d_l[:, sl_heads, sl_rows]
    o, l = ops.update_out_and_lse(tgt_o, tgt_l, blk_o.to(DEV), blk_l.to(DEV), slice_=(slice(None),))
    torch.cuda.synchronize()
    tol = ATOL_O if run_dtype == torch.bfloat16 else (1e-2 if blk_dtype == torch.bfloat16 else 3e-5)
    assert max_abs(d_o[:, sl_rows, sl_heads], ro.to(run_dtype).float()) <= tol
    assert lse_rel_err(d_l[:, sl_heads, sl_rows], rl) <= 1e-5
    # everything outside the target is untouched
    mask_o = torch.ones_like(d_o, dtype=torch.bool); mask_o[:, sl_rows, sl_heads] = False
    mask_l = torch.ones_like(d_l, dtype=torch.bool); mask_l[:, sl_heads, sl_rows] = False
    assert torch.equal(d_o[mask_o], keep_o[mask_o]) and torch.equal(d_l[mask_l], keep_l[mask_l])
