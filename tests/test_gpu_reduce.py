"""Gradient reductions on the GPU, through the C ABI: the running fp32 accumulation of the packs'
reduce() and the one-pass sum of partials, bit for bit against the oracle's restatement of
ring_flash_attn/ring_flash_attn.py:110-118."""
import math

import pytest
import torch

from oracle import attn_oracle as ao
from ultraattn_amd import ops, packed
from ultraattn_amd.executor import BlockSparseExecutor

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def partials(n, count, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(n, generator=g).to(torch.bfloat16) for _ in range(count)]


@pytest.mark.parametrize("cls", [packed.OutputRowBwd, packed.OutputColBwd])
def test_pack_reduce_chain_is_the_fp32_sum_rounded_once(cls):
    shape = (1, 128, 2, 128)
    n = math.prod(shape) * (2 if cls is packed.OutputColBwd else 1)
    parts = partials(n, 8, seed=5)
    want_acc, want = ao.accumulate_gradients(parts)
    packs = [cls(p.clone().to(DEV), shape) for p in parts]
    packs[0].begin_reduce()
    for other in packs[1:]:
        packs[0].reduce(other)
        assert packs[0]._acc is not None
    assert torch.equal(packs[0]._acc.cpu(), want_acc)
    packs[0].end_reduce()
    assert torch.equal(packs[0].data.cpu(), want) and packs[0]._acc is None
    # caller-supplied accumulator (larger than needed): same bits, sum left in the caller's buffer
    again = cls(parts[0].clone().to(DEV), shape)
    mine = torch.full((n + 64,), 7.0, dtype=torch.float32, device=DEV)
    again.begin_reduce(mine)
    for other in packs[1:]:
        again.reduce(other)
    again.end_reduce()
    assert torch.equal(again.data.cpu(), want) and torch.equal(mine[:n].cpu(), want_acc) and (mine[n:] == 7.0).all()


def test_pack_refilled_between_chains_starts_from_the_new_data():
    """A pack is a view of a persistent buffer that kernels and receives rewrite in place
    (orchestrated_attn_impl.py:49-56 keeps the objects alive): a second reduction after the pack
    has been refilled must not see the first one's sum."""
    shape = (1, 64, 2, 128)
    n = math.prod(shape)
    a, b, c, d = partials(n, 4, seed=9)
    pack = packed.OutputRowBwd(a.clone().to(DEV), shape)
    pack.begin_reduce()
    pack.reduce(packed.OutputRowBwd(b.to(DEV), shape))
    pack.end_reduce()
    assert torch.equal(pack.data.cpu(), ao.accumulate_gradients([a, b])[1])
    pack.dQ.copy_(c.view(shape))                               # the kernel writes fresh gradients
    pack.begin_reduce()
    pack.reduce(packed.OutputRowBwd(d.to(DEV), shape))
    pack.end_reduce()
    assert torch.equal(pack.data.cpu(), ao.accumulate_gradients([c, d])[1])
    # outside a chain reduce() keeps no state at all
    pack.dQ.copy_(a.view(shape))
    pack.reduce(packed.OutputRowBwd(b.to(DEV), shape))
    assert pack._acc is None
    pack.dQ.copy_(c.view(shape))
    pack.reduce(packed.OutputRowBwd(d.to(DEV), shape))
    assert torch.equal(pack.data.cpu(), (c.float() + d.float()).to(torch.bfloat16))


@pytest.mark.parametrize("count", [1, 2, 8, 16])
@pytest.mark.parametrize("fp32", [False, True])
def test_grad_sum_is_the_fp32_sum_of_the_partials(count, fp32):
    shape = (2, 24, 3, 128)
    n = math.prod(shape)
    parts = partials(n, count, seed=count)
    if fp32:
        g = torch.Generator().manual_seed(100 + count)
        parts = [torch.randn(n, generator=g) for _ in range(count)]
    acc = parts[0].float()
    for p in parts[1:]:
        acc = acc + p.float()
    dev_parts = [p.view(shape).to(DEV) for p in parts]
    got = ops.grad_sum(dev_parts)
    assert torch.equal(got.cpu().view(-1), acc.to(torch.bfloat16))
    if not fp32:
        assert torch.equal(BlockSparseExecutor.reduce_bwd(dev_parts).cpu().view(-1), ao.accumulate_gradients(parts)[1])
    # strided output view and a scale (the split backward writes dq = scale * sum of fp32 partials this way)
    big = torch.zeros(shape[0], shape[1], 2 * shape[2], 128, dtype=torch.bfloat16, device=DEV)
    view = big[:, :, 1::2]
    ops.grad_sum(dev_parts, out=view, scale=0.5)
    assert torch.equal(view.cpu().reshape(-1), (acc * 0.5).to(torch.bfloat16))
    assert (big[:, :, 0::2] == 0).all()


def test_grad_accumulate_argument_checks():
    x = torch.zeros(64, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops.grad_accumulate(x, x[:32])
    with pytest.raises(ValueError):
        ops.grad_accumulate(x, x.float())
    with pytest.raises(RuntimeError):
        ops.grad_accumulate(x[:12], x[16:28])          # not a multiple of 8 elements
