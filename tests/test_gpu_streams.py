"""The entry points take the stream they are given, keep no global state and never synchronise:
two host-side sequences on two streams give the results of the same calls run one after the
other, and a HIP graph captured from the calls replays to the eager results."""
import numpy as np
import pytest
import torch

from tests.gpu_util import SCALE
from ultraattn_amd import masks, ops
from ultraattn_amd.tilelist import build_tile_list

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _inputs(mask, block, nh, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    mk = lambda n: torch.randn(1, n * block, nh, 128, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    return mk(mask.shape[0]), mk(mask.shape[1]), mk(mask.shape[1]), mk(mask.shape[0])


def _step(tl, q, k, v, do, bufs):
    o, lse, delta, dq, dk, dv = bufs
    ops.bsa_fwd(q, k, v, tl, SCALE, out=o, lse=lse)
    ops.softmax_delta(o, do, delta=delta)
    ops.bsa_bwd(do, q, k, v, None, lse, tl, SCALE, softmax_d=delta, dq=dq, dk=dk, dv=dv)


def _buffers(q, k):
    B, S, Nh, _ = q.shape
    stat = lambda: torch.empty(B, Nh, S, dtype=torch.float32, device=DEV)
    return (torch.empty_like(q), stat(), stat(), torch.empty_like(q), torch.empty_like(k), torch.empty_like(k))


def test_two_streams_equal_serial_execution():
    cases = [(masks.config_strided(16, 2, 4), 512, 4, 1), (masks.config_global_local(12, 1, 2), 512, 4, 2)]
    tls = [build_tile_list(m, b) for m, b, _, _ in cases]
    ins = [_inputs(m, b, nh, seed) for m, b, nh, seed in cases]
    for tl in tls:
        tl.on(DEV)                                    # device copies of the lists made up front
    serial = [_buffers(i[0], i[1]) for i in ins]
    for tl, i, bufs in zip(tls, ins, serial):
        _step(tl, *i, bufs)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(device=DEV) for _ in cases]
    overlapped = [_buffers(i[0], i[1]) for i in ins]
    for _ in range(3):                                # interleave the launches of the two sequences
        for st, tl, i, bufs in zip(streams, tls, ins, overlapped):
            with torch.cuda.stream(st):
                _step(tl, *i, bufs)
    torch.cuda.synchronize()
    for a, b in zip(serial, overlapped):
        for x, y in zip(a, b):
            assert torch.equal(x, y)


def test_forward_backward_replay_from_a_hip_graph():
    mask, block, nh = masks.config_strided(8, 2, 4), 512, 4
    tl = build_tile_list(mask, block)
    tl.on(DEV)
    q, k, v, do = _inputs(mask, block, nh, 5)
    eager = _buffers(q, k)
    _step(tl, q, k, v, do, eager)
    torch.cuda.synchronize()
    graphed = _buffers(q, k)
    side = torch.cuda.Stream(device=DEV)
    with torch.cuda.stream(side):                     # warm-up on the capture stream, as torch asks
        _step(tl, q, k, v, do, graphed)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        _step(tl, q, k, v, do, graphed)
    for rep in range(3):
        for t in graphed:
            t.fill_(float("nan")) if t.dtype != torch.float32 else t.fill_(-1.0)
        q2 = q.clone()                                # eager work and a synchronisation between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for x, y in zip(eager, graphed):
            assert torch.equal(x, y), rep
        del q2
