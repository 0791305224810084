"""Dense rectangles through ua_dense_fwd / ua_dense_bwd (the flash-attn shim): shapes that the
library cuts into parts (few tile lines, long walks) against the oracle and against the unsplit
run, and a first call at a new shape captured into a HIP graph."""
import ctypes

import numpy as np
import pytest
import torch

from oracle import attn_oracle as ao
from tests.gpu_util import ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs
from ultraattn_amd import _lib, ops
from ultraattn_amd import flash_attn_interface as fai
from ultraattn_amd.flash_attn_interface import _flash_attn_backward, _flash_attn_forward
from ultraattn_amd.tilelist import build_tile_list

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def inputs(sq, sk, nh, seed, batch=1):
    g = torch.Generator().manual_seed(seed)
    mk = lambda n: torch.randn(batch, n, nh, 128, generator=g).to(torch.bfloat16)
    return mk(sq), mk(sk), mk(sk), mk(sq)


def keep_mask(sq, sk, causal):
    if not causal:
        return torch.ones(sq, sk, dtype=torch.bool)
    return torch.arange(sk)[None, :] <= torch.arange(sq)[:, None] + (sk - sq)


def dense_unsplit(lib, q, k, v, do, causal):
    """The same entry points with no workspace: one workgroup per line."""
    B, Sq, Nh, D = q.shape
    st = torch.cuda.current_stream().cuda_stream
    s3 = _lib.strides3
    o, lse = torch.empty_like(q), torch.empty(B, Nh, Sq, dtype=torch.float32, device=q.device)
    rc = lib.ua_dense_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), B, Nh, Sq, k.shape[1], D,
                          s3(q), s3(k), s3(v), s3(o), SCALE, int(causal), None, 0, st)
    assert rc == 0
    delta = ops.softmax_delta(o, do)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    rc = lib.ua_dense_bwd(do.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                          dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, Nh, Sq, k.shape[1], D,
                          s3(q), s3(k), s3(v), s3(do), s3(dq), s3(dk), s3(dv), SCALE, int(causal), None, 0, st)
    assert rc == 0
    return o, lse, delta, dq, dk, dv


@pytest.mark.parametrize("sq,sk,nh,causal", [
    (256, 1024, 1, False),      # 2 query tiles x 8 key tiles: forward and dQ split over keys
    (1024, 256, 1, False),      # 8 x 2: dK/dV split over queries
    (1024, 1024, 1, True),      # causal: parts of a row's range may be empty
    (512, 1536, 2, True),       # bottom-right aligned diagonal, off = 8 tiles
    (1536, 512, 1, True),       # rows above the first key see nothing
    (640, 2048, 3, False),      # ragged last part
    (128, 128, 1, True),        # a single tile: never splits
])
def test_split_rectangles_match_the_oracle_and_the_unsplit_run(lib, sq, sk, nh, causal):
    q, k, v, do = inputs(sq, sk, nh, seed=sq + sk + nh)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    splits = (lib.ua_dense_workspace_bytes(1, nh, sq, sk, 0) > 0, lib.ua_dense_workspace_bytes(1, nh, sq, sk, 1) > 0)
    if sq * sk > 128 * 128:
        assert any(splits), "the shape is meant to exercise the split path"
    res = _flash_attn_forward(qd, kd, vd, 0.0, SCALE, causal=causal)
    O, lse = res[0], res[5]
    keep = keep_mask(sq, sk, causal)
    ro, rl = ao.dense_fwd(q, k, v, SCALE, keep)
    assert max_abs(O, ro) <= ATOL_O and lse_rel_err(lse, rl) <= RTOL_LSE
    uo, ul, delta, udq, udk, udv = dense_unsplit(lib, qd, kd, vd, dod, causal)
    assert max_abs(O, uo.cpu()) <= 8e-3 and lse_rel_err(lse, ul.cpu()) <= 1e-5
    dq, dk, dv, _ = _flash_attn_backward(dod, qd, kd, vd, None, ul, None, None, None, 0.0, SCALE, causal, softmax_d=delta)
    torch.cuda.synchronize()
    rq, rk, rv = ao.dense_bwd_autograd(q, k, v, do, SCALE, keep)
    for got, unsplit, want in ((dq, udq, rq), (dk, udk, rk), (dv, udv, rv)):
        assert max_abs(got, want) <= ATOL_O and max_abs(unsplit, want) <= ATOL_O
        # fp32 partials summed once: at least as close to the unsplit bf16 result as one bf16 rounding
        assert max_abs(got, unsplit.cpu()) <= ATOL_O / 2


@pytest.mark.parametrize("causal", [False, True])
def test_split_with_batch_and_strided_views(lib, causal):
    """Batch > 1 and q / k / v / gradients as strided views of packed buffers (token stride 2 * Nh * 128):
    the partials are laid out [part][batch, tokens, heads, 128] whatever the callers' strides."""
    B, sq, sk, nh = 2, 256, 1280, 2
    g = torch.Generator().manual_seed(17)
    pack = lambda n: torch.randn(B, n, 2 * nh, 128, generator=g).to(torch.bfloat16)
    qp, kp, vp, dop = pack(sq), pack(sk), pack(sk), pack(sq)
    q, k, v, do = qp[:, :, 0::2], kp[:, :, 1::2], vp[:, :, 0::2], dop[:, :, 1::2]
    assert lib.ua_dense_workspace_bytes(B, nh, sq, sk, 0) > 0 and lib.ua_dense_workspace_bytes(B, nh, sq, sk, 1) > 0
    dev = lambda t: t.to(DEV)
    qd, kd, vd, dod = dev(qp)[:, :, 0::2], dev(kp)[:, :, 1::2], dev(vp)[:, :, 0::2], dev(dop)[:, :, 1::2]
    res = _flash_attn_forward(qd, kd, vd, 0.0, SCALE, causal=causal)
    O, lse = res[0], res[5]
    gbuf = torch.zeros(B, sk, 2 * nh, 128, dtype=torch.bfloat16, device=DEV)
    dk, dv = gbuf[:, :, 0::2], gbuf[:, :, 1::2]                    # [dK | dV] interleaved by head: strided outputs
    dq = torch.empty_like(O)
    _flash_attn_backward(dod, qd, kd, vd, O, lse, dq, dk, dv, 0.0, SCALE, causal)
    torch.cuda.synchronize()
    keep = keep_mask(sq, sk, causal)
    for b in range(B):
        sl = lambda t: t[b:b + 1].contiguous()
        ro, rl = ao.dense_fwd(sl(q), sl(k), sl(v), SCALE, keep)
        rq, rk, rv = ao.dense_bwd_autograd(sl(q), sl(k), sl(v), sl(do), SCALE, keep)
        assert max_abs(O[b:b + 1], ro) <= ATOL_O and lse_rel_err(lse[b:b + 1], rl) <= RTOL_LSE
        assert max_abs(dq[b:b + 1], rq) <= ATOL_O and max_abs(dk[b:b + 1], rk) <= ATOL_O and max_abs(dv[b:b + 1], rv) <= ATOL_O


@pytest.mark.parametrize("sq,sk,nh,causal", [(8192, 8192, 1, True), (4096, 16384, 1, False), (16384, 2048, 2, False)])
def test_large_split_rectangles_equal_the_unsplit_run(lib, sq, sk, nh, causal):
    """The reference planner's low-parallelism keys at their real sizes (one or two heads, thousands of
    tokens: up to 16 parts per walk): split and unsplit runs of the same entry points agree to the
    rounding of one bf16 result, and sampled rows agree with the oracle."""
    g = torch.Generator(device=DEV).manual_seed(sq + sk)
    mk = lambda n: torch.randn(1, n, nh, 128, device=DEV, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(sq), mk(sk), mk(sk), mk(sq)
    assert lib.ua_dense_workspace_bytes(1, nh, sq, sk, 0) > 0 or lib.ua_dense_workspace_bytes(1, nh, sq, sk, 1) > 0
    uo, ul, delta, udq, udk, udv = dense_unsplit(lib, q, k, v, do, causal)
    res = _flash_attn_forward(q, k, v, 0.0, SCALE, causal=causal)
    dq, dk, dv, _ = _flash_attn_backward(do, q, k, v, None, ul, None, None, None, 0.0, SCALE, causal, softmax_d=delta)
    torch.cuda.synchronize()
    assert max_abs(res[0], uo.cpu()) <= 8e-3 and lse_rel_err(res[5], ul.cpu()) <= 1e-5
    for got, unsplit in ((dq, udq), (dk, udk), (dv, udv)):
        assert max_abs(got, unsplit.cpu()) <= ATOL_O / 2
    # sampled query rows against the dense formula (fp32 on the device, one head)
    rows = torch.tensor([0, 1, 127, 128, sq // 2 + 5, sq - 129, sq - 1])
    qs = q[0, rows, 0].float()
    sc = (qs @ k[0, :, 0].float().T) * SCALE
    if causal:
        sc = sc.masked_fill(torch.arange(sk, device=DEV)[None, :] > rows.to(DEV)[:, None] + (sk - sq), float("-inf"))
    want_lse = torch.logsumexp(sc, -1)
    want_o = torch.softmax(sc, -1) @ v[0, :, 0].float()
    assert (res[0][0, rows, 0].float() - want_o).abs().max().item() <= ATOL_O
    assert ((res[5][0, 0, rows] - want_lse).abs() / want_lse.abs().clamp_min(1)).max().item() <= RTOL_LSE


def test_dense_equals_the_tile_list_of_the_same_rectangle(lib):
    """List-free enumeration = the tile list that the block-mask builder gives for the same rectangle
    (bit for bit when nothing is split: same tiles in the same order)."""
    sq, sk, nh = 512, 768, 16                       # 64 workgroups... unsplit only without a workspace
    q, k, v, do = (t.to(DEV) for t in inputs(sq, sk, nh, seed=3))
    for causal in (False, True):
        m = np.ones((sq // 128, sk // 128), np.uint8)
        if causal:
            i, j = np.arange(sq // 128)[:, None] + (sk - sq) // 128, np.arange(sk // 128)[None, :]
            m = np.where(j < i, 1, np.where(j == i, 2, 0)).astype(np.uint8)
        tl = build_tile_list(m, block=128)
        o1, l1 = ops.bsa_fwd(q, k, v, tl, SCALE)
        delta = ops.softmax_delta(o1, do)
        g1 = ops.bsa_bwd(do, q, k, v, None, l1, tl, SCALE, softmax_d=delta)
        o2, l2, _, dq, dk, dv = dense_unsplit(lib, q, k, v, do, causal)
        torch.cuda.synchronize()
        assert torch.equal(o1, o2) and torch.equal(l1, l2)
        assert torch.equal(g1[0], dq) and torch.equal(g1[1], dk) and torch.equal(g1[2], dv)


def test_first_call_at_a_new_shape_can_be_captured(lib):
    """Nothing in the shim builds, copies or caches a tile list, and nothing synchronises: a first
    call at a shape never seen before (workspace growth included) is captured into a HIP graph, and
    every replay on new inputs equals the eager result."""
    assert lib.ua_init() == 0
    sq, sk, nh = 384, 1152, 2                       # not used by any other test: forward and backward both split
    assert lib.ua_dense_workspace_bytes(1, nh, sq, sk, 0) > 0 and lib.ua_dense_workspace_bytes(1, nh, sq, sk, 1) > 0
    q, k, v, do = (t.to(DEV) for t in inputs(sq, sk, nh, seed=1))
    o = torch.empty_like(q)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    fai._workspaces.clear()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        lse = _flash_attn_forward(q, k, v, 0.0, SCALE, causal=True, out=o)[5]
        delta = _flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, 0.0, SCALE, True)[3]
    for seed in (2, 3, 4):
        nq, nk, nv, ndo = (t.to(DEV) for t in inputs(sq, sk, nh, seed=seed))
        q.copy_(nq); k.copy_(nk); v.copy_(nv); do.copy_(ndo)
        for t in (o, dq, dk, dv):
            t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (o, lse, delta, dq, dk, dv)]
        # eager work and synchronisations between the replays
        eo = _flash_attn_forward(nq, nk, nv, 0.0, SCALE, causal=True)
        eg = _flash_attn_backward(ndo, nq, nk, nv, eo[0], eo[5], None, None, None, 0.0, SCALE, True)
        torch.cuda.synchronize()
        want = [eo[0], eo[5], eg[3], eg[0], eg[1], eg[2]]
        for a, b in zip(got, want):
            assert torch.equal(a, b)


def test_dense_argument_checks(lib):
    s = (ctypes.c_int64 * 3)(128 * 128, 128, 128)
    x = torch.zeros(1, 128, 1, 128, dtype=torch.bfloat16, device=DEV)
    l = torch.zeros(1, 1, 128, dtype=torch.float32, device=DEV)
    p, lp = x.data_ptr(), l.data_ptr()
    assert lib.ua_dense_fwd(p, p, p, p, lp, 1, 1, 100, 128, 128, s, s, s, s, SCALE, 0, None, 0, None) == -2
    assert lib.ua_dense_fwd(p, p, p, p, lp, 1, 1, 128, 128, 64, s, s, s, s, SCALE, 0, None, 0, None) == -3
    assert lib.ua_dense_fwd(None, p, p, p, lp, 1, 1, 128, 128, 128, s, s, s, s, SCALE, 0, None, 0, None) == -1
    assert lib.ua_dense_bwd(p, p, p, p, lp, lp, None, p, p, 1, 1, 128, 128, 128, s, s, s, s, s, s, s, SCALE, 0, None, 0, None) == -1
    assert lib.ua_dense_workspace_bytes(1, 32, 131072, 131072, 0) == 0          # fills the device: never splits
    assert lib.ua_dense_workspace_bytes(1, 1, 1024, 4096, 0) > 0
    assert lib.ua_dense_workspace_bytes(1, 1, 1000, 4096, 0) == 0               # not a multiple of 128: nothing to size
