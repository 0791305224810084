"""Device-side tile-list builder (bit-exact) and the flash-attn call-signature shim, on the GPU."""
import numpy as np
import pytest
import torch

from oracle import attn_oracle as ao
from oracle import tilelist_oracle as to
from tests.gpu_util import ATOL_O, RTOL_LSE, SCALE, lse_rel_err, max_abs, seeded_inputs
from ultraattn_amd import masks
from ultraattn_amd.flash_attn_interface import _flash_attn_backward, _flash_attn_forward
from ultraattn_amd.tilelist import build_tile_list, build_tile_list_device

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FIELDS = ("row_ptr", "col_idx", "flag", "col_ptr", "row_idx", "cflag", "q_order", "k_order")


@pytest.mark.parametrize("make,block", [
    (lambda: masks.config_causal(16), 512), (lambda: masks.config_strided(), 512),
    (lambda: masks.config_global_local(), 512), (lambda: masks.config_streaming_shard(), 512),
    (lambda: masks.canonical_block_table(3), 1024), (lambda: np.zeros((2, 3), np.uint8), 256),
    (lambda: np.random.RandomState(3).randint(0, 3, size=(7, 5)).astype(np.uint8), 384),
    (lambda: np.random.RandomState(4).randint(0, 2, size=(33, 17)).astype(np.uint8), 128),
    (lambda: np.tril(np.random.RandomState(5).randint(0, 2, size=(24, 24))).astype(np.uint8), 256),
    (lambda: np.triu(np.random.RandomState(6).randint(0, 3, size=(19, 31))).astype(np.uint8), 512),
    (lambda: masks.canonical_block_table(0), 512), (lambda: masks.canonical_block_table(1), 256),
])
def test_device_builder_bit_exact(make, block):
    m = make()
    host = build_tile_list(m, block)
    oracle = to.build_tile_list(m, block // 128)
    dev = build_tile_list_device(torch.from_numpy(m).to(DEV), block, nnz=host.nnz)
    torch.cuda.synchronize()
    for f in FIELDS:
        got = dev[f].cpu().numpy()
        assert got.dtype == oracle[f].dtype and np.array_equal(got, oracle[f]), f
        assert np.array_equal(got, getattr(host, f)), f


def test_device_builder_reports_invalid_mask_entries():
    """The host builder rejects a mask value other than 0/1/2 (UA_ERR_MASK); the device builder cannot
    return an error without a synchronisation, treats the entry as EMPTY and counts it."""
    m = masks.config_strided(8, 2, 4).copy()
    ok = build_tile_list_device(torch.from_numpy(m).to(DEV), 256, check=True)
    bad = m.copy()
    bad[3, 1] = 7
    with pytest.raises(RuntimeError, match="EMPTY"):
        build_tile_list(bad, 256)
    with pytest.raises(ValueError, match="1 entries"):
        build_tile_list_device(torch.from_numpy(bad).to(DEV), 256, check=True)
    as_empty = bad.copy()
    as_empty[3, 1] = 0
    want = build_tile_list(as_empty, 256)
    got = build_tile_list_device(torch.from_numpy(bad).to(DEV), 256, nnz=want.nnz)
    torch.cuda.synchronize()
    for f in FIELDS:
        assert np.array_equal(got[f].cpu().numpy(), getattr(want, f)), f
    assert ok["row_ptr"].shape[0] == 8 * 2 + 1


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("sq,sk", [(256, 256), (128, 384), (384, 384), (384, 128)])
def test_flash_attn_shim(causal, sq, sk):
    """Same call as fwd_comp_func / bwd_comp_func make (orchestrated_attn_impl.py:326-337,
    578-596), checked against the oracle's dense tile.  The reference only runs causal tiles
    on square diagonal chunks; for Sq != Skv the shim follows flash-attn 2.1+'s bottom-right
    alignment (query i sees key j iff j <= i + Skv - Sq), checked here against the oracle's
    dense formula under that explicit element mask (rows without a visible key: O = 0,
    LSE = -inf)."""
    g = torch.Generator().manual_seed(sq + sk)
    mk = lambda n: torch.randn(1, n, 3, 128, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(sq), mk(sk), mk(sk), mk(sq)
    qd, kd, vd, dod = (t.to(DEV) for t in (q, k, v, do))
    out_buf = torch.empty_like(qd)
    res = _flash_attn_forward(qd, kd, vd, 0.0, SCALE, causal=causal, window_size=(-1, -1), alibi_slopes=None,
                              return_softmax=False, out=out_buf)
    assert len(res) == 8 and res[0].data_ptr() == out_buf.data_ptr()
    O, lse = res[0], res[5]
    keep = torch.ones(sq, sk, dtype=torch.bool)
    if causal:
        keep = torch.arange(sk)[None, :] <= torch.arange(sq)[:, None] + (sk - sq)
    ro, rl = ao.dense_fwd(q, k, v, SCALE, keep)
    if sq == sk or not causal:
        to_, tl_ = ao.tile_fwd(q, k, v, SCALE, causal)          # the square case is the reference's own
        assert torch.equal(to_, ro) and torch.equal(tl_, rl)
    assert lse.shape == (1, 3, sq)
    assert max_abs(O, ro) <= ATOL_O and lse_rel_err(lse, rl) <= RTOL_LSE
    delta = ao.softmax_delta(ro, do).to(DEV)
    # dq/dk/dv given: written in place and returned
    dq, dk, dv = torch.empty_like(qd), torch.empty_like(kd), torch.empty_like(vd)
    ret = _flash_attn_backward(dod, qd, kd, vd, qd, lse, dq, dk, dv, 0.0, SCALE, causal, (-1, -1), None, False,
                               rng_state=None, softmax_d=delta)
    assert ret[0].data_ptr() == dq.data_ptr() and ret[1].data_ptr() == dk.data_ptr() and ret[2].data_ptr() == dv.data_ptr()
    # dq/dk/dv = None (allowed by flash-attn's API): allocated by the shim and returned
    ret2 = _flash_attn_backward(dod, qd, kd, vd, qd, lse, None, None, None, 0.0, SCALE, causal, (-1, -1), None, False,
                                rng_state=None, softmax_d=delta)
    torch.cuda.synchronize()
    rq, rk, rv = ao.dense_bwd_autograd(q, k, v, do, SCALE, keep)
    for got in ((dq, dk, dv), ret2[:3]):
        assert max_abs(got[0], rq) <= ATOL_O and max_abs(got[1], rk) <= ATOL_O and max_abs(got[2], rv) <= ATOL_O


def test_shim_rejects_unsupported_features():
    q = torch.zeros(1, 128, 1, 128, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):
        _flash_attn_forward(q, q, q, 0.1, SCALE, causal=False)
    with pytest.raises(NotImplementedError):
        _flash_attn_forward(q, q, q, 0.0, SCALE, causal=False, window_size=(64, 0))
    with pytest.raises(NotImplementedError):
        _flash_attn_forward(q, q, q, 0.0, SCALE, causal=False, alibi_slopes=torch.ones(1))
