"""Pins the CPU oracle (oracle/attn_oracle.py) against library routines, closed forms,
invariants and brute force, chosen so that a dropped term, a wrong sign or a transposed
operand fails at least one check.  No GPU."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attn_oracle as ao

torch.manual_seed(0)


def rnd(*shape, dtype=torch.float64, std=1.0):
    return torch.randn(*shape, dtype=dtype) * std


# ---------------------------------------------------------------- tile forward
@pytest.mark.parametrize("causal", [False, True])
def test_tile_fwd_matches_sdpa_and_logsumexp(causal):
    B, S, Nh, D = 2, 24, 3, 16
    q, k, v = rnd(B, S, Nh, D), rnd(B, S, Nh, D), rnd(B, S, Nh, D)
    scale = 0.37
    o, lse = ao.tile_fwd(q, k, v, scale, causal, dtype=torch.float64)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         is_causal=causal, scale=scale).transpose(1, 2)
    assert torch.allclose(o, ref, atol=1e-12)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) * scale
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-12)


def test_tile_fwd_rectangular_sdpa():
    q, k, v = rnd(1, 8, 2, 16), rnd(1, 40, 2, 16), rnd(1, 40, 2, 16)
    o, _ = ao.tile_fwd(q, k, v, 0.25, False, dtype=torch.float64)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), scale=0.25)
    assert torch.allclose(o, ref.transpose(1, 2), atol=1e-12)


def test_tile_fwd_closed_forms():
    B, S, Nh, D = 1, 16, 2, 8
    k, v = rnd(B, S, Nh, D), rnd(B, S, Nh, D)
    # Q = 0: uniform weights -> O = mean of visible V rows, LSE = log(#visible)
    o, lse = ao.tile_fwd(torch.zeros(B, S, Nh, D, dtype=torch.float64), k, v, 1.0, True, dtype=torch.float64)
    for i in range(S):
        assert torch.allclose(o[0, i], v[0, :i + 1].mean(0), atol=1e-12)
        assert torch.allclose(lse[0, :, i], torch.full((Nh,), math.log(i + 1), dtype=torch.float64))
    # constant V -> O = that constant whatever Q, K
    q = rnd(B, S, Nh, D)
    o, _ = ao.tile_fwd(q, k, torch.full_like(v, 2.5), 0.7, False, dtype=torch.float64)
    assert torch.allclose(o, torch.full_like(o, 2.5), atol=1e-12)
    # causal row 0 sees one key: O = V[0], LSE = scale * q0.k0
    o, lse = ao.tile_fwd(q, k, v, 0.7, True, dtype=torch.float64)
    assert torch.allclose(o[0, 0], v[0, 0], atol=1e-12)
    assert torch.allclose(lse[0, :, 0], 0.7 * (q[0, 0] * k[0, 0]).sum(-1), atol=1e-12)


def test_tile_fwd_invariants():
    B, S, Nh, D = 1, 32, 2, 8
    q, k, v = rnd(B, S, Nh, D), rnd(B, S, Nh, D), rnd(B, S, Nh, D)
    o, lse = ao.tile_fwd(q, k, v, 0.5, False, dtype=torch.float64)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) * 0.5
    assert (lse >= s.max(-1).values - 1e-12).all()
    assert (lse <= s.max(-1).values + math.log(S) + 1e-12).all()
    assert (o.amax(1) <= v.amax(1) + 1e-12).all() and (o.amin(1) >= v.amin(1) - 1e-12).all()
    perm = torch.randperm(S)
    o2, lse2 = ao.tile_fwd(q, k[:, perm], v[:, perm], 0.5, False, dtype=torch.float64)
    assert torch.allclose(o, o2, atol=1e-12) and torch.allclose(lse, lse2, atol=1e-12)
    # shifting every key by a vector c shifts the scores of row i by scale*q_i.c -> O unchanged
    c = rnd(D)
    o3, lse3 = ao.tile_fwd(q, k + c, v, 0.5, False, dtype=torch.float64)
    assert torch.allclose(o, o3, atol=1e-10)
    assert torch.allclose(lse3 - lse, 0.5 * torch.einsum("bqhd,d->bhq", q, c), atol=1e-10)


@pytest.mark.parametrize("pattern", ["causal", "random"])
def test_against_python_loop_brute_force(pattern):
    B, Sq, Sk, Nh, D = 1, 12, 16, 2, 4
    q, k, v = rnd(B, Sq, Nh, D), rnd(B, Sk, Nh, D), rnd(B, Sk, Nh, D)
    if pattern == "causal":
        keep = torch.arange(Sk)[None] <= torch.arange(Sq)[:, None] + 4
    else:
        keep = torch.rand(Sq, Sk) < 0.4
        keep[3] = False                      # a row without any key
    o, lse = ao.dense_fwd(q, k, v, 0.6, keep, dtype=torch.float64)
    bo, bl = ao.brute_force_fwd(q, k, v, 0.6, keep)
    assert torch.allclose(o, bo, atol=1e-12)
    assert torch.equal(torch.isinf(lse), torch.isinf(bl))
    fin = torch.isfinite(bl)
    assert torch.allclose(lse[fin], bl[fin], atol=1e-12)
    if pattern == "random":
        assert (o[0, 3] == 0).all() and torch.isinf(lse[0, :, 3]).all()


# ---------------------------------------------------------------- merge
def split_case(S=16, Sk=48, Nh=2, D=8, cuts=(0, 10, 30, 48)):
    q, k, v = rnd(1, S, Nh, D), rnd(1, Sk, Nh, D), rnd(1, Sk, Nh, D)
    full = ao.tile_fwd(q, k, v, 0.4, False, dtype=torch.float64)
    parts = [ao.tile_fwd(q, k[:, a:b], v[:, a:b], 0.4, False, dtype=torch.float64)
             for a, b in zip(cuts[:-1], cuts[1:])]
    return full, parts


def test_merge_recurrence_equals_single_pass_over_union():
    (fo, fl), parts = split_case()
    out, lse = None, None
    for bo, bl in parts:
        out, lse = ao.update_out_and_lse(out, lse, bo, bl)
    assert torch.allclose(out, fo, atol=1e-12)
    assert torch.allclose(lse.squeeze(-1).transpose(-2, -1), fl, atol=1e-12)
    mo, ml = ao.merge_partials([p[0] for p in parts], [p[1] for p in parts], dtype=torch.float64)
    assert torch.allclose(mo, fo, atol=1e-12) and torch.allclose(ml, fl, atol=1e-12)


def test_merge_order_independent_and_logaddexp():
    (_, _), parts = split_case()
    a = ao.merge_partials([p[0] for p in parts], [p[1] for p in parts], dtype=torch.float64)
    b = ao.merge_partials([p[0] for p in parts[::-1]], [p[1] for p in parts[::-1]], dtype=torch.float64)
    assert torch.allclose(a[0], b[0], atol=1e-12) and torch.allclose(a[1], b[1], atol=1e-12)
    two = ao.merge_partials([parts[0][0], parts[1][0]], [parts[0][1], parts[1][1]], dtype=torch.float64)
    assert torch.allclose(two[1], torch.logaddexp(parts[0][1], parts[1][1]), atol=1e-12)


def test_merge_special_cases():
    o1, o2 = rnd(1, 8, 2, 4), rnd(1, 8, 2, 4)
    l = rnd(1, 2, 8)
    o, lse = ao.merge_partials([o1, o2], [l, l], dtype=torch.float64)        # equal LSE -> average
    assert torch.allclose(o, (o1 + o2) / 2, atol=1e-12) and torch.allclose(lse, l + math.log(2), atol=1e-12)
    ninf = torch.full_like(l, float("-inf"))
    o, lse = ao.merge_partials([o1, o2], [l, ninf], dtype=torch.float64)     # -inf partial -> identity
    assert torch.allclose(o, o1) and torch.allclose(lse, l)
    o, lse = ao.merge_partials([o1], [l], dtype=torch.float64)               # P = 1 -> copy
    assert torch.equal(o, o1) and torch.equal(lse, l)
    o, lse = ao.merge_partials([o1, o2], [ninf, ninf], dtype=torch.float64)  # nothing visible at all
    assert (o == 0).all() and torch.isinf(lse).all() and (lse < 0).all()
    # |difference| of 100: the stabilised form neither overflows nor loses the big partial
    o, lse = ao.merge_partials([o1, o2], [l, l + 100], dtype=torch.float32)
    assert torch.isfinite(o).all() and torch.allclose(o.double(), o2, atol=1e-6)
    assert torch.allclose(lse.double(), l + 100, atol=1e-4)
    o, lse = ao.merge_partials([o1, o2], [l, l - 100], dtype=torch.float32)
    assert torch.allclose(o.double(), o1, atol=1e-6)


def test_literal_recurrence_equals_stabilised_form_on_ordinary_inputs():
    o1, o2 = rnd(1, 8, 2, 4), rnd(1, 8, 2, 4)
    l1, l2 = rnd(1, 2, 8, std=3), rnd(1, 2, 8, std=3)
    out, lse = ao.update_out_and_lse(None, None, o1, l1)
    out, lse = ao.update_out_and_lse(out, lse, o2, l2)
    mo, ml = ao.merge_partials([o1, o2], [l1, l2], dtype=torch.float64)
    assert torch.allclose(out, mo, atol=1e-12)
    assert torch.allclose(lse.squeeze(-1).transpose(-2, -1), ml, atol=1e-12)


def test_update_out_and_lse_slice_semantics():
    # second half of the rows gets one more partial (hierarchy_attn_impl.py:80 uses this form)
    (fo, fl), parts = split_case(S=16, Sk=32, cuts=(0, 16, 32))
    out, lse = ao.update_out_and_lse(None, None, parts[0][0].clone(), parts[0][1].clone())
    half = (slice(None), slice(8, None))
    bo, bl = parts[1][0][:, 8:], parts[1][1][:, :, 8:]
    out, lse = ao.update_out_and_lse(out, lse, bo, bl, slice_=half)
    assert torch.allclose(out[:, 8:], fo[:, 8:], atol=1e-12)
    assert torch.allclose(out[:, :8], parts[0][0][:, :8], atol=0)
    with pytest.raises(RuntimeError):
        ao.update_out_and_lse(None, None, bo, bl, slice_=half)


# ---------------------------------------------------------------- block loop
@pytest.mark.parametrize("table", [
    np.array([[2, 0, 0], [1, 2, 0], [1, 0, 2]], np.uint8),
    np.array([[1, 1, 0, 1], [0, 1, 1, 0]], np.uint8),
    np.array([[2, 0], [0, 0]], np.uint8),
])
def test_block_loop_equals_dense_masked(table):
    blk, Nh, D = 8, 2, 8
    nqb, nkb = table.shape
    q, k, v = rnd(1, nqb * blk, Nh, D), rnd(1, nkb * blk, Nh, D), rnd(1, nkb * blk, Nh, D)
    keep = ao.element_mask(table, blk)
    do, dl = ao.dense_fwd(q, k, v, 0.3, keep, dtype=torch.float64)
    bo, bl = ao.block_loop_fwd(q, k, v, table, blk, 0.3, dtype=torch.float64)
    assert torch.allclose(bo, do, atol=1e-12)
    assert torch.equal(torch.isinf(bl), torch.isinf(dl))
    assert torch.allclose(bl[torch.isfinite(dl)], dl[torch.isfinite(dl)], atol=1e-12)


def test_element_mask_brute_force():
    table = np.array([[2, 0, 1], [1, 2, 0]], np.uint8)
    keep = ao.element_mask(table, 4)
    for i in range(8):
        for j in range(12):
            t = table[i // 4, j // 4]
            want = t == 1 or (t == 2 and j % 4 <= i % 4)
            assert bool(keep[i, j]) == want


# ---------------------------------------------------------------- backward
def test_tile_bwd_matches_autograd():
    B, S, Sk, Nh, D = 1, 12, 20, 2, 8
    q, k, v, do = rnd(B, S, Nh, D), rnd(B, Sk, Nh, D), rnd(B, Sk, Nh, D), rnd(B, S, Nh, D)
    keep = torch.ones(S, Sk, dtype=torch.bool)
    o, lse = ao.tile_fwd(q, k, v, 0.45, False, dtype=torch.float64)
    delta = ao.softmax_delta(o, do, dtype=torch.float64)
    dq, dk, dv = ao.tile_bwd(do, q, k, v, lse, delta, 0.45, False, dtype=torch.float64)
    rq, rk, rv = ao.dense_bwd_autograd(q, k, v, do, 0.45, keep)
    for a, r in ((dq, rq), (dk, rk), (dv, rv)):
        assert torch.allclose(a, r, atol=1e-12)


def test_block_loop_bwd_sums_to_dense_gradient():
    table = np.array([[2, 0, 0], [1, 2, 0], [1, 0, 2]], np.uint8)
    blk, Nh, D = 8, 2, 8
    q, k, v, do = (rnd(1, 24, Nh, D) for _ in range(4))
    keep = ao.element_mask(table, blk)
    o, lse = ao.dense_fwd(q, k, v, 0.3, keep, dtype=torch.float64)
    dq, dk, dv = ao.block_loop_bwd(do, q, k, v, o, lse, table, blk, 0.3, dtype=torch.float64)
    rq, rk, rv = ao.dense_bwd_autograd(q, k, v, do, 0.3, keep)
    for a, r in ((dq, rq), (dk, rk), (dv, rv)):
        assert torch.allclose(a, r, atol=1e-12)


def test_dense_autograd_passes_gradcheck_and_finite_differences():
    S, Sk, Nh, D = 5, 7, 1, 3
    q, k, v = (rnd(1, n, Nh, D).requires_grad_(True) for n in (S, Sk, Sk))
    keep = torch.rand(S, Sk) < 0.7
    keep[:, 0] = True
    assert torch.autograd.gradcheck(lambda a, b, c: ao.dense_fwd(a, b, c, 0.8, keep, dtype=torch.float64)[0],
                                    (q, k, v), eps=1e-6, atol=1e-6)
    do = rnd(1, S, Nh, D)
    dq, dk, dv = ao.dense_bwd_autograd(q, k, v, do, 0.8, keep)
    f = lambda a, b, c: (ao.dense_fwd(a, b, c, 0.8, keep, dtype=torch.float64)[0] * do).sum().item()
    for which, g, idx in ((0, dq, (0, 2, 0, 1)), (1, dk, (0, 4, 0, 2)), (2, dv, (0, 6, 0, 0))):
        base = [q.detach().clone(), k.detach().clone(), v.detach().clone()]
        hi, lo = [x.clone() for x in base], [x.clone() for x in base]
        hi[which][idx] += 1e-5
        lo[which][idx] -= 1e-5
        assert abs((f(*hi) - f(*lo)) / 2e-5 - g[idx].item()) < 1e-6


def test_backward_identities():
    B, S, Nh, D = 1, 16, 2, 8
    q, k, v, do = (rnd(B, S, Nh, D) for _ in range(4))
    o, lse = ao.tile_fwd(q, k, v, 0.5, True, dtype=torch.float64)
    delta = ao.softmax_delta(o, do, dtype=torch.float64)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) * 0.5
    s = s.masked_fill(torch.triu(torch.ones(S, S, dtype=torch.bool), 1), float("-inf"))
    p = torch.exp(s - lse[..., None])
    dp = torch.einsum("bqhd,bkhd->bhqk", do, v)
    assert torch.allclose((p * dp).sum(-1), delta, atol=1e-12)        # D = rowsum(P*dP) = rowsum(dO*O)
    ds = p * (dp - delta[..., None])
    assert torch.allclose(ds.sum(-1), torch.zeros_like(delta), atol=1e-12)   # rows of dS sum to 0
    _, _, dv = ao.tile_bwd(do, q, k, v, lse, delta, 0.5, True, dtype=torch.float64)
    assert torch.allclose(dv, torch.einsum("bhqk,bqhd->bkhd", p, do), atol=1e-12)


# ---------------------------------------------------------------- golden twins
@pytest.mark.parametrize("name", ["c1_causal", "c3_strided", "c4_global_local", "c5_streaming"])
def test_block_loop_oracle_reproduces_committed_twins(name, golden_dir):
    import hashlib
    import os
    g = np.load(os.path.join(golden_dir, f"twin_{name}.npz"))
    from tests.golden.make_golden import twin_inputs
    mask, block = g["mask"], int(g["block"])
    q, k, v, do = twin_inputs(mask, block, int(g["seed"]))
    digest = hashlib.sha256(b"".join(t.float().numpy().tobytes() for t in (q, k, v, do))).hexdigest()
    assert digest == str(g["inputs_sha256"]), "seeded inputs differ from those the fixture was made from"
    scale = 1.0 / math.sqrt(128)
    o, lse = ao.block_loop_fwd(q, k, v, mask, block, scale, dtype=torch.float32)
    assert np.abs(o[:, g["qrows"]].numpy() - g["o"]).max() < 2e-5
    fin = np.isfinite(g["lse"])
    assert np.abs(lse.numpy()[fin] - g["lse"][fin]).max() < 2e-5
    dq, dk, dv = ao.block_loop_bwd(do, q, k, v, o, lse, mask, block, scale, dtype=torch.float32)
    assert np.abs(dq[:, g["qrows"]].numpy() - g["dq"]).max() < 1e-4
    assert np.abs(dk[:, g["krows"]].numpy() - g["dk"]).max() < 1e-4
    assert np.abs(dv[:, g["krows"]].numpy() - g["dv"]).max() < 1e-4
