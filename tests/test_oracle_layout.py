"""Pins oracle/layout_oracle.py: explicit index loops, the reference's torch expression, round trip."""
import numpy as np
import pytest
import torch

from oracle import layout_oracle as lo

SHAPES = [(2, (1, 4, 2, 8)), (3, (2, 5, 3, 8)), (1, (1, 3, 1, 8)), (5, (1, 2, 2, 16))]


@pytest.mark.parametrize("Y,ks", SHAPES)
def test_gather_matches_index_loop_and_reference_expression(Y, ks):
    B, S, Nh, D = ks
    n = 2 * Y * B * S * Nh * D
    buf = np.arange(n, dtype=np.int32)
    got = lo.cols_gather(buf, Y, ks)
    assert got.shape == (2, B, Y * S, Nh, D)
    src = buf.reshape(Y, 2, B, S, Nh, D)
    for c in range(2):
        for b in range(B):
            for y in range(Y):
                for s in range(S):
                    assert np.array_equal(got[c, b, y * S + s], src[y, c, b, s])
    # the expression at orchestrated_attn_impl.py:269
    t = torch.from_numpy(buf).view([Y, 2] + list(ks)).transpose(0, 1).transpose(1, 2).flatten(2, 3).contiguous()
    assert np.array_equal(got, t.numpy())


@pytest.mark.parametrize("Y,ks", SHAPES)
def test_scatter_matches_index_loop_and_inverts_gather(Y, ks):
    B, S, Nh, D = ks
    n = 2 * Y * B * S * Nh * D
    buf = np.arange(n, dtype=np.int32)[::-1].copy()
    got = lo.cols_scatter(buf, Y, ks)
    assert got.shape == (Y, 2, B, S, Nh, D)
    src = buf.reshape(2, B, Y * S, Nh, D)
    for y in range(Y):
        for c in range(2):
            for b in range(B):
                assert np.array_equal(got[y, c, b], src[c, b, y * S:(y + 1) * S])
    assert np.array_equal(lo.cols_gather(got.reshape(-1), Y, ks).reshape(-1), buf)
    if B == 1:      # the expression at orchestrated_attn_impl.py:548
        t = torch.from_numpy(buf).view(2, Y, S * Nh * D).transpose(0, 1).contiguous()
        assert np.array_equal(got.reshape(-1), t.numpy().reshape(-1))
