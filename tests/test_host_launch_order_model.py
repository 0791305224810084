"""Quality of the launch orders (q_order, k_order) under a model of one XCD: 64 resident workgroups
that take rows in the kernels' dispatch order (two heads at a time, teams of four positions, heads
alternating team by team), every workgroup one tile per step, and an LRU cache of 64 K/V (or Q/dO)
tiles = the 4 MiB L2 of an XCD.  The model reproduced the measured effect of the order on the device
(strided 128k forward: 80 -> 22 GB fetched per launch, +6 %); here it guards the rule against
regressions on the benchmark masks.  No GPU."""
import collections

import numpy as np
import pytest

from ultraattn_amd import masks
from ultraattn_amd.tilelist import build_tile_list


def lists_of(ptr, idx):
    return [tuple(int(x) for x in idx[ptr[i]:ptr[i + 1]]) for i in range(len(ptr) - 1)]


def simulate(lists, order, slots=64, cap=64, heads=2, team=4):
    """(miss rate of the tile cache, mean occupancy of the slots until the last row ends)."""
    n = len(order)
    seq = []
    full = (n // team) * team
    for t0 in range(0, full, team):
        for h in range(heads):
            seq += [(h, order[t0 + m]) for m in range(team)]
    for h in range(heads):
        seq += [(h, order[p]) for p in range(full, n)]
    cache, miss, acc = collections.OrderedDict(), 0, 0
    active, nxt, steps, busy = [], 0, 0, 0
    while nxt < len(seq) or active:
        while len(active) < slots and nxt < len(seq):
            h, r = seq[nxt]
            nxt += 1
            if lists[r]:
                active.append([h, r, 0])
        if not active:
            break
        steps += 1
        busy += len(active)
        for a in active:
            key = (a[0], lists[a[1]][a[2]])
            acc += 1
            if key in cache:
                cache.move_to_end(key)
            else:
                miss += 1
                cache[key] = 1
                if len(cache) > cap:
                    cache.popitem(last=False)
            a[2] += 1
        active = [a for a in active if a[2] < len(lists[a[1]])]
    return miss / acc, busy / (steps * slots)


def lexicographic(lists):
    """The plain order the rule replaced: very long rows first, the rest by their padded lists."""
    n, nnz = len(lists), sum(map(len, lists))
    key = lambda i: (0, (-len(lists[i]),), i) if len(lists[i]) * n > 2 * nnz else (1, lists[i] + (1 << 40,), i)
    return sorted(range(n), key=key)


CASES = [("strided 128k rows", masks.config_strided, "q", 0.12), ("strided 128k columns", masks.config_strided, "k", 0.12),
         ("global+local 128k rows", masks.config_global_local, "q", 0.09), ("global+local 128k columns", masks.config_global_local, "k", 0.09),
         ("causal 32k rows", lambda: masks.config_causal(64), "q", 0.09), ("causal 32k columns", lambda: masks.config_causal(64), "k", 0.05),
         ("streaming shard rows", masks.config_streaming_shard, "q", 0.06)]


def _shard_key_range(part):
    """One of the four key-range kernel tiles of the streaming shard (as bench.py splits it)."""
    mask = masks.config_streaming_shard()
    cols = np.array_split(np.nonzero(mask.any(0))[0], 4)[part]
    sub = np.zeros_like(mask)
    sub[:, cols] = mask[:, cols]
    return sub


CASES += [(f"streaming shard, key range {p} of 4, rows", (lambda p=p: _shard_key_range(p)), "q", 0.08) for p in range(4)]


@pytest.mark.parametrize("name,make,side,bound", CASES, ids=[c[0] for c in CASES])
def test_launch_order_keeps_shared_tiles_in_cache(name, make, side, bound):
    tl = build_tile_list(make(), block=512)
    ptr, idx, order = (tl.row_ptr, tl.col_idx, tl.q_order) if side == "q" else (tl.col_ptr, tl.row_idx, tl.k_order)
    lists = lists_of(ptr, idx)
    miss, occupancy = simulate(lists, order.tolist())
    ref_miss, _ = simulate(lists, lexicographic(lists))
    assert miss <= bound, (name, miss)
    assert miss <= ref_miss + 0.005, (name, miss, ref_miss)
    assert occupancy >= (0.985 if "key range" not in name else 0.95), (name, occupancy)
