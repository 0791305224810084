"""Regenerates the fixtures in this directory.  Run from the repo root:

    python tests/golden/make_golden.py

1. ``reference_data.json`` — DATA the reference holds for this path, read as text from
   ``/root/reference`` (only where that directory exists; the committed JSON is what the tests
   use): the canonical block-table strings of ``plot/e2e_pick.py:65-72``, the block tables and
   per-GPU "Allocation Matrix" results printed in ``prof_data/intra_tiles/**/wp_gurobi_*.log``
   and the ``total_sparsity`` the reference logged for the matching configuration
   (``prof_data/fit/wrapper_intra_SP=8_all_BSA_H800.log:8,55``).
2. ``twin_*.npz`` — down-scaled twins of the benchmark configurations (same mask patterns,
   128-token tiles, head_dim 128, 2 heads), inputs drawn from a seeded CPU generator, outputs
   computed by the fp64 dense oracle; sampled rows only, to stay small.
3. ``tilelists.json`` — counts and SHA-256 of the full-size active-tile lists.
"""
import glob
import hashlib
import json
import math
import os
import re
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
REF = "/root/reference"

from oracle import attn_oracle as ao            # noqa: E402
from oracle import tilelist_oracle as to        # noqa: E402


def reference_data():
    out = {}
    src = open(os.path.join(REF, "plot/e2e_pick.py")).read().splitlines()
    out["bsa_reprs"] = {"source": "plot/e2e_pick.py:65-72",
                        "strings": [re.search(r"'(\[\[.*\]\])'", l).group(1) for l in src[65:71]]}
    allocs = []
    for path in sorted(glob.glob(os.path.join(REF, "prof_data/intra_tiles/*/*/wp_gurobi_*.log"))):
        lines = open(path).read().splitlines()
        assert lines[0].startswith("block_table_value")
        table, i = [], 1
        while lines[i].lstrip().startswith("["):
            table.append([int(x) for x in re.findall(r"\d", lines[i])])
            i += 1
        j = lines.index("Allocation Matrix:")
        alloc = [[-1 if t == "/" else int(t) for t in l.split()] for l in lines[j + 1:j + 1 + len(table)]]
        allocs.append({"source": os.path.relpath(path, REF), "block_table": table, "allocation": alloc})
    out["allocations"] = allocs
    log = open(os.path.join(REF, "prof_data/fit/wrapper_intra_SP=8_all_BSA_H800.log")).read().splitlines()
    assert "bsa_config=8_8_lg_1-4_3&3_0&0_2" in log[7] and log[54].startswith("total_sparsity")
    out["sparsity"] = {"source": "prof_data/fit/wrapper_intra_SP=8_all_BSA_H800.log:8,55",
                       "bsa_config": "8_8_lg_1-4_3&3_0&0_2", "total_sparsity": float(log[54].split(":")[1]),
                       "block_table_source": "prof_data/intra_tiles/stride_16_4_3/8x2/wp_gurobi_8_8_lg_1-4_3_0_2_lb_allint.log"}
    return out


def twin_masks():
    from ultraattn_amd import masks
    return {
        "c1_causal": (masks.config_causal(4), 256),
        "c3_strided": (masks.config_strided(16, 4, 8), 128),
        "c4_global_local": (masks.config_global_local(16, 1, 2), 128),
        "c5_streaming": (masks.config_streaming_shard(4, 16, 3), 128),
    }


def twin_inputs(mask, block, seed, nh=2, d=128):
    g = torch.Generator().manual_seed(seed)
    nqb, nkb = mask.shape
    mk = lambda n: torch.randn(1, n * block, nh, d, generator=g, dtype=torch.float32).to(torch.bfloat16)
    return mk(nqb), mk(nkb), mk(nkb), mk(nqb)      # q, k, v, do


def make_twins():
    for name, (mask, block) in twin_masks().items():
        q, k, v, do = twin_inputs(mask, block, seed=1234)
        keep = ao.element_mask(mask, block)
        scale = 1.0 / math.sqrt(128)
        o, lse = ao.dense_fwd(q, k, v, scale, keep, dtype=torch.float64)
        dq, dk, dv = ao.dense_bwd_autograd(q, k, v, do, scale, keep)
        rs = np.random.RandomState(7)
        qrows = np.sort(rs.choice(q.shape[1], 32, replace=False))
        krows = np.sort(rs.choice(k.shape[1], 32, replace=False))
        digest = hashlib.sha256(b"".join(t.float().numpy().tobytes() for t in (q, k, v, do))).hexdigest()
        np.savez_compressed(os.path.join(HERE, f"twin_{name}.npz"), mask=mask, block=block, seed=1234,
                            inputs_sha256=digest, qrows=qrows, krows=krows,
                            o=o[:, qrows].float().numpy(), lse=lse.float().numpy(),
                            dq=dq[:, qrows].float().numpy(), dk=dk[:, krows].float().numpy(),
                            dv=dv[:, krows].float().numpy())
        print(name, "written")


def make_tilelists():
    from ultraattn_amd import masks
    cfgs = {"c1": masks.config_causal(16), "c2": masks.config_causal(64), "c3": masks.config_strided(),
            "c4": masks.config_global_local(), "c5": masks.config_streaming_shard()}
    out = {}
    for name, m in cfgs.items():
        tl = to.build_tile_list(m, 4)
        h = hashlib.sha256()
        for a in (tl["row_ptr"], tl["col_idx"], tl["flag"]):
            h.update(np.ascontiguousarray(a).tobytes())
        out[name] = {"blocks": int((m != 0).sum()), "causal_blocks": int((m == 2).sum()),
                     "tiles": int(tl["col_idx"].shape[0]), "causal_tiles": int(tl["flag"].sum()),
                     "sha256": h.hexdigest()}
    json.dump(out, open(os.path.join(HERE, "tilelists.json"), "w"), indent=1)


if __name__ == "__main__":
    if os.path.isdir(REF):
        json.dump(reference_data(), open(os.path.join(HERE, "reference_data.json"), "w"), indent=1)
    make_tilelists()
    make_twins()
