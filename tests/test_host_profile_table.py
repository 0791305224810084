"""Cost-table emitter (ultraattn_amd.profile_table): key space, format and FLOP columns, checked
with a restatement of the reference's reader and one row the reference's own table holds."""
import json

import numpy as np
import pytest

from ultraattn_amd import profile_table as pt


def convert_profile_data_to_map(profile_list):
    """What the planner does with the table (search_algo/utils.py:229-240): tuple keys, unique,
    values = the first two columns (fwd, bwd microseconds) in seconds."""
    profile_map = {}
    for key, val in profile_list:
        map_key = tuple(key)
        assert map_key not in profile_map
        profile_map[map_key] = np.array(val[:2]) / 1e6
    return profile_map


def test_key_space_is_the_reference_tables():
    """prof_data/fit/time_g13_m2_flash_all.json: 160 keys = 10 sequence lengths 256..131072 x
    Nh {1, 32} x {1/1 causal, 1/1, 2/1, 1/2, 3/1, 1/3, 4/1, 1/4}; bs = 1, D = 128."""
    rows = [pt.format_entry(s, nh, c, r, 1.0, 1.0) for s, nh, c, r in pt.DEFAULT_SHAPES]
    table = json.loads(json.dumps({"flash_attn": rows}))            # what a reader of the file sees
    m = convert_profile_data_to_map(table["flash_attn"])
    assert len(m) == 160
    want = {(s, 1, nh, 128, ratio, causal) for s in (256 << i for i in range(10)) for nh in (1, 32)
            for ratio, causal in [("1/1", True), ("1/1", False), ("2/1", False), ("1/2", False), ("3/1", False),
                                  ("1/3", False), ("4/1", False), ("1/4", False)]}
    assert set(m) == want and max(k[0] for k in m) == 131072
    # the planner's own key for a split (search_algo/search_engine.py:166-196): min(Sq, Skv), bs, Nh, D,
    # "Sq/gcd / Skv/gcd", causal — every ratio it accepts with these entries is present
    for sq, skv in [(8192, 8192), (16384, 8192), (8192, 32768), (24576, 8192)]:
        g = np.gcd(sq, skv)
        assert (min(sq, skv), 1, 32, 128, f"{sq // g}/{skv // g}", False) in m


def test_flop_columns_follow_the_reference_convention():
    # a row of the reference's table (prof_data/fit/time_g13_m2_flash_all.json, last rows):
    # [[131072, 1, 32, 128, "1/3", false], [3577099.365, 10443382.812, 236.064, 202.144]]
    row = pt.format_entry(131072, 32, False, (1, 3), 3577099.365, 10443382.812)
    assert row == [[131072, 1, 32, 128, "1/3", False], [3577099.365, 10443382.812, 236.064, 202.144]]
    # [[1024, 1, 1, 128, "1/1", true], [22.528, 112.64, 11.916, 5.958]]: causal counts half
    row = pt.format_entry(1024, 1, True, (1, 1), 22.528, 112.64)
    assert row == [[1024, 1, 1, 128, "1/1", True], [22.528, 112.64, 11.916, 5.958]]
    assert pt.tile_flops(512, 32, True) == 4 * 512 * 512 * 32 * 128 * 0.5
    assert pt.tile_flops(512, 2, False, (4, 1)) == 4 * 2048 * 512 * 2 * 128


@pytest.mark.gpu
def test_three_entries_on_the_gpu():
    rows = pt.profile_table([(256, 1, True, (1, 1)), (1024, 32, False, (2, 1)), (512, 32, False, (1, 4))],
                            budget_s=0.02)["flash_attn"]
    m = convert_profile_data_to_map(rows)
    assert set(m) == {(256, 1, 1, 128, "1/1", True), (1024, 1, 32, 128, "2/1", False), (512, 1, 32, 128, "1/4", False)}
    for key, val in rows:
        fwd_us, bwd_us, fwd_tf, bwd_tf = val
        assert 0 < fwd_us < bwd_us * 4 and 0 < fwd_tf < 2600 and 0 < bwd_tf < 2600
        r, c = (int(x) for x in key[4].split("/"))
        assert fwd_tf == pytest.approx(pt.tile_flops(key[0], key[2], key[5], (r, c)) / fwd_us / 1e6, rel=1e-3, abs=2e-3)
