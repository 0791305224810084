"""Per-shape tile-kernel profile in the format of the reference's cost-model tables
(``prof_data/fit/time_g13_m2_flash_all.json``, read by ``search_algo/search_engine.py:938`` and
``search_algo/utils.py:229-240``):

    {"flash_attn": [[[min(Sq,Skv), bs, Nh, D, "r/c", causal], [fwd us, bwd us, fwd TFLOP/s, bwd TFLOP/s]], ...]}

with ``Sq/Skv = r/c``, FLOPs = ``4*bs*Sq*Skv*Nh*D*(0.5 if causal else 1)`` and backward = 2.5x
(``search_algo/utils.py:92-103``).  Run:  python -m ultraattn_amd.profile_table > time_mi355x.json
"""
import json
import math
import sys
from typing import Iterable, List, Tuple

DEFAULT_SHAPES: Tuple[Tuple[int, int, bool], ...] = tuple(
    (s, nh, causal) for nh in (1, 32) for s in (256, 512, 1024, 2048, 4096, 8192, 16384, 32768) for causal in (True, False))


def profile_entry(S: int, Nh: int, causal: bool, ratio: Tuple[int, int] = (1, 1), iters: int = 10, D: int = 128):
    import torch
    from .flash_attn_interface import _flash_attn_backward, _flash_attn_forward
    from .ops import softmax_delta
    dev = "cuda:0"
    sq, sk = S * ratio[0], S * ratio[1]
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda n: torch.randn(1, n, Nh, D, device=dev, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(sq), mk(sk), mk(sk), mk(sq)
    o, dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    scale = D ** -0.5

    def fwd():
        return _flash_attn_forward(q, k, v, 0.0, scale, causal=causal, out=o)[5]
    lse = fwd()
    delta = softmax_delta(o, do)

    def bwd():
        _flash_attn_backward(do, q, k, v, q, lse, dq, dk, dv, 0.0, scale, causal, softmax_d=delta)
    bwd()
    torch.cuda.synchronize()
    times = []
    for fn in (fwd, bwd):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) / iters * 1e3)          # us
    flops = 4.0 * sq * sk * Nh * D * (0.5 if causal else 1.0)
    return [[min(sq, sk), 1, Nh, D, f"{ratio[0]}/{ratio[1]}", causal],
            [round(times[0], 3), round(times[1], 3), round(flops / times[0] / 1e6, 3), round(2.5 * flops / times[1] / 1e6, 3)]]


def profile_table(shapes: Iterable[Tuple[int, int, bool]] = DEFAULT_SHAPES) -> dict:
    return {"flash_attn": [profile_entry(s, nh, c) for s, nh, c in shapes]}


if __name__ == "__main__":
    json.dump(profile_table(), sys.stdout)
    sys.stdout.write("\n")
