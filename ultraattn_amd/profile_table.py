"""Per-shape tile-kernel profile in the format of the reference's cost-model tables
(``prof_data/fit/time_g13_m2_flash_all.json``, read by ``search_algo/search_engine.py:938`` through
``convert_profile_data_to_map``, ``search_algo/utils.py:229-240``):

    {"flash_attn": [[[min(Sq,Skv), bs, Nh, D, "r/c", causal], [fwd us, bwd us, fwd TFLOP/s, bwd TFLOP/s]], ...]}

with ``Sq/Skv = r/c`` in lowest terms (the planner's key, ``search_algo/search_engine.py:166-196``),
FLOPs = ``4*bs*Sq*Skv*Nh*D*(0.5 if causal else 1)`` and backward = 2.5x
(``search_algo/utils.py:92-103``).  The default key space is the reference table's: 160 keys,
S = 256 ... 131072, Nh in {1, 32}, ratios 1/1 (causal and not), 2/1, 1/2, 3/1, 1/3, 4/1, 1/4.

Run on the GPU:  python -m ultraattn_amd.profile_table > time_mi355x_flash_all.json
"""
import json
import sys
from typing import Iterable, List, Tuple

S_VALUES = tuple(256 << i for i in range(10))                      # 256 ... 131072
HEADS = (1, 32)
RATIO_CAUSAL = (((1, 1), True), ((1, 1), False), ((2, 1), False), ((1, 2), False), ((3, 1), False),
                ((1, 3), False), ((4, 1), False), ((1, 4), False))
HEAD_DIM = 128

# (S, Nh, causal, (r, c)) for every key of the reference table
DEFAULT_SHAPES: Tuple[Tuple[int, int, bool, Tuple[int, int]], ...] = tuple(
    (s, nh, causal, ratio) for nh in HEADS for ratio, causal in RATIO_CAUSAL for s in S_VALUES)


def tile_flops(S: int, Nh: int, causal: bool, ratio: Tuple[int, int] = (1, 1), bs: int = 1, D: int = HEAD_DIM) -> float:
    """Forward FLOPs of one dense tile by the reference's convention (``search_algo/utils.py:92-103``)."""
    return 4.0 * bs * (S * ratio[0]) * (S * ratio[1]) * Nh * D * (0.5 if causal else 1.0)


def format_entry(S: int, Nh: int, causal: bool, ratio: Tuple[int, int], fwd_us: float, bwd_us: float,
                 bs: int = 1, D: int = HEAD_DIM) -> list:
    """One table row from measured times: key as the planner builds it, times in microseconds,
    TFLOP/s columns = FLOPs / time with the backward counted 2.5x."""
    flops = tile_flops(S, Nh, causal, ratio, bs, D)
    return [[S, bs, Nh, D, f"{ratio[0]}/{ratio[1]}", bool(causal)],
            [round(fwd_us, 3), round(bwd_us, 3), round(flops / fwd_us / 1e6, 3), round(2.5 * flops / bwd_us / 1e6, 3)]]


def time_tile(S: int, Nh: int, causal: bool, ratio: Tuple[int, int] = (1, 1), budget_s: float = 0.25, D: int = HEAD_DIM,
              use_graph: bool = True):
    """(fwd us, bwd us) of one dense ``Sq x Skv`` tile, Sq = S*r, Skv = S*c, through the drop-in
    ``_flash_attn_forward`` / ``_flash_attn_backward`` (``ua_dense_fwd`` / ``ua_dense_bwd``, which cut
    rectangles with few tile lines into parts); the iteration count follows a first timed launch so
    that every shape costs about ``budget_s`` per direction."""
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

    def timed(fn, iters):
        """us per call.  The calls are recorded into one HIP graph and the graph's replay is timed,
        so that what is measured is the device's time per call (kernels and the gaps between
        dependent launches) and not the host's cost of issuing a call from Python, which for tiles
        of a few microseconds would be all that is seen."""
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if use_graph:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for _ in range(iters):
                    fn()
            graph.replay()
            torch.cuda.synchronize()
            e0.record()
            graph.replay()
            e1.record()
        else:
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3                     # us
    out = []
    for fn in (fwd, bwd):
        first = timed(fn, 1)
        iters = max(1, min(50, int(budget_s * 1e6 / max(first, 1.0))))
        out.append(timed(fn, iters) if iters > 1 else first)
    return out[0], out[1]


def profile_entry(S: int, Nh: int, causal: bool, ratio: Tuple[int, int] = (1, 1), budget_s: float = 0.25):
    fwd_us, bwd_us = time_tile(S, Nh, causal, ratio, budget_s)
    return format_entry(S, Nh, causal, ratio, fwd_us, bwd_us)


def profile_table(shapes: Iterable[Tuple[int, int, bool, Tuple[int, int]]] = DEFAULT_SHAPES,
                  budget_s: float = 0.25, progress=None) -> dict:
    rows: List[list] = []
    for s, nh, causal, ratio in shapes:
        rows.append(profile_entry(s, nh, causal, ratio, budget_s))
        if progress:
            progress(rows[-1])
    return {"flash_attn": rows}


if __name__ == "__main__":
    table = profile_table(progress=lambda r: print(json.dumps(r), file=sys.stderr, flush=True))
    json.dump(table, sys.stdout)
    sys.stdout.write("\n")
