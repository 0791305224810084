#!/usr/bin/env python3
"""Benchmark of the block-sparse attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3|c4|c2|c5] [--no-extra] [--no-cpu]

A step is one pass of the hot path over one batch of synthetic input: forward, delta, dK/dV and
dQ for the forward+backward workloads (c3 = strided 128k, the default; c4 = global+local 128k),
forward only for c2 (causal 32k) and forward tiles + merge for c5 (streaming shard).  Inputs are
resident in HBM before the timed region.  Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

BLOCK = 512
HEADS = 32
SCALE = 1.0 / math.sqrt(128)
HBM_PEAK_GBPS = 8000.0            # MI355X HBM3E, published
FLOP_PER_CLK_PER_CU = 4096        # dense bf16 MFMA, CDNA4


# HBM-side bytes per launch, NOT measured by this run: constants copied from the rocprofv3 --pmc
# summaries under profiles/ (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, scaling explained there).  Every
# roofline entry names the file its figure comes from; a kernel without a summary gets null.
TRAFFIC_BYTES = {}        # filled from profiles/hbm_traffic_<workload>.txt by load_traffic()


def load_traffic():
    """Parse the 'HBM-side bytes per launch after scaling' tables of profiles/hbm_traffic_*.txt."""
    import glob
    import re
    for path in sorted(glob.glob(os.path.join(ROOT, "profiles", "hbm_traffic_*.txt"))):
        w = os.path.basename(path)[len("hbm_traffic_"):-4]
        for m in re.finditer(r"^\s+ua::(\S+)\s+([0-9.]+) GB\s*$", open(path).read(), flags=re.M):
            TRAFFIC_BYTES[(w, m.group(1))] = (float(m.group(2)) * 1e9, os.path.relpath(path, ROOT))


MEASURED_MFMA_CEILING = [None]     # TFLOP/s, set from this run's own register-only MFMA probe


def roof_entry(workload, kernel, bound, achieved, peak, unit, kernel_ms, algorithmic, kernel_ms_min=None):
    """`achieved`, `kernel_ms`: median over the repeats of the timed block; `*_min`: the best repeat."""
    tr = TRAFFIC_BYTES.get((workload, kernel))
    e = {"workload": workload, "kernel": kernel, "bound": bound, "achieved": achieved, "peak": peak, "unit": unit,
         "frac": achieved / peak, "kernel_ms": kernel_ms,
         "traffic": tr[0] if tr else None,
         "traffic_source": (tr[1] + " (rocprofv3 --pmc, a constant from that file, not measured in this run)") if tr else None}
    e["algorithmic_flops" if bound == "mfma" else "algorithmic_bytes"] = algorithmic
    if kernel_ms_min:
        e["kernel_ms_min"] = kernel_ms_min
        e["achieved_best"] = achieved * kernel_ms / kernel_ms_min
    if bound == "mfma" and MEASURED_MFMA_CEILING[0]:
        # against what the matrix pipes of THIS device deliver to a register-only loop on random bf16 data
        e["measured_mfma_ceiling"] = MEASURED_MFMA_CEILING[0]
        e["frac_of_measured_mfma_ceiling"] = achieved / MEASURED_MFMA_CEILING[0]
    return e


def attention_roofs(workload, res, peak):
    """Roofline entries of the attention kernels of one workload result (algorithmic flops by the
    reference's convention: forward F, dK/dV 4 of the backward's 5 GEMMs = 2.0 F, dQ 1 of 5 = 0.5 F)."""
    F = res["fwd_flops"]
    mn = res.get("min", {})
    launches = 4 if workload == "c5" else 1          # c5 runs the forward as 4 kernel tiles
    per = lambda key: mn[key] / launches if key in mn else None
    out = [roof_entry(workload, "fwd_kernel", "mfma", res["fwd_tflops"], peak, "TFLOP/s", res["fwd_ms"] / launches, F / launches,
                      per("fwd_ms"))]
    if "dkdv_ms" in res:
        out.append(roof_entry(workload, "dkdv_kernel", "mfma", 2.0 * F / res["dkdv_ms"] / 1e9, peak, "TFLOP/s", res["dkdv_ms"], 2.0 * F,
                              mn.get("dkdv_ms")))
        out.append(roof_entry(workload, "dq_kernel", "mfma", 0.5 * F / res["dq_ms"] / 1e9, peak, "TFLOP/s", res["dq_ms"], 0.5 * F,
                              mn.get("dq_ms")))
        nbytes = res["delta_gbps"] * res["delta_ms"] * 1e6
        out.append(roof_entry(workload, "delta_kernel", "hbm", res["delta_gbps"], HBM_PEAK_GBPS, "GB/s", res["delta_ms"], nbytes,
                              mn.get("delta_ms")))
    if "merge_ms" in res:
        out.append(roof_entry(workload, "merge_kernel<4>", "hbm", res["merge_gbps"], HBM_PEAK_GBPS, "GB/s", res["merge_ms"],
                              res["merge_bytes"], mn.get("merge_ms")))
    return out


REPEATS = 3          # the reference's protocol: warm-up, then 3 repeats of the timed block (search_algo/benchmark.py:197-216)


def median_min(repeats):
    """repeats: list of {name: ms}.  -> ({name: median}, {name: min})"""
    keys = repeats[0].keys()
    med = {k: sorted(r[k] for r in repeats)[len(repeats) // 2] for k in keys}
    return med, {k: min(r[k] for r in repeats) for k in keys}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


_probe_lib = None


def probe_lib():
    """libbench_probe.so: the benchmark's own device probes (not part of the product library)."""
    global _probe_lib
    if _probe_lib is None:
        import ctypes
        path = os.path.join(ROOT, "libbench_probe.so")
        if not os.path.exists(path):
            sys.exit(f"{path} is missing: build it with `python -m ultraattn_amd.build`")
        lib = ctypes.CDLL(path)
        vp, ci = ctypes.c_void_p, ctypes.c_int
        lib.bench_probe_mfma.restype, lib.bench_probe_mfma.argtypes = ci, [vp, vp, ci, ci, vp]
        lib.bench_probe_mfma_rotating.restype, lib.bench_probe_mfma_rotating.argtypes = ci, [vp, vp, ci, ci, vp]
        lib.bench_probe_mfma16_rotating.restype, lib.bench_probe_mfma16_rotating.argtypes = ci, [vp, vp, ci, ci, vp]
        lib.bench_atomic_rate.restype, lib.bench_atomic_rate.argtypes = ci, [vp, ctypes.c_int64, ci, ci, ci, vp]
        lib.bench_stream_mix.restype = ci
        lib.bench_stream_mix.argtypes = [ctypes.POINTER(vp), ci, vp, ctypes.c_int64, ci, ci, vp]
        lib.bench_issue_mix.restype, lib.bench_issue_mix.argtypes = ci, [vp, ci, ci, ci, ci, vp]
        _probe_lib = lib
    return _probe_lib


def workload_mask(name):
    from ultraattn_amd import masks
    return {"c2": masks.config_causal(64), "c3": masks.config_strided(), "c4": masks.config_global_local(),
            "c5": masks.config_streaming_shard()}[name]


def fwd_flops(mask, nh=HEADS, block=BLOCK):
    """Reference convention (search_algo/utils.py:92-103): 4*Sq*Skv*Nh*D*density, CAUSAL = 0.5."""
    nf, nc = int((mask == 1).sum()), int((mask == 2).sum())
    return 4.0 * block * block * 128 * nh * (nf + 0.5 * nc)


class Timer:
    """HIP events on the stream the kernels are launched on (torch's current stream)."""

    def __init__(self, torch, names):
        self.torch, self.names = torch, names
        self.acc = {n: 0.0 for n in names}
        self.marks = []

    def mark(self):
        e = self.torch.cuda.Event(enable_timing=True)
        e.record()
        self.marks.append(e)

    def collect(self):
        """Call after a synchronize: fold the recorded marks into per-kernel sums."""
        per = len(self.names) + 1
        for i in range(0, len(self.marks), per):
            for j, n in enumerate(self.names):
                self.acc[n] += self.marks[i + j].elapsed_time(self.marks[i + j + 1])
        self.marks = []


def run_attention(name, steps, warmup, backward):
    import torch
    from ultraattn_amd import ops
    from ultraattn_amd.tilelist import build_tile_list
    dev = "cuda:0"
    mask = workload_mask(name)
    nqb, nkb = mask.shape
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda n: torch.randn(1, n * BLOCK, HEADS, 128, device=dev, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v = mk(nqb), mk(nkb), mk(nkb)
    t0 = time.perf_counter()
    tl = build_tile_list(mask, BLOCK)
    tl.on(dev)
    t_build = time.perf_counter() - t0
    o = torch.empty_like(q)
    lse = torch.empty(1, HEADS, nqb * BLOCK, dtype=torch.float32, device=dev)
    names = ["fwd"]
    if backward:
        do = mk(nqb)
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        delta = torch.empty_like(lse)
        names += ["delta", "bwd"]

    def step(t=None):
        if t: t.mark()
        ops.bsa_fwd(q, k, v, tl, SCALE, out=o, lse=lse)
        if t: t.mark()
        if backward:
            ops.softmax_delta(o, do, delta)
            if t: t.mark()
            ops.bsa_bwd(do, q, k, v, None, lse, tl, SCALE, dq=dq, dk=dk, dv=dv, softmax_d=delta)
            if t: t.mark()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    reps = []
    for _ in range(REPEATS):                  # each repeat times exactly `steps` steps
        timer = Timer(torch, names)
        t0 = time.perf_counter()
        for _ in range(steps):
            step(timer)
        torch.cuda.synchronize()
        rep = {"ms_per_step": (time.perf_counter() - t0) * 1e3 / steps}
        timer.collect()
        rep.update({n + "_ms": timer.acc[n] / steps for n in names})
        reps.append(rep)
    ms, mn = median_min(reps)
    wall_ms = ms["ms_per_step"]
    F = fwd_flops(mask)
    res = {"workload": name, "tiles_per_head": tl.nnz, "tilelist_sha256": tl.sha256(), "tilelist_build_ms": t_build * 1e3,
           "ms_per_step": wall_ms, "fwd_ms": ms["fwd_ms"], "fwd_tflops": F / ms["fwd_ms"] / 1e9, "fwd_flops": F,
           "repeats": reps, "min": mn, "fwd_tflops_best": F / mn["fwd_ms"] / 1e9}
    if backward:
        res.update(bwd_ms=ms["bwd_ms"], delta_ms=ms["delta_ms"], bwd_tflops=2.5 * F / (ms["bwd_ms"] + ms["delta_ms"]) / 1e9,
                   fwd_bwd_tflops=3.5 * F / wall_ms / 1e9, fwd_bwd_tflops_best=3.5 * F / mn["ms_per_step"] / 1e9,
                   delta_gbps=(2 * q.numel() * 2 + lse.numel() * 4) / ms["delta_ms"] / 1e6)
    return res


def time_bwd_kernels(name, steps):
    """Separate event timing of the two backward kernels (dK/dV walks the CSC, dQ the CSR)."""
    import ctypes
    import torch
    from ultraattn_amd import _lib, ops
    from ultraattn_amd.tilelist import build_tile_list
    dev = "cuda:0"
    mask = workload_mask(name)
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda n: torch.randn(1, n * BLOCK, HEADS, 128, device=dev, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(mask.shape[0]), mk(mask.shape[1]), mk(mask.shape[1]), mk(mask.shape[0])
    tl = build_tile_list(mask, BLOCK)
    d = tl.on(dev)
    o, lse = ops.bsa_fwd(q, k, v, tl, SCALE)
    delta = ops.softmax_delta(o, do)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    s3 = _lib.strides3

    def dkdv():
        _lib.check(lib.ua_bsa_bwd_dkdv(q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(),
                                       delta.data_ptr(), dk.data_ptr(), dv.data_ptr(), d["col_ptr"].data_ptr(),
                                       d["row_idx"].data_ptr(), d["cflag"].data_ptr(), d["k_order"].data_ptr(),
                                       1, HEADS, tl.n_qtiles, tl.n_ktiles, tl.nnz, 128, s3(q), s3(k), s3(v), s3(do), s3(dk),
                                       s3(dv), SCALE, st), "dkdv")

    def dqk():
        _lib.check(lib.ua_bsa_bwd_dq(q.data_ptr(), k.data_ptr(), v.data_ptr(), do.data_ptr(), lse.data_ptr(),
                                     delta.data_ptr(), dq.data_ptr(), d["row_ptr"].data_ptr(), d["col_idx"].data_ptr(),
                                     d["flag"].data_ptr(), d["q_order"].data_ptr(), 1, HEADS, tl.n_qtiles,
                                     tl.n_ktiles, tl.nnz, 128, s3(q), s3(k), s3(v), s3(do), s3(dq), SCALE, st), "dq")
    dkdv(); dqk()
    torch.cuda.synchronize()
    reps = []
    for _ in range(REPEATS):
        t = Timer(torch, ["dkdv", "dq"])
        for _ in range(steps):
            t.mark(); dkdv(); t.mark(); dqk(); t.mark()
        torch.cuda.synchronize()
        t.collect()
        reps.append({n + "_ms": t.acc[n] / steps for n in t.names})
    return median_min(reps)


def run_c5(steps, warmup):
    """Streaming shard: 4 key-range kernel tiles -> partial (O, LSE) -> merge."""
    import numpy as np
    import torch
    from ultraattn_amd import ops
    from ultraattn_amd.tilelist import build_tile_list
    dev = "cuda:0"
    mask = workload_mask("c5")
    nqb, nkb = mask.shape
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda n: torch.randn(1, n * BLOCK, HEADS, 128, device=dev, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v = mk(nqb), mk(nkb), mk(nkb)
    cols = np.nonzero(mask.any(0))[0]
    tls = []
    for c in np.array_split(cols, 4):
        sub = np.zeros_like(mask)
        sub[:, c] = mask[:, c]
        tls.append(build_tile_list(sub, BLOCK))
    p_o = [torch.empty_like(q) for _ in tls]
    p_l = [torch.empty(1, HEADS, nqb * BLOCK, dtype=torch.float32, device=dev) for _ in tls]
    o, lse = torch.empty_like(q), torch.empty_like(p_l[0])

    def step(t=None):
        if t: t.mark()
        for tl, po, pl in zip(tls, p_o, p_l):
            ops.bsa_fwd(q, k, v, tl, SCALE, out=po, lse=pl)
        if t: t.mark()
        ops.merge_partials(p_o, p_l, out=o, lse=lse)
        if t: t.mark()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    reps = []
    for _ in range(REPEATS):
        timer = Timer(torch, ["fwd_tiles", "merge"])
        t0 = time.perf_counter()
        for _ in range(steps):
            step(timer)
        torch.cuda.synchronize()
        rep = {"ms_per_step": (time.perf_counter() - t0) * 1e3 / steps}
        timer.collect()
        rep.update(fwd_ms=timer.acc["fwd_tiles"] / steps, merge_ms=timer.acc["merge"] / steps)
        reps.append(rep)
    med, mn = median_min(reps)
    wall_ms = med["ms_per_step"]
    F = fwd_flops(mask)
    rows = nqb * BLOCK * HEADS
    merge_bytes = (len(tls) + 1) * rows * (128 * 2 + 4)
    m_ms, f_ms = med["merge_ms"], med["fwd_ms"]
    # the device's rate for the merge's memory pattern without its arithmetic: 4 streams read, 1 written,
    # 16-byte accesses, one load step per workgroup, on the same buffers
    import ctypes
    lib = probe_lib()
    nb = p_o[0].numel() * 2
    arr = (ctypes.c_void_p * 4)(*[t.data_ptr() for t in p_o])
    st = torch.cuda.current_stream().cuda_stream
    blocks = nb // (256 * 4 * 16)
    assert lib.bench_stream_mix(arr, 4, o.data_ptr(), nb, blocks, 1, st) == 0
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        lib.bench_stream_mix(arr, 4, o.data_ptr(), nb, blocks, 1, st)
    e1.record()
    torch.cuda.synchronize()
    mix_gbps = 5 * nb / (e0.elapsed_time(e1) / 10) / 1e6
    return {"workload": "c5", "stream_mix_4r1w_gbps": mix_gbps, "merge_frac_of_stream_mix": merge_bytes / m_ms / 1e6 / mix_gbps, "ms_per_step": wall_ms, "fwd_ms": f_ms, "fwd_tflops": F / f_ms / 1e9, "fwd_flops": F,
            "merge_ms": m_ms, "merge_bytes": merge_bytes, "merge_gbps": merge_bytes / m_ms / 1e6,
            "merge_frac_of_hbm": merge_bytes / m_ms / 1e6 / HBM_PEAK_GBPS,
            "merge_gbps_best": merge_bytes / mn["merge_ms"] / 1e6,
            "fwd_plus_merge_tflops": F / wall_ms / 1e9, "repeats": reps, "min": mn}


def run_mask_builder(name, steps):
    """Device tile-list builder on one workload's block mask: 4 small launches (count, scan,
    fill, order).  Bytes = block mask read + the eight tile-list arrays written."""
    import torch
    from ultraattn_amd.tilelist import build_tile_list, build_tile_list_device
    mask = workload_mask(name)
    host = build_tile_list(mask, BLOCK)
    m = torch.from_numpy(mask.astype("uint8")).to("cuda:0")
    dev = build_tile_list_device(m, BLOCK, nnz=host.nnz)
    torch.cuda.synchronize()
    same = all(bool((dev[n].cpu() == torch.from_numpy(getattr(host, n))).all())
               for n in ("row_ptr", "col_idx", "flag", "col_ptr", "row_idx", "cflag", "q_order", "k_order"))
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        build_tile_list_device(m, BLOCK, nnz=host.nnz)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    nbytes = mask.size + 2 * host.nnz * 5 + 4 * (2 * (host.n_qtiles + host.n_ktiles) + 2)
    return {"workload": name, "ms": ms, "bytes": nbytes, "gbps": nbytes / ms / 1e6, "nnz_tiles": host.nnz,
            "matches_host_builder": same, "note": "latency-bound: 11 small dependent launches over a few MB"}


def run_cols_gather(steps):
    """Column gather of a fused rectangle at the 128k shape: 4 chunks of [K | V], 32768 keys each."""
    import torch
    from ultraattn_amd import packed
    Y, ks = 4, (1, 32768, HEADS, 128)
    n = 2 * Y * ks[1] * ks[2] * ks[3]
    buf = torch.empty(n, dtype=torch.bfloat16, device="cuda:0").normal_()
    out = torch.empty_like(buf)
    packed.gather_cols(buf, Y, ks, out=out)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        packed.gather_cols(buf, Y, ks, out=out)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    return {"ms": ms, "bytes": 4 * n, "gbps": 4 * n / ms / 1e6, "frac_of_hbm": 4 * n / ms / 1e6 / HBM_PEAK_GBPS,
            "shape": "[4, 2, 1, 32768, 32, 128] -> [2, 1, 131072, 32, 128] bf16, read + write"}


def run_dense_split(steps):
    """A dense rectangle with few tile lines (Sq=1024, Skv=4096, one head: 8 query tiles x 32 key tiles)
    through the flash-attn call signature: the library cuts the walks into parts that fill the device
    (forward: partial (O, LSE) + merge; backward: fp32 partial gradients + one sum).  Device time per
    call from a HIP graph replay, next to the same entry points run unsplit (no workspace)."""
    import torch
    from ultraattn_amd import _lib, ops
    from ultraattn_amd.flash_attn_interface import _flash_attn_backward, _flash_attn_forward
    dev = "cuda:0"
    sq, sk = 1024, 4096
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda n: torch.randn(1, n, 1, 128, device=dev, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(sq), mk(sk), mk(sk), mk(sq)
    o, dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    lse = _flash_attn_forward(q, k, v, 0.0, SCALE, causal=False, out=o)[5]
    delta = ops.softmax_delta(o, do)
    lib = _lib.load()
    s3 = _lib.strides3

    def unsplit_fwd():
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.ua_dense_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), lse.data_ptr(), 1, 1, sq, sk, 128,
                                    s3(q), s3(k), s3(v), s3(o), SCALE, 0, None, 0, st), "ua_dense_fwd")

    def unsplit_bwd():
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.ua_dense_bwd(do.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), lse.data_ptr(), delta.data_ptr(),
                                    dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), 1, 1, sq, sk, 128, s3(q), s3(k), s3(v), s3(do),
                                    s3(dq), s3(dk), s3(dv), SCALE, 0, None, 0, st), "ua_dense_bwd")
    runs = {"fwd_split_us": lambda: _flash_attn_forward(q, k, v, 0.0, SCALE, causal=False, out=o),
            "fwd_unsplit_us": unsplit_fwd,
            "bwd_split_us": lambda: _flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, 0.0, SCALE, False, softmax_d=delta),
            "bwd_unsplit_us": unsplit_bwd}
    res = {"shape": "Sq=1024 Skv=4096 Nh=1 d=128 bf16, not causal (8 x 32 tiles)"}
    for key, fn in runs.items():
        fn()
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(steps):
                fn()
        graph.replay()
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(REPEATS):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            graph.replay()
            e1.record()
            torch.cuda.synchronize()
            best = min(best, e0.elapsed_time(e1) / steps * 1e3)
        res[key] = best
    res["reference_h800_us"] = {"fwd": 23.392, "bwd": 86.88,
                                "source": "prof_data/fit/time_g40_m2_flash_all.json, key [1024, 1, 1, 128, \"1/4\", false]"}
    return res


def run_per_rectangle(name):
    """What the single launch over a tile list replaces: the reference's executors run a device's
    share as one dense flash-attention call per (row chunk, column chunk) rectangle and fold the
    partial (O, LSE) pairs (orchestrated_attn_impl.py:348-349, ring_flash_attn/utils.py:78-99).  The
    same kernels driven that way (BlockSparseExecutor.forward_per_rectangle: ua_dense_fwd +
    ua_merge_update per rectangle), forward only: issued from Python, and as one HIP graph replay
    (device time without the host's launch cost), next to the single launch."""
    import torch
    from ultraattn_amd.executor import BlockSparseExecutor
    dev = "cuda:0"
    mask = workload_mask(name)
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda n: torch.randn(1, n * BLOCK, HEADS, 128, device=dev, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v = mk(mask.shape[0]), mk(mask.shape[1]), mk(mask.shape[1])
    ex = BlockSparseExecutor(mask, BLOCK, softmax_scale=SCALE)
    o1, l1 = ex.forward(q, k, v)
    o2, l2 = ex.forward_per_rectangle(q, k, v)
    torch.cuda.synchronize()
    fin = torch.isfinite(l1)
    res = {"workload": name, "rectangles": int((mask != 0).sum()),
           "max_abs_o_vs_single_launch": (o1.float() - o2.float()).abs().max().item(),
           "max_abs_lse_vs_single_launch": (l1[fin] - l2[fin]).abs().max().item()}

    def timed(fn, n):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / n
    res["single_launch_ms"] = timed(lambda: ex.forward(q, k, v, out=o1, lse=l1), 5)
    t0 = time.perf_counter()
    res["per_rectangle_eager_ms"] = timed(lambda: ex.forward_per_rectangle(q, k, v), 1)
    res["per_rectangle_eager_wall_ms"] = (time.perf_counter() - t0) * 1e3
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        ex.forward_per_rectangle(q, k, v)
    graph.replay()
    torch.cuda.synchronize()
    res["per_rectangle_graph_replay_ms"] = min(timed(graph.replay, 1) for _ in range(REPEATS))
    # without the folding, as the reference's harness runs it (its reduce() is a stub)
    res["per_rectangle_no_fold_ms"] = min(timed(lambda: ex.forward_per_rectangle(q, k, v, fold=False), 1) for _ in range(2))
    F = fwd_flops(mask)
    res["single_launch_tflops"] = F / res["single_launch_ms"] / 1e9
    res["per_rectangle_graph_tflops"] = F / res["per_rectangle_graph_replay_ms"] / 1e9
    res["speedup_vs_graph_replay"] = res["per_rectangle_graph_replay_ms"] / res["single_launch_ms"]
    res["speedup_vs_no_fold"] = res["per_rectangle_no_fold_ms"] / res["single_launch_ms"]
    return res


class PowerSampler:
    """Samples the socket power and the shader clock with `amd-smi metric -p -c` from a host thread
    while the GPU works (nothing is sampled inside the timed step loop of the benchmark)."""

    def __init__(self):
        import shutil
        self.exe = shutil.which("amd-smi")
        self.samples = []
        self._stop = False

    def _poll(self):
        import subprocess
        while not self._stop:
            try:
                out = subprocess.run([self.exe, "metric", "-p", "-c"], capture_output=True, text=True, timeout=5).stdout
            except Exception:
                break
            watts = mhz = None
            section = ""
            for line in out.splitlines():
                t = line.strip()
                if t.endswith(":"):
                    section = t
                if t.startswith("SOCKET_POWER:"):
                    watts = t.split()[1]
                if section.startswith("GFX_0") and t.startswith("CLK:"):
                    mhz = t.split()[1]
            try:
                self.samples.append((float(watts), float(mhz)))
            except (TypeError, ValueError):
                pass
            time.sleep(0.1)

    def measure(self, fn, seconds, sync):
        """Runs fn() repeatedly for `seconds`; returns median power / clock over the samples taken
        after the first third of the interval, or None without amd-smi."""
        import threading
        if not self.exe:
            return None
        self.samples, self._stop = [], False
        th = threading.Thread(target=self._poll)
        th.start()
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(3):
                fn()
            sync()
        self._stop = True
        th.join()
        keep = self.samples[len(self.samples) // 3:]
        if not keep:
            return None
        med = lambda xs: sorted(xs)[len(xs) // 2]
        return {"socket_power_w": med([w for w, _ in keep]), "gfx_clock_mhz": med([c for _, c in keep]), "samples": len(keep)}


def run_power(name):
    """Socket power and shader clock while each kernel of the workload runs back to back, next to a
    register-only MFMA loop and a plain copy: shows which kernels sit at the board's power limit."""
    import torch
    from ultraattn_amd import _lib, ops
    from ultraattn_amd.tilelist import build_tile_list
    dev = "cuda:0"
    sampler = PowerSampler()
    if not sampler.exe:
        return None
    mask = workload_mask(name)
    g = torch.Generator(device=dev).manual_seed(0)
    mk = lambda n: torch.randn(1, n * BLOCK, HEADS, 128, device=dev, dtype=torch.float32, generator=g).to(torch.bfloat16)
    q, k, v, do = mk(mask.shape[0]), mk(mask.shape[1]), mk(mask.shape[1]), mk(mask.shape[0])
    tl = build_tile_list(mask, BLOCK)
    o, lse = ops.bsa_fwd(q, k, v, tl, SCALE)
    delta = ops.softmax_delta(o, do)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    rnd = torch.randn(512 * 8, device=dev).to(torch.bfloat16)
    one = torch.ones(512 * 8, dtype=torch.bfloat16, device=dev)
    sink = torch.empty(512 * 256, dtype=torch.float32, device=dev)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    runs = {
        "forward": lambda: ops.bsa_fwd(q, k, v, tl, SCALE, out=o, lse=lse),
        "backward": lambda: ops.bsa_bwd(do, q, k, v, None, lse, tl, SCALE, dq=dq, dk=dk, dv=dv, softmax_d=delta),
        "mfma_random_operands": lambda: probe_lib().bench_probe_mfma(rnd.data_ptr(), sink.data_ptr(), 512, 20000, st),
        "mfma_constant_operands": lambda: probe_lib().bench_probe_mfma(one.data_ptr(), sink.data_ptr(), 512, 20000, st),
        "copy_1GiB": lambda: dst.copy_(src),
    }
    out = {"workload": name}
    for key, fn in runs.items():
        out[key] = sampler.measure(fn, 1.5, torch.cuda.synchronize)
    return out


def probe_mfma(peak):
    """Sustained register-only MFMA rates: constant and random operand bits; both dense bf16
    instructions (32x32x16 and 16x16x32) with operands that change on every instruction, at 1 and at
    2 waves per SIMD.  `measured_ceiling_tflops` = the best of the random-data figures: what the
    matrix pipes of this device deliver to any bf16 kernel fed with ordinary data."""
    import torch
    lib = probe_lib()
    dev = "cuda:0"
    out = torch.empty(512 * 256, dtype=torch.float32, device=dev)
    g = torch.Generator(device=dev).manual_seed(0)
    ops_ = {"constant": torch.ones(512 * 8, dtype=torch.bfloat16, device=dev),
            "random": torch.randn(512 * 8, dtype=torch.float32, device=dev, generator=g).to(torch.bfloat16)}
    res = {}
    st = torch.cuda.current_stream().cuda_stream
    rot = torch.randn(16 * 256 * 8, dtype=torch.float32, device=dev, generator=g).to(torch.bfloat16)
    # (key, entry point, operands, workgroups of 4 waves, iterations, flop per thread-iteration / 64 lanes)
    f32 = 4 * 32768.0          # 4 MFMAs of 32x32x16 per wave and iteration
    f16 = 8 * 16384.0          # 8 MFMAs of 16x16x32
    runs = [(name + "_operands_tflops", lib.bench_probe_mfma, t, 512, 40000, f32) for name, t in ops_.items()]
    runs += [("rotating_random_operands_tflops", lib.bench_probe_mfma_rotating, rot, 512, 40000, f32),
             ("rotating_random_1_wave_per_simd_tflops", lib.bench_probe_mfma_rotating, rot, 256, 80000, f32),
             ("rotating_random_16x16x32_tflops", lib.bench_probe_mfma16_rotating, rot, 512, 40000, f16),
             ("rotating_random_16x16x32_1_wave_per_simd_tflops", lib.bench_probe_mfma16_rotating, rot, 256, 80000, f16)]
    for key, fn, t, n_blocks, iters, flop in runs:
        assert fn(t.data_ptr(), out.data_ptr(), n_blocks, 2000, st) == 0
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        assert fn(t.data_ptr(), out.data_ptr(), n_blocks, iters, st) == 0
        e1.record()
        torch.cuda.synchronize()
        res[key] = n_blocks * 4 * iters * flop / e0.elapsed_time(e1) / 1e9
    res["frac_of_peak_random"] = res["random_operands_tflops"] / peak
    res["measured_ceiling_tflops"] = max(v for k, v in res.items() if "random" in k and k.endswith("_tflops"))
    res["measured_ceiling_frac_of_peak"] = res["measured_ceiling_tflops"] / peak
    res["note"] = ("register-only MFMA loops, 512 (2 waves per SIMD) or 256 (1 wave per SIMD) workgroups of 4 waves: one A/B "
                   "operand pair reused for ever (constant bits, random N(0,1) bits), and 8x8 random fragments cycled so that "
                   "the operands change on every instruction, for v_mfma_f32_32x32x16_bf16 and v_mfma_f32_16x16x32_bf16; the "
                   "clock follows power, power follows operand bit activity, so the best random figure is the practical "
                   "ceiling of any bf16 MFMA kernel on this device")
    return res


def run_grad_accumulate(steps):
    """One step of the gradient packs' fp32 accumulation at the 128k shape ([dK | dV] of one device:
    2 x 131072 x 32 x 128 elements): reads fp32 + bf16, writes fp32 + bf16 = 12 bytes per element."""
    import torch
    from ultraattn_amd import ops
    n = 2 * 131072 * HEADS * 128
    acc = torch.zeros(n, dtype=torch.float32, device="cuda:0")
    part = torch.empty(n, dtype=torch.bfloat16, device="cuda:0").normal_()
    out = torch.empty_like(part)
    ops.grad_accumulate(part, out, acc=acc)
    torch.cuda.synchronize()
    reps = []
    for _ in range(REPEATS):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            ops.grad_accumulate(part, out, acc=acc)
        e1.record()
        torch.cuda.synchronize()
        reps.append({"ms": e0.elapsed_time(e1) / steps})
    med, mn = median_min(reps)
    return {"ms": med["ms"], "ms_min": mn["ms"], "bytes": 12 * n, "gbps": 12 * n / med["ms"] / 1e6,
            "frac_of_hbm": 12 * n / med["ms"] / 1e6 / HBM_PEAK_GBPS,
            "shape": "acc fp32 += partial bf16, out bf16 = round(acc); 2 x 131072 x 32 x 128 elements"}


def device_ceilings(peak):
    """What the device delivers to the simplest possible kernels: register-only MFMA loops with their
    socket power and clock, L2 atomics and plain stores, streaming reads/writes.  These bound the
    attention and merge kernels; `python bench.py --device-ceilings` prints them alone."""
    import ctypes
    import torch
    lib = probe_lib()
    dev = "cuda:0"
    st = torch.cuda.current_stream().cuda_stream
    out = {"mfma": probe_mfma(peak)}
    sampler = PowerSampler()
    if sampler.exe:
        sink = torch.empty(512 * 256, dtype=torch.float32, device=dev)
        g = torch.Generator(device=dev).manual_seed(0)
        rot = torch.randn(16 * 256 * 8, dtype=torch.float32, device=dev, generator=g).to(torch.bfloat16)
        one = torch.ones(16 * 256 * 8, dtype=torch.bfloat16, device=dev)
        for key, fn, t in (("constant", lib.bench_probe_mfma, one), ("random", lib.bench_probe_mfma, rot),
                           ("rotating_random", lib.bench_probe_mfma_rotating, rot)):
            out["mfma"][key + "_power"] = sampler.measure(lambda: fn(t.data_ptr(), sink.data_ptr(), 512, 20000, st), 1.5,
                                                          torch.cuda.synchronize)
    atom = {}
    n_blocks, iters = 2048, 2048
    for mib in (8, 1024):
        buf = torch.zeros(mib << 18, dtype=torch.float32, device=dev)
        for mode, name, dwords in ((0, "f32_add", 1), (1, "u32_add", 1), (2, "f64_add", 2), (3, "dword_store", 1)):
            assert lib.bench_atomic_rate(buf.data_ptr(), buf.numel(), mode, n_blocks, 64, st) == 0
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            assert lib.bench_atomic_rate(buf.data_ptr(), buf.numel(), mode, n_blocks, iters, st) == 0
            e1.record()
            torch.cuda.synchronize()
            ops_ = n_blocks * 256 * iters
            ms = e0.elapsed_time(e1)
            atom[f"{name}_{mib}MiB"] = {"g_lane_ops_per_s": ops_ / ms / 1e6, "payload_gbps": ops_ * 4 * dwords / ms / 1e6}
        del buf
    out["l2_atomics"] = atom
    out["l2_atomics_note"] = ("2048 workgroups x 256 threads x 2048 operations, a wave instruction covers two 128-byte lines; "
                              "target region 8 MiB (stays in L2) and 1 GiB")
    n = 512 << 20
    srcs = [torch.empty(n, dtype=torch.uint8, device=dev) for _ in range(4)]
    dst = torch.empty(n, dtype=torch.uint8, device=dev)
    mix = {}
    for ns in (1, 2, 4):
        arr = (ctypes.c_void_p * ns)(*[t.data_ptr() for t in srcs[:ns]])
        blocks = n // (256 * 4 * 16)
        lib.bench_stream_mix(arr, ns, dst.data_ptr(), n, blocks, 1, st)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            lib.bench_stream_mix(arr, ns, dst.data_ptr(), n, blocks, 1, st)
        e1.record()
        torch.cuda.synchronize()
        mix[f"{ns}_read_1_write_gbps"] = (ns + 1) * n / (e0.elapsed_time(e1) / 10) / 1e6
    out["stream_mix"] = mix
    out["stream_mix_note"] = "512 MiB per stream, 16-byte non-temporal accesses, one load step per workgroup"
    del srcs, dst
    # instruction mix of the forward per 32 keys, registers and LDS only, zero data: what share of the time the bare
    # 16-MFMA loop takes
    sink = torch.empty(256 * 512, dtype=torch.float32, device=dev)
    names = ("16 MFMA", "16 MFMA + 40 fma + 16 exp2", "16 MFMA + 8 ds_read_b128 + 16 ds_read_b64_tr_b16",
             "16 MFMA + 40 fma + 16 exp2 + 8 ds_read_b128 + 16 ds_read_b64_tr_b16", "40 fma + 16 exp2", "8 ds_read_b128 + 16 ds_read_b64_tr_b16")
    issue = {}
    for wps in (1, 2):
        ms = []
        for mix in range(6):
            assert lib.bench_issue_mix(sink.data_ptr(), 256, wps, mix, 2000, st) == 0
            torch.cuda.synchronize()
            best = float("inf")
            for _ in range(3):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                assert lib.bench_issue_mix(sink.data_ptr(), 256, wps, mix, 20000, st) == 0
                e1.record()
                torch.cuda.synchronize()
                best = min(best, e0.elapsed_time(e1))
            ms.append(best)
        issue[f"{wps}_waves_per_simd"] = {n: {"ms": t, "rel_to_bare_mfma_loop": t / ms[0], "matrix_pipe_share": ms[0] / t if i < 4 else None}
                                           for i, (n, t) in enumerate(zip(names, ms))}
    out["issue_mix"] = issue
    out["issue_mix_note"] = ("256 workgroups (one per CU), 20000 iterations per wave, zero operands (the clock stays at its maximum); "
                             "matrix_pipe_share = time of the bare MFMA loop / time of the mix")
    return out


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline():
    """The reference's block-loop path restated on the CPU (oracle.block_loop_fwd), timed on
    config 1 exactly: B=1, S=8192, Nh=8, d=128, fp32, 16x16 causal block grid, forward only."""
    import torch
    from oracle import attn_oracle as ao
    from ultraattn_amd import masks
    mask = masks.config_causal(16)
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(1, 8192, 8, 128, generator=g, dtype=torch.float32) for _ in range(3))
    F = fwd_flops(mask, nh=8)
    times = []
    while len(times) < 4 or (sum(times) < 12.0 and len(times) < 200):     # 1 warm-up, then >= 3 runs, ~12 s of CPU work
        t0 = time.perf_counter()
        ao.block_loop_fwd(q, k, v, mask, BLOCK, SCALE)
        times.append(time.perf_counter() - t0)
        if sum(times) > 40:
            break
    timed = times[1:] or times
    best = min(timed)
    return {"value": F / best / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "config 1 whole: B=1 S=8192 Nh=8 d=128 fp32 causal 16x16 blocks of 512, forward, "
                      f"{len(timed)} runs, min {best:.3f} s, median {sorted(timed)[len(timed) // 2]:.3f} s",
            "affinity_cores": len(os.sched_getaffinity(0)), "cpu_model": cpu_model(), "flops": F,
            "parity": config1_parity(ao, mask, q, k, v)}


def config1_parity(ao, mask, q, k, v):
    """The HIP path against the CPU block loop on config 1's workload (the same bf16-rounded q, k, v
    and a seeded dO on both sides): largest deviations of O, LSE, dQ, dK, dV."""
    import torch
    from ultraattn_amd import ops
    from ultraattn_amd.tilelist import build_tile_list
    g = torch.Generator().manual_seed(1)
    do = torch.randn(q.shape, generator=g, dtype=torch.float32)
    qb, kb, vb, dob = (t.to(torch.bfloat16) for t in (q, k, v, do))
    ro, rl = ao.block_loop_fwd(qb, kb, vb, mask, BLOCK, SCALE)
    rq, rk, rv = ao.block_loop_bwd(dob, qb, kb, vb, ro, rl, mask, BLOCK, SCALE)
    tl = build_tile_list(mask, BLOCK)
    qd, kd, vd, dod = (t.to("cuda:0") for t in (qb, kb, vb, dob))
    o, lse = ops.bsa_fwd(qd, kd, vd, tl, SCALE)
    dq, dk, dv = ops.bsa_bwd(dod, qd, kd, vd, o, lse, tl, SCALE)
    torch.cuda.synchronize()
    err = lambda a, b: (a.detach().float().cpu() - b.float()).abs().max().item()
    lse_c, rl = lse.cpu().double(), rl.double()
    return {"workload": "config 1 (S=8192, Nh=8, 16x16 causal blocks), bf16-rounded inputs, against the CPU block loop",
            "o_max_abs": err(o, ro), "lse_max_rel": ((lse_c - rl).abs() / rl.abs().clamp_min(1.0)).max().item(),
            "dq_max_abs": err(dq, rq), "dk_max_abs": err(dk, rk), "dv_max_abs": err(dv, rv),
            "bounds": {"o_dq_dk_dv_max_abs": 2e-2, "lse_max_rel": 1e-3}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c3", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--no-extra", action="store_true", help="skip the other workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--device-ceilings", action="store_true",
                    help="print only the device's ceilings (MFMA loops, L2 atomics, streaming mixes) as one JSON line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (known size, for scaling rocprof byte counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the path: run it with --gpus 1 "
                 "(no multi-GPU figure exists for this build)")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs an MI355X (no CPU fallback for the kernels)")
    prop = torch.cuda.get_device_properties(0)
    clock_ghz = getattr(prop, "clock_rate", 2400000) / 1e6
    peak = prop.multi_processor_count * FLOP_PER_CLK_PER_CU * clock_ghz / 1e3      # TFLOP/s
    log(f"device {prop.name}: {prop.multi_processor_count} CUs @ {clock_ghz:.2f} GHz -> bf16 MFMA peak {peak:.1f} TFLOP/s")

    if a.device_ceilings:
        print(json.dumps(device_ceilings(peak)), flush=True)
        return
    if a.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    mfma_probe = probe_mfma(peak)
    MEASURED_MFMA_CEILING[0] = mfma_probe["measured_ceiling_tflops"]
    log(json.dumps(mfma_probe))
    if a.workload == "c5":
        main_res = run_c5(a.steps, a.warmup)
    else:
        main_res = run_attention(a.workload, a.steps, a.warmup, backward=a.workload in ("c3", "c4"))
    log(json.dumps(main_res))
    load_traffic()
    backward = "fwd_bwd_tflops" in main_res
    if backward:
        kt, kt_min = time_bwd_kernels(a.workload, max(3, a.steps // 2))
        F = main_res["fwd_flops"]
        main_res.update(dkdv_ms=kt["dkdv_ms"], dq_ms=kt["dq_ms"], dkdv_tflops=2.0 * F / kt["dkdv_ms"] / 1e9,
                        dq_tflops=0.5 * F / kt["dq_ms"] / 1e9)
        main_res["min"].update(kt_min)
        value = main_res["fwd_bwd_tflops"]
        metric = "effective TFLOP/s on active blocks, forward+backward"
    else:
        value = main_res.get("fwd_plus_merge_tflops", main_res["fwd_tflops"])
        metric = "effective TFLOP/s on active blocks, forward"
    value_best = value * main_res["ms_per_step"] / main_res["min"]["ms_per_step"]
    roofs = attention_roofs(a.workload, main_res, peak)
    # the dominant kernel of the step: dK/dV for the forward+backward workloads, the forward otherwise
    roof = dict(next(r for r in roofs if r["kernel"] == ("dkdv_kernel" if backward else "fwd_kernel")))

    extra = {}
    if not a.no_extra:
        for w in ("c3", "c4", "c2", "c5"):
            if w == a.workload:
                continue
            torch.cuda.empty_cache()
            r = run_c5(max(3, a.steps // 2), 2) if w == "c5" else \
                run_attention(w, max(3, a.steps // 2), 2, backward=w in ("c3", "c4"))
            if "fwd_bwd_tflops" in r:
                torch.cuda.empty_cache()
                kt, kt_min = time_bwd_kernels(w, 3)
                r.update(dkdv_ms=kt["dkdv_ms"], dq_ms=kt["dq_ms"])
                r["min"].update(kt_min)
            roofs += attention_roofs(w, r, peak)
            for key in ("tilelist_sha256", "fwd_flops", "repeats"):
                r.pop(key, None)
            r["fwd_frac_of_peak"] = r["fwd_tflops"] / peak
            if "fwd_bwd_tflops" in r:
                r["fwd_bwd_frac_of_peak"] = r["fwd_bwd_tflops"] / peak
            extra[w] = r
            log(json.dumps(r))
    out = {"metric": metric, "value": value, "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
           "repeats": REPEATS, "value_is": "median over the repeats of the timed block of `steps` steps", "value_best": value_best,
           "ms_per_step": main_res["ms_per_step"], "ms_per_step_min": main_res["min"]["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
           "dtype": "bf16", "data": "synthetic N(0,1) q/k/v/dO from a seeded device generator, random, no weights",
           "config": {"workload": {"c2": "causal 32k (config 2), forward", "c3": "strided 128k (config 3), forward+backward",
                                   "c4": "global+local 128k (config 4), forward+backward",
                                   "c5": "streaming shard 64k x 512k (config 5), 4 forward kernel tiles + merge"}[a.workload],
                      "seed": 0, "batch": 1, "heads": HEADS, "head_dim": 128, "block": BLOCK, "tile": 128,
                      "seq_q": int(workload_mask(a.workload).shape[0]) * BLOCK,
                      "seq_kv": int(workload_mask(a.workload).shape[1]) * BLOCK},
           "frac_of_bf16_mfma_peak": value / peak, "frac_of_measured_mfma_ceiling": value / MEASURED_MFMA_CEILING[0],
           "peak_tflops": peak, "detail": main_res,
           "fwd_frac_of_peak": main_res["fwd_tflops"] / peak, "roofline": roof, "rooflines": roofs, "extra": extra}
    if not a.no_extra:
        out["mask_builder"] = run_mask_builder(a.workload if a.workload != "c5" else "c3", 20)
        log(json.dumps(out["mask_builder"]))
        out["cols_gather"] = run_cols_gather(10)
        log(json.dumps(out["cols_gather"]))
        torch.cuda.empty_cache()
        out["grad_accumulate"] = run_grad_accumulate(10)
        log(json.dumps(out["grad_accumulate"]))
        out["dense_split"] = run_dense_split(20)
        log(json.dumps(out["dense_split"]))
        if a.workload in ("c3", "c4"):
            torch.cuda.empty_cache()
            out["per_rectangle_baseline"] = run_per_rectangle(a.workload)
            log(json.dumps(out["per_rectangle_baseline"]))
        if a.workload != "c5":
            torch.cuda.empty_cache()
            out["power"] = run_power(a.workload)
            log(json.dumps(out["power"]))
    out["mfma_probe"] = mfma_probe
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
        out["parity"] = out["cpu_baseline"]["parity"]          # the same object, at the top level too
        log(json.dumps(out["cpu_baseline"]))
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
