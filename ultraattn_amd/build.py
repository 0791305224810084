"""Build step: compile the HIP sources in ``csrc/`` for gfx950 into ``libultraattn_hip.so``
next to this file.  Run ``python -m ultraattn_amd.build`` (hipcc cross-compiles without a GPU).
"""
import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libultraattn_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)
SOURCES = ["api.hip", "tilelist.hip", "merge.hip", "glue.hip", "reduce.hip", "fwd.hip", "bwd.hip"]
# benchmark-only probes (register-only MFMA loop, streaming-mix ceiling): built beside bench.py,
# never linked into the product library
BENCH_SRC = os.path.join(os.path.dirname(PKG_DIR), "bench_probe.hip")
BENCH_LIB_PATH = os.path.join(os.path.dirname(PKG_DIR), "libbench_probe.so")
# -packed-fp32-ops: keep the compiler from forming v_pk_{add,mul,fma}_f32 out of scalar code.
HIPCC_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-result",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def build_library(verbose: bool = False, jobs: int = 4) -> str:
    """Compile every source and link the shared library; returns its path."""
    objdir = os.path.join(PKG_DIR, "build")
    os.makedirs(objdir, exist_ok=True)
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc_path(), *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, obj, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        while sum(p.poll() is None for _, _, p in procs) >= jobs:
            for _, _, p in procs:
                if p.poll() is None:
                    p.wait()
                    break
    objs = []
    for src, obj, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
        if verbose and out.strip():
            print(out)
        objs.append(obj)
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}")
    return LIB_PATH


def build_bench_probe(verbose: bool = False) -> str:
    """Compile bench_probe.hip into libbench_probe.so at the repository root (used by bench.py only)."""
    cmd = [hipcc_path(), *HIPCC_FLAGS, "-shared", BENCH_SRC, "-o", BENCH_LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on bench_probe.hip:\n{r.stdout}")
    return BENCH_LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose="-v" in sys.argv))
    if os.path.exists(BENCH_SRC):
        print(build_bench_probe(verbose="-v" in sys.argv))
