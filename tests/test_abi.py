"""The C-ABI library loads and exports every symbol that include/ultraattn.h declares; argument
checks that need no GPU return the documented codes.  No GPU, no kernel launches."""
import ctypes
import os
import re

import numpy as np
import pytest

from ultraattn_amd import _lib
from ultraattn_amd.build import LIB_PATH

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "ultraattn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ua_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported(lib):
    names = declared_symbols()
    assert {"ua_bsa_fwd", "ua_bsa_bwd_dkdv", "ua_bsa_bwd_dq", "ua_bsa_bwd_delta", "ua_merge", "ua_merge_update",
            "ua_tilelist_build", "ua_tilelist_size", "ua_tilelist_build_device", "ua_strerror",
            "ua_version"} <= set(names)
    assert "ua_probe_mfma" not in names, "bench-only diagnostics stay out of the product ABI"
    raw = ctypes.CDLL(LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/ultraattn.h but not exported"
    assert sorted(_lib.SIGNATURES) == names, "python binding and header disagree"
    header = open(os.path.join(ROOT, "include", "ultraattn.h")).read()
    assert lib.ua_version() == int(re.search(r"#define UA_VERSION (\d+)", header).group(1)) >= 102


def test_argument_checks_without_gpu(lib):
    s = (ctypes.c_int64 * 3)(128 * 128, 128, 128)
    buf = np.zeros(64, np.uint8).ctypes.data // 16 * 16 + 16     # any aligned non-null address; never dereferenced
    # NULL q
    assert lib.ua_bsa_fwd(None, buf, buf, buf, buf, buf, buf, buf, buf, 1, 1, 1, 1, 1, 128, s, s, s, s, 0.1, None) == -1
    # head_dim != 128
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, buf, buf, buf, 1, 1, 1, 1, 1, 64, s, s, s, s, 0.1, None) == -3
    # non-positive scale
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, buf, buf, buf, 1, 1, 1, 1, 1, 128, s, s, s, s, 0.0, None) == -3
    # sizes
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, buf, buf, buf, 0, 1, 1, 1, 1, 128, s, s, s, s, 0.1, None) == -2
    # a non-empty list needs col_idx and flag; a negative nnz is a shape error
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, None, buf, buf, 1, 1, 1, 1, 1, 128, s, s, s, s, 0.1, None) == -1
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, buf, None, buf, 1, 1, 1, 1, 1, 128, s, s, s, s, 0.1, None) == -1
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, buf, buf, buf, 1, 1, 1, 1, -1, 128, s, s, s, s, 0.1, None) == -2
    # misaligned pointer / stride not a multiple of 8
    assert lib.ua_bsa_fwd(buf + 2, buf, buf, buf, buf, buf, buf, buf, buf, 1, 1, 1, 1, 1, 128, s, s, s, s, 0.1, None) == -4
    bad = (ctypes.c_int64 * 3)(128 * 128, 132, 128)
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, buf, buf, buf, 1, 1, 1, 1, 1, 128, bad, s, s, s, 0.1, None) == -4
    # merge: too many partials, bad seqlen
    arr = (ctypes.c_void_p * 17)(*([buf] * 17))
    assert lib.ua_merge(arr, arr, 17, buf, buf, 1, 16, 1, 128, None) == -3
    assert lib.ua_merge(arr, arr, 0, buf, buf, 1, 16, 1, 128, None) == -3
    assert lib.ua_merge(arr, arr, 2, buf, buf, 1, 0, 1, 128, None) == -2
    assert lib.ua_merge(None, arr, 2, buf, buf, 1, 16, 1, 128, None) == -1
    # backward
    assert lib.ua_bsa_bwd_delta(buf, None, buf, 1, 16, 1, 128, s, s, None) == -1
    assert lib.ua_bsa_bwd_delta(buf, buf, buf, 1, 16, 1, 96, s, s, None) == -3
    assert lib.ua_bsa_bwd_dq(buf, buf, buf, buf, buf, buf, None, buf, buf, buf, buf, 1, 1, 1, 1, 1, 128,
                             s, s, s, s, s, 0.1, None) in (-1, -7)
    # backward kernels: NULL index arrays with a non-empty list
    assert lib.ua_bsa_bwd_dq(buf, buf, buf, buf, buf, buf, buf, buf, None, buf, buf, 1, 1, 1, 1, 1, 128,
                             s, s, s, s, s, 0.1, None) == -1
    assert lib.ua_bsa_bwd_dkdv(buf, buf, buf, buf, buf, buf, buf, buf, buf, buf, None, buf, 1, 1, 1, 1, 1, 128,
                               s, s, s, s, s, s, 0.1, None) == -1
    # in-place update of a running (out, lse): NULL, head_dim, sizes, row alignment (fp32 rows: strides in multiples of 4)
    ls = (ctypes.c_int64 * 3)(16, 1, 16)
    ok = (buf, buf, buf, buf, buf, buf)
    assert lib.ua_merge_update(*ok[:5], None, 1, 16, 1, 128, 0, 0, 0, s, ls, s, ls, s, ls, None) == -1
    assert lib.ua_merge_update(*ok, 1, 16, 1, 64, 0, 0, 0, s, ls, s, ls, s, ls, None) == -3
    assert lib.ua_merge_update(*ok, 1, 0, 1, 128, 0, 0, 0, s, ls, s, ls, s, ls, None) == -2
    odd = (ctypes.c_int64 * 3)(128 * 128, 132, 128)          # bf16 rows need strides in multiples of 8
    assert lib.ua_merge_update(*ok, 1, 16, 1, 128, 0, 0, 0, odd, ls, s, ls, s, ls, None) == -4
    # the same pointer for out and new_out needs the same element type and strides
    s2 = (ctypes.c_int64 * 3)(128 * 256, 256, 128)
    assert lib.ua_merge_update(buf, buf, buf + 64, buf, buf, buf, 1, 16, 1, 128, 0, 0, 1, s, ls, s, ls, s, ls, None) == -2
    assert lib.ua_merge_update(buf, buf, buf + 64, buf, buf, buf, 1, 16, 1, 128, 0, 0, 0, s, ls, s, ls, s2, ls, None) == -2
    # flag arrays are read as aligned 32-bit words
    assert lib.ua_bsa_fwd(buf, buf, buf, buf, buf, buf, buf, buf + 1, buf, 1, 1, 1, 1, 1, 128, s, s, s, s, 0.1, None) == -4
    assert lib.ua_bsa_bwd_dq(buf, buf, buf, buf, buf, buf, buf, buf, buf, buf + 2, buf, 1, 1, 1, 1, 1, 128,
                             s, s, s, s, s, 0.1, None) == -4
    # gradient reductions
    assert lib.ua_grad_accumulate(buf, None, buf, 64, 0, None) == -1
    assert lib.ua_grad_accumulate(None, buf, None, 64, 0, None) == -1
    assert lib.ua_grad_accumulate(None, buf, buf, 64, 1, None) == -1      # init_from_out needs an accumulator
    assert lib.ua_grad_accumulate(buf, buf, buf, 0, 0, None) == -2
    assert lib.ua_grad_accumulate(buf, buf, buf, 60, 0, None) == -4
    assert lib.ua_grad_accumulate(buf, buf + 2, buf, 64, 0, None) == -4
    arr1 = (ctypes.c_void_p * 17)(*([buf] * 17))
    assert lib.ua_grad_sum(arr1, 17, 0, buf, 1, 16, 1, 128, s, 1.0, None) == -3
    assert lib.ua_grad_sum(arr1, 2, 0, buf, 1, 16, 1, 64, s, 1.0, None) == -3
    assert lib.ua_grad_sum(arr1, 2, 0, buf, 1, 0, 1, 128, s, 1.0, None) == -2
    assert lib.ua_grad_sum(None, 2, 0, buf, 1, 16, 1, 128, s, 1.0, None) == -1
    # device tile-list builders: NULL, sizes, and the no-allocation variant's limit on the number of lines
    args = (buf,) * 8
    assert lib.ua_tilelist_build_device(buf, 1, 1, 4, *args, None, None) == -1
    assert lib.ua_tilelist_build_device(buf, 0, 1, 4, *args, buf, None) == -2
    assert lib.ua_tilelist_build_device_noalloc(None, 1, 1, 4, *args, None, None) == -1
    assert lib.ua_tilelist_build_device_noalloc(buf, 16384, 16384, 4, *args, None, None) == -8
    assert lib.ua_tilelist_build_device_noalloc(buf, 8192, 8192, 4, *args, None, None) == -8    # 65536 lines > 65532
    # column-buffer layout changes: NULL, sizes, alignment, overlap
    assert lib.ua_cols_gather(None, buf, 2, 1, 1024, None) == -1
    assert lib.ua_cols_gather(buf, buf + (1 << 20), 0, 1, 1024, None) == -2
    assert lib.ua_cols_scatter(buf, buf + (1 << 20), 2, 1, 1020, None) == -4
    assert lib.ua_cols_scatter(buf, buf + 16, 2, 1, 1024, None) == -2                            # overlapping buffers
    for code in range(-8, 1):
        assert lib.ua_strerror(code) != b"unknown error code"
    assert lib.ua_strerror(-99) == b"unknown error code"


def test_dense_entry_points_without_gpu(lib):
    """Argument checks of ua_dense_fwd / ua_dense_bwd and the split policy behind
    ua_dense_workspace_bytes (pure host arithmetic): a launch that fills the device or a short walk
    never splits; else enough parts for ~2 workgroups per CU, at least two tiles each, at most 16."""
    s = (ctypes.c_int64 * 3)(128 * 128, 128, 128)
    buf = np.zeros(64, np.uint8).ctypes.data // 16 * 16 + 16
    assert lib.ua_dense_fwd(None, buf, buf, buf, buf, 1, 1, 128, 128, 128, s, s, s, s, 0.1, 0, None, 0, None) == -1
    assert lib.ua_dense_fwd(buf, buf, buf, buf, buf, 1, 1, 100, 128, 128, s, s, s, s, 0.1, 0, None, 0, None) == -2
    assert lib.ua_dense_fwd(buf, buf, buf, buf, buf, 1, 1, 128, 0, 128, s, s, s, s, 0.1, 0, None, 0, None) == -2
    assert lib.ua_dense_fwd(buf, buf, buf, buf, buf, 1, 1, 128, 128, 64, s, s, s, s, 0.1, 0, None, 0, None) == -3
    assert lib.ua_dense_fwd(buf + 2, buf, buf, buf, buf, 1, 1, 128, 128, 128, s, s, s, s, 0.1, 0, None, 0, None) == -4
    bwd = lambda *a: lib.ua_dense_bwd(*a, 1, 1, 128, 128, 128, s, s, s, s, s, s, s, 0.1, 1, None, 0, None)
    assert bwd(buf, buf, buf, buf, buf, buf, None, buf, buf) == -1
    assert bwd(buf, buf, buf, buf, None, buf, buf, buf, buf) == -1
    assert lib.ua_dense_bwd(buf, buf, buf, buf, buf, buf, buf, buf, buf, 1, 1, 128, 130, 128, s, s, s, s, s, s, s, 0.1, 1,
                            None, 0, None) == -2
    ws = lib.ua_dense_workspace_bytes
    assert ws(1, 32, 131072, 131072, 0) == 0 and ws(1, 32, 131072, 131072, 1) == 0       # 32768 workgroups
    assert ws(1, 1, 256, 256, 0) == 0                                                  # 2 x 2 tiles: walks too short
    assert ws(1, 1, 1000, 4096, 0) == 0 and ws(0, 1, 1024, 4096, 0) == 0                # nothing to size
    al = lambda x: (x + 255) // 256 * 256
    # Sq=1024, Skv=4096, one head: 8 query tiles, 32 key tiles -> min(16, ceil(512/8), 32/2) = 16 parts
    assert ws(1, 1, 1024, 4096, 0) == 16 * (al(1024 * 128 * 2) + al(1024 * 4))
    # backward: dQ 16 parts of fp32 [1024, 128]; dK, dV: 32 key tiles x 2 -> ceil(512/64) = 8, min(8, 16, 8/2) = 4 parts
    assert ws(1, 1, 1024, 4096, 1) == 16 * al(1024 * 128 * 4) + 4 * 2 * al(4096 * 128 * 4)
    # 32 heads x 8 query tiles = 256 workgroups < 384 -> ceil(512/256) = 2 parts
    assert ws(1, 32, 1024, 4096, 0) == 2 * (al(32 * 1024 * 128 * 2) + al(32 * 1024 * 4))
    assert ws(1, 32, 2048, 4096, 0) == 0                                               # 512 workgroups: full launch


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "ultraattn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith(".py"):
                src = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", src, flags=re.M), f
