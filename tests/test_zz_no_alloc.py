"""The entry point that allocates nothing (ua_tilelist_build_device_noalloc) against the
ordinary device builder, through the C ABI: two calls in a row, the second on a smaller mask."""
import ctypes

import numpy as np
import pytest
import torch

from ultraattn_amd import _lib, masks

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FIELDS = ("row_ptr", "col_idx", "flag", "col_ptr", "row_idx", "cflag", "q_order", "k_order")


def _buffers(nqt, nkt, nnz):
    i32 = dict(dtype=torch.int32, device=DEV)
    u8 = dict(dtype=torch.uint8, device=DEV)
    n = max(nnz, 1)
    # poisoned, so that an entry the builder failed to write shows up
    mk = lambda size, kw: torch.full((size,), 77, **kw)
    return dict(row_ptr=mk(nqt + 1, i32), col_idx=mk(n, i32), flag=mk(n, u8), col_ptr=mk(nkt + 1, i32),
                row_idx=mk(n, i32), cflag=mk(n, u8), q_order=mk(nqt, i32), k_order=mk(nkt, i32))


def _build(lib, mask, rate, noalloc):
    m = torch.from_numpy(mask).to(DEV)
    nqb, nkb = mask.shape
    nqt, nkt = nqb * rate, nkb * rate
    n1, n2, nnz = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
    sized = np.ascontiguousarray(np.where(mask > 2, 0, mask).astype(np.uint8))     # the host side rejects other values
    assert lib.ua_tilelist_size(sized.ctypes.data, nqb, nkb, rate, ctypes.byref(n1), ctypes.byref(n2), ctypes.byref(nnz)) == 0
    out = _buffers(nqt, nkt, nnz.value)
    st = torch.cuda.current_stream().cuda_stream
    ptrs = [out[f].data_ptr() for f in FIELDS]
    if noalloc:
        bad = torch.full((1,), -1, dtype=torch.int32, device=DEV)
        rc = lib.ua_tilelist_build_device_noalloc(m.data_ptr(), nqb, nkb, rate, *ptrs, bad.data_ptr(), st)
    else:
        work = torch.empty(nqt + nkt + 7, dtype=torch.int32, device=DEV)
        rc = lib.ua_tilelist_build_device(m.data_ptr(), nqb, nkb, rate, *ptrs, work.data_ptr(), st)
        bad = work[nqt + nkt + 2:nqt + nkt + 3]
    assert rc == 0, lib.ua_strerror(rc)
    torch.cuda.synchronize()
    return {f: out[f][:nnz.value].cpu().numpy() if f in ("col_idx", "flag", "row_idx", "cflag") else out[f].cpu().numpy()
            for f in FIELDS}, int(bad.item())


def test_noalloc_builder_equals_the_builder_with_caller_scratch(lib):
    big = masks.config_streaming_shard()                         # 128 x 1024 blocks: 512 + 4096 tile lines
    small = np.random.RandomState(4).randint(0, 3, size=(5, 7)).astype(np.uint8)
    for mask, rate in ((big, 4), (small, 3), (masks.config_strided(), 4), (np.zeros((2, 2), np.uint8), 1)):
        want, bad_w = _build(lib, mask, rate, noalloc=False)
        got, bad_g = _build(lib, mask, rate, noalloc=True)
        assert bad_w == bad_g == 0
        for f in FIELDS:
            assert got[f].dtype == want[f].dtype and np.array_equal(got[f], want[f]), (mask.shape, f)
    # an entry that is no Block_Type is counted (and treated as EMPTY) by both
    odd = small.copy()
    odd[1, 2] = 9
    want, bad_w = _build(lib, odd, 2, noalloc=False)
    got, bad_g = _build(lib, odd, 2, noalloc=True)
    assert bad_w == bad_g == 1 and all(np.array_equal(got[f], want[f]) for f in FIELDS)


def test_noalloc_builder_rejects_what_its_scratch_cannot_hold(lib):
    m = torch.zeros(8, dtype=torch.uint8, device=DEV)
    p = m.data_ptr()
    st = torch.cuda.current_stream().cuda_stream
    # 40000 + 40000 tile lines > UA_NOALLOC_MAX_LINES: refused before anything is launched
    rc = lib.ua_tilelist_build_device_noalloc(p, 10000, 10000, 4, p, p, p, p, p, p, p, p, None, st)
    assert rc == -8 and b"scratch" in lib.ua_strerror(rc)
    assert lib.ua_tilelist_build_device_noalloc(p, 1, 1, 1, p, p, p, p, p, p, p, None, None, st) == -1


def test_noalloc_builder_leaves_device_memory_alone_and_runs_under_capture(lib):
    """The second and later calls must not change the device's free memory, and after ua_init()
    (which resolves the per-device lookups outside capture) a call can be captured into a HIP
    graph: every replay rebuilds the lists of whatever mask is in the input buffer."""
    assert lib.ua_init() == 0 and lib.ua_init() == 0              # idempotent
    a = masks.config_strided(16, 2, 4)
    b = masks.config_global_local(16, 2, 1)
    rate = 2
    nqt = nkt = 16 * rate
    cap = nqt * nkt
    m = torch.from_numpy(a).to(DEV)
    out = _buffers(nqt, nkt, cap)
    bad = torch.zeros(1, dtype=torch.int32, device=DEV)
    ptrs = [out[f].data_ptr() for f in FIELDS]
    side = torch.cuda.Stream()
    call = lambda st: lib.ua_tilelist_build_device_noalloc(m.data_ptr(), 16, 16, rate, *ptrs, bad.data_ptr(), st)
    with torch.cuda.stream(side):
        assert call(side.cuda_stream) == 0                        # warm, eager
    torch.cuda.synchronize()
    unchanged = []
    for _ in range(2):      # the runtime may grow its own pools once, on any launch: two rounds, one must be exact
        free0 = torch.cuda.mem_get_info()[0]
        alloc0 = torch.cuda.memory_allocated()
        with torch.cuda.stream(side):
            for _ in range(3):
                assert call(side.cuda_stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == alloc0
        unchanged.append(torch.cuda.mem_get_info()[0] == free0)
    assert any(unchanged)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert call(torch.cuda.current_stream().cuda_stream) == 0
    for mask in (b, a, b):
        m.copy_(torch.from_numpy(mask))
        for f in FIELDS:
            out[f].fill_(77)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want, _ = _build(lib, mask, rate, noalloc=False)
        nnz = want["col_idx"].shape[0]
        for f in FIELDS:
            got = out[f].cpu().numpy()
            got = got[:nnz] if f in ("col_idx", "flag", "row_idx", "cflag") else got
            assert np.array_equal(got, want[f]), f
        assert int(bad.item()) == 0
