"""insc_grid_insert_noalloc, the insert for callers that cannot allocate device memory, against
insc_grid_insert through the C ABI: same site of every row, same site count, same coordinate
table (bit for bit), on two calls in a row - the second with fewer rows, so that stale scratch
entries of the first call lie behind the ones in use - and no device memory taken by the calls."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
I64 = ctypes.c_int64


def _coords(n, seed, side):
    rng = np.random.default_rng(seed)
    c = rng.integers(0, side, (n, 4)).astype(np.int32)
    c[:, 3] = rng.integers(0, 2, n)
    return c


def _table(lib, g, n):
    out = torch.empty((n, 4), dtype=torch.int32, device="cuda")
    hip = ctypes.CDLL("libamdhip64.so")
    torch.cuda.synchronize()
    assert hip.hipMemcpy(ctypes.c_void_p(out.data_ptr()), ctypes.c_void_p(lib.insc_grid_coords(g)),
                         ctypes.c_size_t(n * 16), 3) == 0
    return out


def test_insert_without_allocation_equals_insert():
    from sparseconvnet._lib import InscError, ensure_init, lib, ptr, stream_ptr

    ensure_init(0)
    st = stream_ptr()
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    lib.insc_grid_create(I64(40000), ctypes.byref(a))
    lib.insc_grid_create(I64(40000), ctypes.byref(b))
    # first call: the largest list one call takes, with many repeated voxels; second call: a short
    # list that repeats voxels of the first and adds new ones
    first = _coords(16384, 1, 24)
    second = np.concatenate([first[100:400], _coords(700, 2, 40)])[np.random.default_rng(3).permutation(1000)]
    n_a, n_b = I64(0), I64(0)
    for pts in (first, second):
        c = torch.from_numpy(np.ascontiguousarray(pts)).cuda()
        sa = torch.full((len(pts),), -9, dtype=torch.int32, device="cuda")
        sb = torch.full((len(pts),), -7, dtype=torch.int32, device="cuda")
        lib.insc_grid_insert(a, ptr(c), I64(len(pts)), ptr(sa), ctypes.byref(n_a), st)
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        lib.insc_grid_insert_noalloc(b, ptr(c), I64(len(pts)), ptr(sb), ctypes.byref(n_b), st)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0, "the call took or released device memory"
        assert n_a.value == n_b.value
        assert torch.equal(sa, sb)
        assert torch.equal(_table(lib, a, n_a.value), _table(lib, b, n_b.value))
        # and both agree with numbering by first appearance
    allp = np.concatenate([first, second])
    _, idx = np.unique(allp.view([("", np.int32)] * 4), return_index=True)
    assert n_b.value == len(idx)
    assert np.array_equal(_table(lib, b, n_b.value).cpu().numpy(), allp[np.sort(idx)])
    # without the count read-back the call only enqueues work; the result is the same
    third = _coords(500, 4, 60)
    c = torch.from_numpy(third).cuda()
    sa = torch.empty(500, dtype=torch.int32, device="cuda")
    sb = torch.empty(500, dtype=torch.int32, device="cuda")
    lib.insc_grid_insert(a, ptr(c), I64(500), ptr(sa), None, st)
    lib.insc_grid_insert_noalloc(b, ptr(c), I64(500), ptr(sb), None, st)
    lib.insc_grid_size(a, ctypes.byref(n_a), st)
    lib.insc_grid_size(b, ctypes.byref(n_b), st)
    assert n_a.value == n_b.value and torch.equal(sa, sb)
    q = torch.empty(500, dtype=torch.int32, device="cuda")
    lib.insc_grid_query(b, ptr(c), I64(500), ptr(q), st)
    assert torch.equal(q, sb)
    # limits: more rows than one call takes; a list that may not fit the capacity
    big = torch.zeros((16385, 4), dtype=torch.int32, device="cuda")
    sbig = torch.empty(16385, dtype=torch.int32, device="cuda")
    with pytest.raises(InscError) as e:
        lib.insc_grid_insert_noalloc(b, ptr(big), I64(16385), ptr(sbig), None, st)
    assert e.value.code == -3 and "16384" in str(e.value)
    small = ctypes.c_void_p()
    lib.insc_grid_create(I64(1024), ctypes.byref(small))
    with pytest.raises(InscError) as e:
        lib.insc_grid_insert_noalloc(small, ptr(big), I64(2000), ptr(sbig), None, st)
    assert e.value.code == -3 and "insc_grid_reserve" in str(e.value)
    lib.insc_grid_insert_noalloc(b, None, I64(0), None, ctypes.byref(n_b), st)  # an empty list is fine
    assert n_b.value == n_a.value
    for g in (a, b, small):
        lib.insc_grid_destroy(g)
