"""Properties at the full sizes of the benchmark workloads, where the CPU oracle would take
minutes: round trips and invariants of the integer structures (bit-exact), and for the
convolution independence of the processing order and of the staging path (bit-exact), plus one
case that reduces to a 1x1 layer.  The incremental U-Net sweep is compared with a full
recompute over all 50 frames' points at the end (bit-exact)."""
import ctypes

import numpy as np
import pytest
import torch

from workloads import scenes

pytestmark = pytest.mark.gpu
SZ = torch.LongTensor([4096, 4096, 4096])
I64 = ctypes.c_int64


@pytest.fixture(scope="module")
def S():
    from sparseconvnet import SCN
    from sparseconvnet._lib import ensure_init

    ensure_init(0)
    return SCN


def test_workload2_grid_and_rulebooks_invariants(S):
    """200k voxels on 1024^3 (+10 % repeated points): insert/query round trip, symmetry of the
    3^3 map, consistency of the stride-2 maps."""
    from sparseconvnet._lib import lib, ptr, stream_ptr

    rng = np.random.default_rng(2)
    vox = scenes.planes_boxes_scene(seed=2, n=200000).astype(np.int32)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), 20000)]])
    pts = pts[rng.permutation(len(pts))]
    c4 = torch.from_numpy(np.ascontiguousarray(pts[:, :4])).cuda()
    P = len(pts)
    grid, coarse = ctypes.c_void_p(), ctypes.c_void_p()
    lib.insc_grid_create(I64(300000), ctypes.byref(grid))
    lib.insc_grid_create(I64(300000), ctypes.byref(coarse))
    sop = torch.empty(P, dtype=torch.int32, device="cuda")
    n = I64(0)
    lib.insc_grid_insert(grid, ptr(c4), I64(P), ptr(sop), ctypes.byref(n), stream_ptr())
    N = n.value
    assert N == 200000
    # every point maps to a site that carries its coordinates; ids follow first appearance
    coords = torch.empty((N, 4), dtype=torch.int32, device="cuda")
    src = ctypes.c_void_p(lib.insc_grid_coords(grid))
    torch.cuda.synchronize()
    hip = ctypes.CDLL("libamdhip64.so")
    assert hip.hipMemcpy(ctypes.c_void_p(coords.data_ptr()), src, ctypes.c_size_t(N * 16), 3) == 0
    assert torch.equal(coords[sop.long()], c4)
    first = np.unique(np.ascontiguousarray(pts[:, :4]).view([("", np.int32)] * 4), return_index=True)[1]
    assert np.array_equal(sop.cpu().numpy()[np.sort(first)], np.arange(N))
    q = torch.empty(P, dtype=torch.int32, device="cuda")
    lib.insc_grid_query(grid, ptr(c4), I64(P), ptr(q), stream_ptr())
    assert torch.equal(q, sop)
    # 3^3 map: centre is the site itself; j = nbr[i][k]  <=>  i = nbr[j][26-k]; coordinates differ by the offset
    nbr = torch.empty((N, 27), dtype=torch.int32, device="cuda")
    lib.insc_rulebook_ssc3(grid, I64(0), I64(N), ptr(nbr), 0, stream_ptr())
    ar = torch.arange(N, device="cuda", dtype=torch.int32)
    assert torch.equal(nbr[:, 13], ar)
    for k in (0, 5, 12, 14, 22, 26):
        j = nbr[:, k].long()
        ok = j >= 0
        assert torch.equal(nbr[j[ok], 26 - k], ar[ok])
        d = torch.tensor([k // 9 - 1, (k // 3) % 3 - 1, k % 3 - 1, 0], dtype=torch.int32, device="cuda")
        assert torch.equal(coords[j[ok]], coords[ok] + d)
    assert 8.0 < (nbr >= 0).sum().item() / N < 14.0
    # stride 2: parent coordinates = coordinates >> 1, offset = parity bits, child map inverts parent/offset
    parent = torch.empty(N, dtype=torch.int32, device="cuda")
    offset = torch.empty(N, dtype=torch.int32, device="cuda")
    child = torch.full((300000, 8), -1, dtype=torch.int32, device="cuda")
    lib.insc_rulebook_down2(grid, coarse, I64(0), I64(N), ptr(parent), ptr(offset), ptr(child), I64(300000), stream_ptr())
    nc = I64(0)
    lib.insc_grid_size(coarse, ctypes.byref(nc), stream_ptr())
    Nc = nc.value
    ccoords = torch.empty((Nc, 4), dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    assert hip.hipMemcpy(ctypes.c_void_p(ccoords.data_ptr()), ctypes.c_void_p(lib.insc_grid_coords(coarse)),
                         ctypes.c_size_t(Nc * 16), 3) == 0
    half = coords.clone()
    half[:, :3] >>= 1
    assert torch.equal(ccoords[parent.long()], half)
    assert torch.equal(offset, (coords[:, 0] & 1) * 4 + (coords[:, 1] & 1) * 2 + (coords[:, 2] & 1))
    assert torch.equal(child[parent.long(), offset.long()], ar)
    assert (child[:Nc] >= 0).sum().item() == N and (child[Nc:] >= 0).sum().item() == 0
    lib.insc_grid_destroy(grid)
    lib.insc_grid_destroy(coarse)


@pytest.mark.parametrize("C", [32, 64])
def test_workload3_convolution_is_independent_of_order_and_staging(S, C):
    """500k voxels: the planned path over the sorted order, the site-indexed path over the sorted
    order and over a random order give the same bits; a filter with only its centre tap equals
    the 1x1 layer."""
    import sparseconvnet as scn

    vox = scenes.indoor_scene(seed=3, n=500000)
    g = torch.Generator().manual_seed(3)
    f = torch.randn(len(vox), C, generator=g).cuda()
    x = scn.InputLayer(3, SZ, mode=4)([torch.from_numpy(vox.astype(np.int64)), f, 1])
    m = x.metadata
    sc = m.ssc_rulebook(SZ)
    W = (torch.randn(27, C, C, generator=g) * (2.0 / C / 27) ** 0.5).cuda()
    a = torch.empty(sc.n, C, device="cuda")
    b = torch.full((sc.n, C), 7.0, device="cuda")
    c = torch.full((sc.n, C), -7.0, device="cuda")
    S.ssc_rows_planned(x.features, a, W, None, sc, m.ssc_plan(sc))
    S.conv_rows(x.features, b, W, None, sc.nbr.t, 27, sc.order.t, None, sc.n)
    perm = torch.randperm(sc.n, generator=g).to(torch.int32).cuda()
    S.conv_rows(x.features, c, W, None, sc.nbr.t, 27, perm, None, sc.n)
    assert torch.equal(a, b)
    assert torch.equal(a, c)
    assert torch.isfinite(a).all() and a.abs().mean().item() > 0.1
    Wc = torch.zeros_like(W)
    Wc[13] = W[13]
    S.ssc_rows_planned(x.features, a, Wc, None, sc, m.ssc_plan(sc))
    S.NetworkInNetwork_updateOutput(x.features, b, W[13].contiguous(), torch.Tensor())
    torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-6)


def test_workload5_sweep_ends_equal_to_a_full_forward():
    """All 50 frames of the sweep through the executor, then a second executor runs ONE full
    forward over every point in arrival order: the features of all points must be equal bit for
    bit, and the phase timer must report a plausible frame."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    seq = scenes.sweep_sequence()
    model = NaiveUNet(m=32, levels=7, seed=4).cuda()
    net = scn.compile(model.sparseModel, capacity_sites=1 << 18)
    dev = lambda p, c: [torch.from_numpy(p.astype(np.int32)).cuda(), torch.from_numpy(c).cuda(), 1]
    with torch.no_grad():
        net(dev(*seq[0]), increment=False)
        net.profile(True)
        for p, c in seq[1:]:
            out = net(dev(p, c), increment=True, all_points=True)
        phases = net.profile(False)
        ref_net = scn.compile(model.sparseModel, capacity_sites=1 << 18)
        allp = np.concatenate([p for p, _ in seq])
        allc = np.concatenate([c for _, c in seq])
        ref = ref_net(dev(allp, allc), increment=False)
    assert net.n_sites == ref_net.n_sites == 150000
    assert out.shape == ref.shape == (len(allp), 32)
    assert torch.equal(out, ref)
    assert set(phases) == {"structure", "dirty", "layers", "output"}
    assert 0.5 < sum(phases.values()) < 50.0
