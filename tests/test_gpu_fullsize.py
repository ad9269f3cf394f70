"""The five benchmark workloads at their full sizes.  The CPU oracle handles these sizes in
seconds, so every workload is compared with it directly: integer structures bit for bit (raw ids
and the canonical sorted form), float outputs to 1e-4 relative / 1e-5 absolute.  Beside that,
size-independent properties: round trips and invariants of the integer structures, independence
of the convolution from the processing order and the staging path (bit-exact), one case that
reduces to a 1x1 layer, and - for the incremental sweep - equality with a full recompute every
tenth frame and at the end (bit-exact)."""
import ctypes

import numpy as np
import pytest
import torch

import parity
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


def test_workload2_grid_and_rulebooks_against_oracle(S, orc):
    """200k voxels on 1024^3 (+10 % repeated points): site ids, site coordinates, the 3^3 neighbour
    map, its list form and the stride-2 maps equal the oracle's bit for bit - raw (both number
    sites by first appearance) and after the canonical sort by (offset, in, out) over coordinates."""
    rng = np.random.default_rng(2)
    vox = scenes.planes_boxes_scene(seed=2, n=200000).astype(np.int32)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), 20000)]])
    pts = pts[rng.permutation(len(pts))]
    m = S.Metadata_3()
    out = torch.empty(0, device="cuda")
    f = torch.zeros((len(pts), 1), device="cuda")
    S.InputLayer_updateOutput(m, SZ, torch.from_numpy(pts.astype(np.int64)), f, out, 0, 4)
    sop, sc, cnt = orc.grid_build(pts)
    assert m.getNActive(SZ) == len(sc) == 200000
    assert np.array_equal(m.site_of_point.cpu().numpy(), sop)
    loc = m.getSpatialLocations(SZ).numpy()
    assert np.array_equal(loc, sc)
    # 3^3 rulebook: dense map and the reference's list form
    nbr_o, counts_o, pairs_o = orc.ssc_rules(sc)
    scale = m.ssc_rulebook(SZ)
    assert np.array_equal(scale.nbr.t[:scale.n].cpu().numpy(), nbr_o)
    counts, pairs = S.ssc_rulebook_lists(m, SZ)
    assert np.array_equal(counts.numpy(), counts_o)
    assert np.array_equal(pairs.numpy(), pairs_o)
    assert np.array_equal(orc.canonical_rules(counts.numpy(), pairs.numpy(), loc, loc),
                          orc.canonical_rules(counts_o, pairs_o, sc, sc))
    # stride-2 size-2 rulebook and the coarse grid
    parent_o, off_o, cc_o = orc.down2_rules(sc)
    fine, coarse, d = m.down_rulebook(SZ, SZ // 2)
    assert coarse.n == len(cc_o)
    assert np.array_equal(d.parent.t[:fine.n].cpu().numpy(), parent_o)
    assert np.array_equal(d.offset.t[:fine.n].cpu().numpy(), off_o)
    cloc = m.getSpatialLocations(SZ // 2).numpy()
    assert np.array_equal(cloc, cc_o)
    dcounts, dpairs = S.down_rulebook_lists(m, SZ, SZ // 2)
    dc_o, dp_o = orc.down2_pairs(parent_o, off_o)
    assert np.array_equal(dcounts.numpy(), dc_o)
    assert np.array_equal(orc.canonical_rules(dcounts.numpy(), dpairs.numpy(), loc, cloc),
                          orc.canonical_rules(dc_o, dp_o, sc, cc_o))


@pytest.mark.parametrize("C", [32, 64])
def test_workload3_layer_stack_against_oracle(S, orc, C):
    """500k voxels, 4 x [SubmanifoldConvolution(3) + BatchNormReLU] through the default dispatch (at
    this size: the filter-in-LDS kernel for C = 32, the shared-weights kernel for C = 64) against the
    oracle's convolution and batch norm, layer by layer and end to end, 1e-4 / 1e-5."""
    import sparseconvnet as scn

    vox = scenes.indoor_scene(seed=3, n=500000)
    g = torch.Generator().manual_seed(30 + C)
    f = torch.randn(len(vox), C, generator=g)
    x = scn.InputLayer(3, SZ, mode=4)([torch.from_numpy(vox.astype(np.int64)), f.cuda(), 1])
    _, sc, _ = orc.grid_build(vox)
    _, counts, pairs = orc.ssc_rules(sc)
    ref = f.numpy()  # one point per voxel, so the input layer hands the rows through in site order
    assert np.array_equal(x.features.cpu().numpy(), ref)
    torch.manual_seed(C)
    with torch.no_grad():
        for layer in range(4):
            conv = scn.SubmanifoldConvolution(3, C, C, 3, layer % 2 == 1).cuda()
            bn = scn.BatchNormReLU(C).cuda().eval()
            bn.running_mean.normal_(0, 1)
            bn.running_var.uniform_(0.5, 2.0)
            bn.weight.uniform_(0.5, 1.5)
            bn.bias.normal_(0, 0.1)
            if layer % 2 == 1:
                conv.bias.normal_(0, 0.5)
            y = conv(x)
            b = conv.bias.cpu().numpy() if layer % 2 == 1 else None
            # the layer on its own: oracle fed with the HIP path's input
            one, _ = orc.conv_forward(x.features.cpu().numpy(), conv.weight.cpu().numpy(), b, pairs, counts, len(sc))
            np.testing.assert_allclose(y.features.cpu().numpy(), one, rtol=1e-4, atol=1e-5)
            x = bn(y)
            # the stack end to end: oracle fed with its own previous output
            ref, _ = orc.conv_forward(ref, conv.weight.cpu().numpy(), b, pairs, counts, len(sc))
            ref = orc.bn_forward(ref, bn.running_mean.cpu().numpy(), bn.running_var.cpu().numpy(),
                                 bn.weight.cpu().numpy(), bn.bias.cpu().numpy(), bn.eps, 0.0)
            parity.check("workload 3, C=%d, end to end after layer %d" % (C, layer), x.features.cpu().numpy(), ref)


def test_workload4_full_unet_forward_against_oracle(orc):
    """The 150k-voxel scene (165k points) through the network executor and through the module tree,
    against the same module tree evaluated on the CPU oracle in fp32 and in double precision: every
    element within 1e-5 + 1e-4 * |reference| of both (nothing scaled by the tensor's maximum)."""
    import sparseconvnet as scn
    from oracle import oracle_net
    from workloads.netdefs import NaiveUNet

    pts, rgb, vox = scenes.unet_scene()
    model = NaiveUNet(m=32, levels=7, seed=4).cuda()
    net = scn.compile(model.sparseModel, capacity_sites=1 << 18)
    with torch.no_grad():
        x = [torch.from_numpy(pts.astype(np.int32)).cuda(), torch.from_numpy(rgb).cuda(), 1]
        feats = net(x, increment=False)
        feats_mod = model.sparseModel([torch.from_numpy(pts[:, :3].astype(np.int64)), x[1], 1])
    assert net.n_sites == len(vox) == 150000
    assert torch.equal(feats, feats_mod)
    ref = oracle_net.forward(model.sparseModel, [pts, rgb, 1])
    with orc.double_precision():
        ref64 = oracle_net.forward(model.sparseModel, [pts, rgb, 1])
    assert feats.shape == ref.shape == (len(pts), 32)
    parity.check("workload 4, full U-Net forward, 150k voxels", feats.cpu().numpy(), ref, ref64)


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


def test_workload5_sweep_equals_a_full_forward_every_tenth_frame(orc):
    """All 50 frames of the sweep through the executor; after every tenth frame and after the last
    one a second executor runs ONE full forward over every point seen so far, in arrival order: the
    features of all points must be equal bit for bit.  The final scene is also compared with the CPU
    oracle, and the phase timer must report a plausible frame."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    seq = scenes.sweep_sequence()
    model = NaiveUNet(m=32, levels=7, seed=4).cuda()
    net = scn.compile(model.sparseModel, capacity_sites=1 << 18)
    dev = lambda p, c: [torch.from_numpy(p.astype(np.int32)).cuda(), torch.from_numpy(c).cuda(), 1]
    with torch.no_grad():
        net(dev(*seq[0]), increment=False)
        net.profile(True)
        ref_net = scn.compile(model.sparseModel, capacity_sites=1 << 18)
        for f in range(1, len(seq)):
            out = net(dev(*seq[f]), increment=True, all_points=True)
            if f % 10 == 0 or f == len(seq) - 1:
                allp = np.concatenate([p for p, _ in seq[:f + 1]])
                allc = np.concatenate([c for _, c in seq[:f + 1]])
                ref = ref_net(dev(allp, allc), increment=False)
                assert net.n_sites == ref_net.n_sites
                assert out.shape == ref.shape == (len(allp), 32)
                assert torch.equal(out, ref), "frame %d: max |incremental - full| = %.3e" % (
                    f, (out - ref).abs().max().item())
        phases = net.profile(False)
    assert net.n_sites == ref_net.n_sites == 150000
    from oracle import oracle_net

    oref = oracle_net.forward(model.sparseModel, [allp, allc, 1])
    with orc.double_precision():
        oref64 = oracle_net.forward(model.sparseModel, [allp, allc, 1])
    parity.check("workload 5, last frame of the sweep, 150k voxels", out.cpu().numpy(), oref, oref64)
    assert set(phases) == {"structure", "dirty", "layers", "output"}
    assert 0.5 < sum(phases.values()) < 50.0


@pytest.mark.parametrize("old_from", ["scene", "frontier"])
def test_target_frame_5k_new_voxels_on_a_150k_scene(orc, old_from):
    """The frame the latency target is stated on (one full pass, then ONE frame with increment=True, as
    in the reference's demo.py:26-38): full forward over the first 145 000 voxels of the room in sweep
    order, then an incremental frame of exactly 5 000 new voxels plus 1 500 re-observed ones.  The
    incremental result must equal a full recompute over all points bit for bit - through the executor
    and through the module tree fed with CPU int64 coordinates as the reference's callers pass them -
    and match the CPU oracle (fp32 and double precision) per element."""
    import sparseconvnet as scn
    from oracle import oracle_net
    from workloads.netdefs import NaiveUNet

    (p0, c0), (p1, c1) = scenes.target_frame(old_from=old_from)
    assert len(p0) == 145000 and len(p1) == 6500
    model = NaiveUNet(m=32, levels=7, seed=4).cuda()
    net = scn.compile(model.sparseModel, capacity_sites=1 << 18)
    ref_net = scn.compile(model.sparseModel, capacity_sites=1 << 18)
    dev = lambda p, c: [torch.from_numpy(p.astype(np.int32)).cuda(), torch.from_numpy(c).cuda(), 1]
    ref_cpu = lambda p, c: [torch.from_numpy(p[:, :3].astype(np.int64)), torch.from_numpy(c).cuda(), 1]
    allp, allc = np.concatenate([p0, p1]), np.concatenate([c0, c1])
    with torch.no_grad():
        net(dev(p0, c0), increment=False)
        assert net.n_sites == 145000
        out = net(dev(p1, c1), increment=True, all_points=True)
        assert net.n_sites == 150000
        full = ref_net(dev(allp, allc), increment=False)
        assert torch.equal(out, full), "max |incremental - full| = %.3e" % (out - full).abs().max().item()
        # the same two calls through the reference's own entry: the module tree, CPU int64 coordinates
        model.sparseModel(ref_cpu(p0, c0))
        for m in model.modules():
            if isinstance(m, scn.OutputLayer):
                m.all_points = True
        out_mod = model.sparseModel(ref_cpu(p1, c1), increment=True)
    assert torch.equal(out_mod, full)
    oref = oracle_net.forward(model.sparseModel, [allp, allc, 1])
    with orc.double_precision():
        oref64 = oracle_net.forward(model.sparseModel, [allp, allc, 1])
    parity.check("target frame (5k new + 1.5k re-observed from the %s on 145k voxels)" % old_from, out.cpu().numpy(),
                 oref, oref64)
