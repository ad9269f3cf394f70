"""GPU parity of the feature kernels against the CPU oracle, called through the reference's
op names (sparseconvnet.SCN.*_updateOutput).  Tolerance: 1e-4 relative / 1e-5 absolute, the
bound the north star states for float32 outputs."""
import numpy as np
import pytest
import torch

from workloads import scenes

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5
SZ = torch.LongTensor([4096, 4096, 4096])


@pytest.fixture(scope="module")
def S():
    from sparseconvnet import SCN
    from sparseconvnet._lib import ensure_init

    ensure_init(0)
    return SCN


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def setup_sites(S, pts, C, seed=0, mode=4):
    rng = np.random.default_rng(seed)
    f = rng.normal(size=(len(pts), C)).astype(np.float32)
    m = S.Metadata_3()
    out = torch.empty(0, device="cuda")
    S.InputLayer_updateOutput(m, SZ, torch.from_numpy(pts.astype(np.int64)), cu(f), out, 0, mode)
    return m, f, out


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
def test_input_output_layers(S, orc, mode):
    rng = np.random.default_rng(1)
    if mode == 0:
        pts = scenes.boxes_scene(seed=4, n=5000)
    else:
        pts = np.concatenate([rng.integers(50, 62, (8000, 3)), np.zeros((8000, 1), np.int64)], 1).astype(np.int32)
    m, f, out = setup_sites(S, pts, 3, seed=2, mode=mode)
    sop, sc, cnt = orc.grid_build(pts)
    if mode in (0, 3, 4):
        ref = orc.input_forward(f, sop, cnt, mode=mode)
    else:  # keep first (1) / last (2) row of each site, per Metadata/IOLayersRules.h:104-115
        idx = np.zeros(len(sc), np.int64)
        if mode == 1:
            idx[sop[::-1]] = np.arange(len(pts))[::-1]
        else:
            idx[sop] = np.arange(len(pts))
        ref = f[idx]
    assert out.shape == ref.shape
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)
    o = torch.empty(0, device="cuda")
    S.OutputLayer_updateOutput(m, out, o)
    assert (o.cpu().numpy() == out.cpu().numpy()[sop]).all()
    assert (o.cpu().numpy() == orc.output_forward(out.cpu().numpy(), sop)).all()


@pytest.mark.parametrize("Cin,Cout,bias", [(16, 16, False), (32, 32, True), (64, 64, False), (3, 32, False),
                                            (64, 32, True), (96, 96, False), (32, 20, True), (48, 224, False),
                                            (384, 192, False), (5, 7, True), (32, 288, False)])
def test_submanifold_convolution(S, orc, Cin, Cout, bias):
    pts = scenes.boxes_scene(seed=1, n=20000 if Cin * Cout <= 4096 else 6000)
    m, x, feats = setup_sites(S, pts, Cin, seed=Cin)
    rng = np.random.default_rng(Cout)
    W = (rng.normal(size=(27, Cin, Cout)) * (2.0 / Cin / 27) ** 0.5).astype(np.float32)
    b = rng.normal(size=Cout).astype(np.float32) if bias else None
    out = torch.empty(0, device="cuda")
    flops = S.SubmanifoldConvolution_updateOutput(SZ, torch.LongTensor([3, 3, 3]), m, feats, out, cu(W),
                                                  cu(b) if bias else torch.Tensor(), 1)
    _, sc, _ = orc.grid_build(pts)
    _, counts, pairs = orc.ssc_rules(sc)
    ref, rflops = orc.conv_forward(feats.cpu().numpy(), W, b, pairs, counts, len(sc))
    assert flops == rflops
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("Cin,Cout,bias", [(64, 64, False), (64, 32, True), (96, 96, False), (80, 48, True),
                                            (112, 100, False)])
def test_persistent_kernels_give_the_bits_of_the_per_tile_kernel(S, orc, Cin, Cout, bias):
    """Wide 3^3 layers (64..127 input channels) have three kernels: one block per (tile, output
    block), persistent blocks that walk a cost-ordered tile schedule, and persistent blocks of four
    tiles that share the weight tiles through LDS.  They must agree bit for bit (an incremental frame
    and a full frame may take different ones), and with the oracle to the float tolerance."""
    from sparseconvnet._lib import lib

    pts = scenes.boxes_scene(seed=5, n=7000)
    m, x, feats = setup_sites(S, pts, Cin, seed=Cin + 1)
    sc = m.ssc_rulebook(SZ)
    rng = np.random.default_rng(Cout + 3)
    W = cu((rng.normal(size=(27, Cin, Cout)) * (2.0 / Cin / 27) ** 0.5).astype(np.float32))
    b = rng.normal(size=Cout).astype(np.float32) if bias else None
    bt = cu(b) if bias else None
    a = torch.full((sc.n, Cout), 3.0, device="cuda")
    c = torch.full((sc.n, Cout), -3.0, device="cuda")
    d = torch.full((sc.n, Cout), 5.0, device="cuda")
    e = torch.full((sc.n, Cout), 11.0, device="cuda")
    try:
        lib.insc_conv_set_shared_weights_min_units(1 << 40)
        lib.insc_conv_set_wavefront_per_unit_min_units(1)  # a wavefront of its own per (tile, output block)
        S.ssc_rows_planned(feats, e, W, bt, sc, m.ssc_plan(sc))
        lib.insc_conv_set_wavefront_per_unit_min_units(1 << 40)
        lib.insc_conv_set_persistent_min_units(1)
        S.ssc_rows_planned(feats, a, W, bt, sc, m.ssc_plan(sc))
        lib.insc_conv_set_persistent_min_units(1 << 40)
        S.ssc_rows_planned(feats, c, W, bt, sc, m.ssc_plan(sc))
        lib.insc_conv_set_shared_weights_min_units(1)  # two output blocks per gathered chunk where there are two
        S.ssc_rows_planned(feats, d, W, bt, sc, m.ssc_plan(sc))
        assert torch.equal(d, c)
        # one output block per unit: enough units for that, too few for pairs of output blocks (with
        # three output blocks the pairs always qualify as well)
        groups, nbt = ((sc.n + 31) // 32 + 3) // 4, (Cout + 31) // 32
        lib.insc_conv_set_shared_weights_min_units(groups * nbt)
        d.fill_(9.0)
        S.ssc_rows_planned(feats, d, W, bt, sc, m.ssc_plan(sc))
    finally:
        lib.insc_conv_set_persistent_min_units((1 << 63) - 1)
        lib.insc_conv_set_shared_weights_min_units(896)
        lib.insc_conv_set_wavefront_per_unit_min_units(2400)
    assert torch.equal(a, c)
    assert torch.equal(d, c)
    assert torch.equal(e, c)
    nt = (sc.n + 31) // 32
    plan = m.ssc_plan(sc)
    sched = plan[3][:nt].cpu().numpy()
    tmask = plan[1][:nt].cpu().numpy().astype(np.uint32)
    assert sorted(sched.tolist()) == list(range(nt)), "the schedule is a permutation of the tiles"
    cost = np.array([bin(int(v)).count("1") for v in tmask])[sched]
    assert (np.diff(cost) <= 0).all(), "tiles by falling number of offsets in use"
    ng = (nt + 3) // 4
    gsched = plan[3][plan[2] // 32:plan[2] // 32 + ng].cpu().numpy()
    assert sorted(gsched.tolist()) == list(range(ng)), "the group schedule is a permutation of the groups"
    gmask = [int(np.bitwise_or.reduce(tmask[4 * g:4 * g + 4])) for g in range(ng)]
    gcost = np.array([bin(v).count("1") for v in gmask])[gsched]
    assert (np.diff(gcost) <= 0).all(), "groups by falling number of offsets in use"
    _, osc, _ = orc.grid_build(pts)
    _, counts, pairs = orc.ssc_rules(osc)
    ref, _ = orc.conv_forward(feats.cpu().numpy(), W.cpu().numpy(), b, pairs, counts, len(osc))
    np.testing.assert_allclose(a.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("Cin,Cout,bias", [(16, 16, False), (16, 16, True), (32, 32, False), (32, 32, True),
                                            (16, 32, True), (32, 20, False)])
def test_filter_in_lds_kernel_against_oracle_and_per_tile_kernel(S, orc, Cin, Cout, bias):
    """Narrow 3^3 layers (Cin, Cout <= 32) have two kernels: one wavefront per tile, and - from 4096
    tiles up by default - persistent blocks that keep the whole filter in LDS (the kernel the
    HBM-roofline figure is quoted on).  Here the threshold is lowered so that the 20k-voxel scene of
    workload 1 runs on the second one, planned and unplanned staging, and the result is compared with
    the CPU oracle (1e-4 / 1e-5) and bit for bit with the first kernel."""
    from sparseconvnet._lib import lib

    pts = scenes.boxes_scene(seed=1, n=20000)
    m, x, feats = setup_sites(S, pts, Cin, seed=Cin + 7)
    sc = m.ssc_rulebook(SZ)
    rng = np.random.default_rng(Cout + 11)
    W = cu((rng.normal(size=(27, Cin, Cout)) * (2.0 / Cin / 27) ** 0.5).astype(np.float32))
    b = rng.normal(size=Cout).astype(np.float32) if bias else None
    bt = cu(b) if bias else None
    per_tile = torch.full((sc.n, Cout), 3.0, device="cuda")
    lds_planned = torch.full((sc.n, Cout), -3.0, device="cuda")
    lds_unplanned = torch.full((sc.n, Cout), 5.0, device="cuda")
    lds_permuted = torch.full((sc.n, Cout), 7.0, device="cuda")
    perm = torch.randperm(sc.n, generator=torch.Generator().manual_seed(Cin)).to(torch.int32).cuda()
    try:
        lib.insc_conv_set_filter_lds_min_tiles(1 << 40)
        S.ssc_rows_planned(feats, per_tile, W, bt, sc, m.ssc_plan(sc))
        lib.insc_conv_set_filter_lds_min_tiles(1)
        S.ssc_rows_planned(feats, lds_planned, W, bt, sc, m.ssc_plan(sc))
        S.conv_rows(feats, lds_unplanned, W, bt, sc.nbr.t, 27, sc.order.t, None, sc.n)
        S.conv_rows(feats, lds_permuted, W, bt, sc.nbr.t, 27, perm, None, sc.n)
    finally:
        lib.insc_conv_set_filter_lds_min_tiles(4096)
    assert torch.equal(lds_planned, per_tile)
    assert torch.equal(lds_unplanned, per_tile)
    assert torch.equal(lds_permuted, per_tile)
    _, osc, _ = orc.grid_build(pts)
    _, counts, pairs = orc.ssc_rules(osc)
    ref, _ = orc.conv_forward(feats.cpu().numpy(), W.cpu().numpy(), b, pairs, counts, len(osc))
    np.testing.assert_allclose(lds_planned.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("n", [1, 20, 33, 130, 1025])
def test_persistent_kernels_on_tiny_and_ragged_scenes(S, n):
    """One site, one tile, two tiles, a group of four tiles with a partial fifth, a partial last tile:
    all four kernels of a 64->64 layer give the same bits."""
    from sparseconvnet._lib import lib

    rng = np.random.default_rng(n)
    side = max(2, int(round((3 * n) ** (1 / 3))))  # a third of the cube's voxels
    vox = np.unique(rng.integers(0, side, (8 * n + 8, 3)), axis=0)
    pts = (vox[rng.permutation(len(vox))[:n]] + 100).astype(np.int64)
    assert len(pts) == n
    m, x, feats = setup_sites(S, pts, 64, seed=n)
    sc = m.ssc_rulebook(SZ)
    W = cu((rng.normal(size=(27, 64, 64)) * 0.05).astype(np.float32))
    outs = []
    try:
        for pers, shared, own in [(1 << 40, 1 << 40, 1 << 40), (1, 1 << 40, 1 << 40), (1 << 40, 1, 1 << 40),
                                  (1 << 40, 1 << 40, 1)]:
            lib.insc_conv_set_persistent_min_units(pers)
            lib.insc_conv_set_shared_weights_min_units(shared)
            lib.insc_conv_set_wavefront_per_unit_min_units(own)
            o = torch.full((sc.n, 64), float(len(outs)), device="cuda")
            S.ssc_rows_planned(feats, o, W, None, sc, m.ssc_plan(sc))
            outs.append(o)
    finally:
        lib.insc_conv_set_persistent_min_units((1 << 63) - 1)
        lib.insc_conv_set_shared_weights_min_units(896)
        lib.insc_conv_set_wavefront_per_unit_min_units(2400)
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(outs[0], outs[2])
    assert torch.equal(outs[0], outs[3])
    assert torch.isfinite(outs[0]).all() and outs[0].abs().max().item() > 0


def test_submanifold_convolution_cfg1_vs_dense_conv3d(S):
    """Workload 1 against the library routine directly (no oracle in the loop)."""
    import torch.nn.functional as F

    pts = scenes.boxes_scene(seed=1, n=20000)
    m, x, feats = setup_sites(S, pts, 16, seed=1)
    W = torch.randn(27, 16, 16, generator=torch.Generator().manual_seed(1)) * (2.0 / 16 / 27) ** 0.5
    out = torch.empty(0, device="cuda")
    S.SubmanifoldConvolution_updateOutput(SZ, torch.LongTensor([3, 3, 3]), m, feats, out, W.cuda(), torch.Tensor(), 1)
    loc = m.getSpatialLocations(SZ)
    G = 128
    dense = torch.zeros(1, 16, G, G, G, dtype=torch.float64)
    dense[0, :, loc[:, 0], loc[:, 1], loc[:, 2]] = feats.cpu().double().t()
    w = W.double().reshape(3, 3, 3, 16, 16).permute(4, 3, 0, 1, 2)
    ref = F.conv3d(dense, w, padding=1)[0, :, loc[:, 0], loc[:, 1], loc[:, 2]].t()
    np.testing.assert_allclose(out.cpu().numpy(), ref.numpy(), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("Cin,Cout", [(32, 64), (64, 96), (16, 8), (3, 5)])
def test_strided_convolution_and_deconvolution(S, orc, Cin, Cout):
    pts = scenes.boxes_scene(seed=5, n=15000)
    m, x, feats = setup_sites(S, pts, Cin, seed=7)
    rng = np.random.default_rng(8)
    W = (rng.normal(size=(8, Cin, Cout)) * (2.0 / Cin / 8) ** 0.5).astype(np.float32)
    two = torch.LongTensor([2, 2, 2])
    out = torch.empty(0, device="cuda")
    flops = S.Convolution_updateOutput(SZ, SZ // 2, two, two, m, feats, out, cu(W), torch.Tensor())
    _, sc, _ = orc.grid_build(pts)
    parent, off, cc = orc.down2_rules(sc)
    counts, pairs = orc.down2_pairs(parent, off)
    ref, rflops = orc.conv_forward(feats.cpu().numpy(), W, None, pairs, counts, len(cc))
    assert flops == rflops and out.shape == ref.shape
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)
    # deconvolution back to the fine sites
    W2 = (rng.normal(size=(8, Cout, Cin)) * (2.0 / Cout / 8) ** 0.5).astype(np.float32)
    b2 = rng.normal(size=Cin).astype(np.float32)
    back = torch.empty(0, device="cuda")
    S.Deconvolution_updateOutput(SZ // 2, SZ, two, two, m, out, back, cu(W2), cu(b2))
    ref2, _ = orc.conv_forward(ref, W2, b2, pairs, counts, len(sc), swap=True)
    np.testing.assert_allclose(back.cpu().numpy(), ref2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("C,leak,affine", [(32, 0.0, True), (96, 0.333, True), (7, 1.0, False), (384, 0.0, True),
                                           (2048, 0.0, True)])
def test_batchnorm(S, orc, C, leak, affine):
    rng = np.random.default_rng(C)
    N = 5001
    x = (rng.normal(size=(N, C)) * 2).astype(np.float32)
    mean, var = rng.normal(size=C).astype(np.float32), rng.uniform(0.5, 2, C).astype(np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32) if affine else None
    b = (rng.normal(size=C) * 0.1).astype(np.float32) if affine else None
    out = torch.empty(0, device="cuda")
    S.BatchNormalization_updateOutput(cu(x), out, None, None, cu(mean), cu(var), cu(g) if affine else torch.Tensor(),
                                      cu(b) if affine else torch.Tensor(), 1e-4, 0.9, False, leak)
    ref = orc.bn_forward(x, mean, var, g, b, 1e-4, leak)
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("Cin,Cout,bias", [(64, 32, False), (384, 192, False), (32, 20, True), (6, 3, True)])
def test_network_in_network(S, orc, Cin, Cout, bias):
    rng = np.random.default_rng(Cin)
    x = rng.normal(size=(7003, Cin)).astype(np.float32)
    W = (rng.normal(size=(Cin, Cout)) * (2.0 / Cin) ** 0.5).astype(np.float32)
    b = rng.normal(size=Cout).astype(np.float32) if bias else None
    out = torch.empty(0, device="cuda")
    flops = S.NetworkInNetwork_updateOutput(cu(x), out, cu(W), cu(b) if bias else torch.Tensor())
    assert flops == 7003 * Cin * Cout
    np.testing.assert_allclose(out.cpu().numpy(), orc.nin_forward(x, W, b), rtol=RTOL, atol=ATOL)


def test_empty_input(S):
    m = S.Metadata_3()
    out = torch.empty(0, device="cuda")
    S.InputLayer_updateOutput(m, SZ, torch.zeros((0, 3), dtype=torch.long), torch.zeros((0, 3), device="cuda"), out,
                              0, 4)
    assert out.shape == (0, 3)
    o2 = torch.empty(0, device="cuda")
    S.SubmanifoldConvolution_updateOutput(SZ, torch.LongTensor([3, 3, 3]), m, out, o2,
                                          torch.zeros(27, 3, 8, device="cuda"), torch.Tensor(), 1)
    assert o2.shape == (0, 8)


def test_row_subset_leaves_other_rows_untouched(S, orc):
    """The `rows` argument of the C ABI: listed rows are recomputed, the rest keep their bytes."""
    pts = scenes.boxes_scene(seed=1, n=8000)
    m, x, feats = setup_sites(S, pts, 32, seed=3)
    sc = m.ssc_rulebook(SZ)
    W = cu((np.random.default_rng(0).normal(size=(27, 32, 32)) * 0.05).astype(np.float32))
    full = torch.empty(0, device="cuda")
    S.SubmanifoldConvolution_updateOutput(SZ, torch.LongTensor([3, 3, 3]), m, feats, full, W, torch.Tensor(), 1)
    out = torch.full_like(full, 123.0)
    rows = torch.arange(0, sc.n, 3, dtype=torch.int32, device="cuda")
    count = torch.tensor([len(rows) - 10], dtype=torch.int32, device="cuda")
    S.conv_rows(feats, out, W, None, sc.nbr.t, 27, rows, count, len(rows))
    done = rows[:len(rows) - 10].long()
    assert torch.equal(out[done], full[done])  # bit-identical: a row's result does not depend on its tile
    mask = torch.ones(sc.n, dtype=torch.bool, device="cuda")
    mask[done] = False
    assert bool((out[mask] == 123.0).all())


@pytest.mark.parametrize("Cin,Cout,n_sites", [(224, 224, 70), (128, 128, 2900), (160, 160, 700), (256, 128, 2900),
                                              (192, 96, 10000)])
def test_split_layers_repeat_bit_for_bit(S, orc, Cin, Cout, n_sites):
    """Wide 3^3 layers at the coarse scales split a tile's items over G = 2, 4 or 8 blocks, which exchange
    partial sums through memory (the block that arrives last adds them in block order).  Nothing in that
    exchange may depend on timing: 300 launches on the same input must give the same bits every time
    (stopping at the first difference), and they must match the oracle."""
    pts = scenes.boxes_scene(seed=9, n=n_sites)
    m, x, feats = setup_sites(S, pts, Cin, seed=Cin + n_sites)
    sc = m.ssc_rulebook(SZ)
    plan = m.ssc_plan(sc)
    rng = np.random.default_rng(Cout)
    W = (rng.normal(size=(27, Cin, Cout)) * (2.0 / Cin / 27) ** 0.5).astype(np.float32)
    Wd = cu(W)
    first = torch.empty((sc.n, Cout), device="cuda")
    S.ssc_rows_planned(feats, first, Wd, None, sc, plan)
    _, osc, _ = orc.grid_build(pts)
    _, counts, pairs = orc.ssc_rules(osc)
    ref, _ = orc.conv_forward(feats.cpu().numpy(), W, None, pairs, counts, len(osc))
    np.testing.assert_allclose(first.cpu().numpy(), ref, rtol=RTOL, atol=ATOL)
    out = torch.empty_like(first)
    for i in range(300):
        out.fill_(float(i))
        S.ssc_rows_planned(feats, out, Wd, None, sc, plan)
        assert torch.equal(out, first), "launch %d differs: max |diff| %.3e" % (i, (out - first).abs().max().item())
