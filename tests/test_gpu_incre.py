"""GPU parity of the residual frame operators (the reference's Incre_* functions) against the
CPU oracle, called through the reference's names (sparseconvnet.SCN.Incre_*_updateOutput) and
through the module tree with increment="residual".  Tolerance: 1e-4 relative / 1e-5 absolute
per operator on values of order one; integer maps are compared exactly."""
import copy

import numpy as np
import pytest
import torch

import parity

from workloads import scenes

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-4, 1e-5
SZ = torch.LongTensor([4096, 4096, 4096])
SZ2 = torch.LongTensor([2048, 2048, 2048])
F3 = torch.LongTensor([3, 3, 3])
F2 = torch.LongTensor([2, 2, 2])


@pytest.fixture(scope="module")
def S():
    from sparseconvnet import SCN
    from sparseconvnet._lib import ensure_init

    ensure_init(0)
    return SCN


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


def _scene(seed, n_a=12000, n_old=2500, n_new=3000):
    vox = scenes.boxes_scene(seed=seed, n=n_a + n_new)
    rng = np.random.default_rng(seed)
    a = vox[:n_a]
    b = np.concatenate([a[rng.choice(n_a, n_old, replace=False)], vox[n_a:]])[rng.permutation(n_old + n_new)]
    return a, b


def _site_sets(S, a, b, C, mode=0):
    """Metadata of the saved scene and of the frame (one point per voxel, features unused)."""
    ma, mb = S.Metadata_3(), S.Metadata_3()
    fa = torch.zeros((len(a), C), device="cuda")
    fb = torch.zeros((len(b), C), device="cuda")
    S.InputLayer_updateOutput(ma, SZ, torch.from_numpy(a.astype(np.int64)), fa, torch.empty(0, device="cuda"), 0, mode)
    S.InputLayer_updateOutput(mb, SZ, torch.from_numpy(b.astype(np.int64)), fb, torch.empty(0, device="cuda"), 0, mode)
    return ma, mb


def test_pre_exist_and_incre_rulebook(S, orc):
    a, b = _scene(1)
    ma, mb = _site_sets(S, a, b, 1)
    pe = host(mb.pre_exist_map(SZ, ma))
    ref = orc.incre_pre_exist(a, b)
    assert (pe == ref).all() and (ref >= 0).sum() == 2500
    nbr_pre = host(mb.incre_ssc_map(SZ, ma))
    counts, pairs = orc.incre_ssc_rules(b, a, ref)
    got = []
    for k in range(27):
        o = np.nonzero(nbr_pre[:, k] >= 0)[0]
        got.append(np.stack([nbr_pre[o, k], o], 1))
        assert len(o) == counts[k]
    assert (np.concatenate(got) == pairs).all()
    assert (nbr_pre[ref >= 0] == -1).all()


@pytest.mark.parametrize("Cin,Cout,bias", [(3, 16, False), (32, 32, True), (64, 64, False), (96, 64, False),
                                            (160, 160, False), (20, 7, True)])
def test_incre_submanifold_convolution(S, orc, Cin, Cout, bias):
    a, b = _scene(2)
    ma, mb = _site_sets(S, a, b, 1)
    rng = np.random.default_rng(Cin + Cout)
    x_a = rng.normal(size=(len(a), Cin)).astype(np.float32)
    r = rng.normal(size=(len(b), Cin)).astype(np.float32)
    W = (rng.normal(size=(27, Cin, Cout)) * (2.0 / Cin / 27) ** 0.5).astype(np.float32)
    bv = rng.normal(size=Cout).astype(np.float32) if bias else None
    out = torch.empty(0, device="cuda")
    flops = S.Incre_SubmanifoldConvolution_updateOutput(SZ, F3, mb, cu(r), out, cu(W),
                                                        cu(bv) if bias else torch.Tensor(), ma, cu(x_a))
    pe = orc.incre_pre_exist(a, b)
    _, counts, pairs = orc.ssc_rules(b)
    rules_pre = orc.incre_ssc_rules(b, a, pe)
    ref = orc.incre_ssc_forward(r, x_a, W, bv, (counts, pairs), rules_pre, len(b))
    assert flops == float(len(pairs) + len(rules_pre[1])) * Cin * Cout
    np.testing.assert_allclose(host(out), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("Cin,Cout", [(32, 32), (64, 64)])
def test_incre_submanifold_convolution_frame_larger_than_saved_set(S, orc, Cin, Cout):
    """The gather of saved features reads a matrix with fewer rows than the frame has sites."""
    a, b = _scene(6, n_a=3000, n_old=2800, n_new=5000)
    ma, mb = _site_sets(S, a, b, 1)
    rng = np.random.default_rng(Cin)
    x_a = rng.normal(size=(len(a), Cin)).astype(np.float32)
    r = rng.normal(size=(len(b), Cin)).astype(np.float32)
    W = (rng.normal(size=(27, Cin, Cout)) * (2.0 / Cin / 27) ** 0.5).astype(np.float32)
    out = torch.empty(0, device="cuda")
    S.Incre_SubmanifoldConvolution_updateOutput(SZ, F3, mb, cu(r), out, cu(W), torch.Tensor(), ma, cu(x_a))
    pe = orc.incre_pre_exist(a, b)
    _, counts, pairs = orc.ssc_rules(b)
    ref = orc.incre_ssc_forward(r, x_a, W, None, (counts, pairs), orc.incre_ssc_rules(b, a, pe), len(b))
    np.testing.assert_allclose(host(out), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("C,leak", [(32, 0.0), (64, 0.3), (7, 0.0), (384, 0.0)])
def test_incre_batchnorm(S, orc, C, leak):
    a, b = _scene(3)
    ma, mb = _site_sets(S, a, b, 1)
    rng = np.random.default_rng(C)
    x_a = rng.normal(size=(len(a), C)).astype(np.float32)
    r = rng.normal(size=(len(b), C)).astype(np.float32)
    mean, var = (rng.normal(size=C) * 0.3).astype(np.float32), rng.uniform(0.5, 2, C).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, C).astype(np.float32), (rng.normal(size=C) * 0.2).astype(np.float32)
    y_a = orc.bn_forward(x_a, mean, var, gamma, beta, 1e-4, leak)
    out = torch.empty(0, device="cuda")
    S.Incre_BatchNormalization_updateOutput(cu(r), out, None, None, cu(mean), cu(var), cu(gamma), cu(beta), 1e-4, 0.9,
                                            False, leak, mb, ma, cu(y_a), cu(x_a), SZ)
    ref = orc.incre_bn_forward(r, mean, var, gamma, beta, 1e-4, leak, orc.incre_pre_exist(a, b), x_a, y_a)
    np.testing.assert_allclose(host(out), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("Cin,Cout", [(32, 64), (64, 32), (128, 96), (6, 4)])
def test_incre_convolution_and_deconvolution(S, orc, Cin, Cout):
    a, b = _scene(4)
    ma, mb = _site_sets(S, a, b, 1)
    rng = np.random.default_rng(Cin * 3 + Cout)
    r = rng.normal(size=(len(b), Cin)).astype(np.float32)
    W = (rng.normal(size=(8, Cin, Cout)) * (2.0 / Cin / 8) ** 0.5).astype(np.float32)
    # the saved scene's coarse scale has to exist (a full forward creates it)
    S.Convolution_updateOutput(SZ, SZ2, F2, F2, ma, torch.zeros((len(a), Cin), device="cuda"),
                               torch.empty(0, device="cuda"), cu(W), torch.Tensor())
    out = torch.empty(0, device="cuda")
    S.Incre_Convolution_updateOutput(SZ, SZ2, F2, F2, mb, cu(r), out, cu(W), torch.Tensor())
    parent_b, off_b, cc_b = orc.down2_rules(b)
    counts, pairs = orc.down2_pairs(parent_b, off_b)
    ref, _ = orc.conv_forward(r, W, None, pairs, counts, len(cc_b))
    np.testing.assert_allclose(host(out), ref, rtol=RTOL, atol=ATOL)

    _, _, cc_a = orc.down2_rules(a)
    Wd = (rng.normal(size=(8, Cout, Cin)) * (2.0 / Cout / 8) ** 0.5).astype(np.float32)
    z_a = rng.normal(size=(len(cc_a), Cout)).astype(np.float32)
    rz = rng.normal(size=(len(cc_b), Cout)).astype(np.float32)
    bias = rng.normal(size=Cin).astype(np.float32)
    out = torch.empty(0, device="cuda")
    S.Incre_Deconvolution_updateOutput(SZ2, SZ, F2, F2, mb, cu(rz), out, cu(Wd), cu(bias), ma, cu(z_a))
    pe_c, pe_f = orc.incre_pre_exist(cc_a, cc_b), orc.incre_pre_exist(a, b)
    assert (host(mb.pre_exist_map(SZ2, ma)) == pe_c).all()
    ref = orc.incre_deconv_forward(rz, z_a, Wd, bias, parent_b, off_b, pe_c, pe_f)
    assert ((pe_f < 0) & (pe_c[parent_b] >= 0)).sum() > 100
    np.testing.assert_allclose(host(out), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("mode", [0, 1, 2, 3, 4])
def test_incre_input_and_output_layers(S, orc, mode):
    a, b = _scene(5, n_a=6000, n_old=1500, n_new=1500)
    rng = np.random.default_rng(mode)
    if mode == 0:
        pts_a, pts_b = a, b
    else:
        pts_a = np.concatenate([a, a[rng.integers(0, len(a), 2000)]])[rng.permutation(len(a) + 2000)]
        pts_b = np.concatenate([b, b[rng.integers(0, len(b), 1500)]])[rng.permutation(len(b) + 1500)]
    f_a = rng.uniform(0, 1, (len(pts_a), 3)).astype(np.float32)
    f_b = rng.uniform(0, 1, (len(pts_b), 3)).astype(np.float32)
    ma, mb = S.Metadata_3(), S.Metadata_3()
    pre = torch.empty(0, device="cuda")
    S.InputLayer_updateOutput(ma, SZ, torch.from_numpy(pts_a.astype(np.int64)), cu(f_a), pre, 0, mode)
    out = torch.empty(0, device="cuda")
    S.Incre_InputLayer_updateOutput(mb, SZ, torch.from_numpy(pts_b.astype(np.int64)), cu(f_b), out, 0, mode, ma, pre)
    sop_a, sc_a, cnt_a = orc.grid_build(pts_a)
    sop_b, sc_b, cnt_b = orc.grid_build(pts_b)
    pe = orc.incre_pre_exist(sc_a, sc_b)
    ref = orc.incre_input_forward(f_b, sop_b, cnt_b, mode, pe, host(pre), cnt_a)
    np.testing.assert_allclose(host(out), ref, rtol=RTOL, atol=ATOL)
    # saved state untouched
    assert ma.getNActive(SZ) == len(sc_a)
    o = torch.empty(0, device="cuda")
    S.Incre_OutputLayer_updateOutput(mb, out, o, ma, pre)
    np.testing.assert_allclose(host(o), orc.incre_output_forward(ref, sop_b, pe, host(pre)), rtol=RTOL, atol=ATOL)
    assert o.shape[0] == len(pts_b)


def _frames(seed):
    vox = scenes.indoor_scene(seed=seed, n=9000, dims=(70, 60, 24), n_boxes=6, side_rng=(6, 16))
    rng = np.random.default_rng(seed)
    order = np.argsort(np.linalg.norm(vox[:, :3] - vox[:, :3].min(0).astype(np.float64), axis=1), kind="stable")
    base = rng.uniform(0, 1, (len(vox), 3)).astype(np.float32)
    n0 = 6000
    f0 = (vox[order[:n0]], base[order[:n0]])
    new = order[n0:n0 + 1500]
    old = order[rng.integers(0, n0, 600)]
    idx = np.concatenate([new, old])
    rgb = base[idx].copy()
    rgb[len(new):] += rng.uniform(-0.1, 0.1, (len(old), 3)).astype(np.float32)
    perm = rng.permutation(len(idx))
    return f0, (vox[idx][perm], rgb[perm]), (vox, base)


def _inp(pts, rgb):
    return [torch.from_numpy(pts[:, :3].astype(np.int64)), torch.from_numpy(rgb).cuda(), 1]


@pytest.mark.parametrize("levels,m", [(3, 16), (5, 32)])
def test_residual_frame_network_vs_oracle(levels, m):
    """Whole network: frame 0 full, frame 1 with increment="residual", against the oracle's
    residual network; then the saved state must be what the full forward left."""
    from oracle import oracle_net
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    f0, f1, _ = _frames(31)
    model = NaiveUNet(m=m, levels=levels, seed=9).cuda()
    cpu = copy.deepcopy(model).cpu()
    ref_model = copy.deepcopy(model)
    with torch.no_grad():
        model(_inp(*f0), increment=False)
        got = model.sparseModel(_inp(*f1), increment="residual")
        again = model.sparseModel(_inp(*f1), "residual")
    save = {}
    oracle_net.forward(cpu.sparseModel, [f0[0][:, :3], f0[1], 1], save)
    ref = oracle_net.forward_residual(cpu.sparseModel, [f1[0][:, :3], f1[1], 1], save)
    assert got.shape == ref.shape == (len(f1[0]), m)
    parity.check("residual frame, %d-level U-Net vs residual oracle" % levels, got.cpu().numpy(), ref)
    # a residual frame leaves the saved state alone: the same frame again gives the same bits,
    # and an exact incremental frame afterwards still equals a full forward over all points
    assert torch.equal(got, again)
    for mod in model.modules():
        if isinstance(mod, scn.OutputLayer):
            mod.all_points = True
    with torch.no_grad():
        exact = model(_inp(*f1), increment="exact")
        both = ref_model(_inp(np.concatenate([f0[0], f1[0]]), np.concatenate([f0[1], f1[1]])), increment=False)
    assert torch.equal(exact, both)


def test_residual_frame_covering_scene_equals_full_forward():
    """A frame that observes every saved voxel again is exact (every operator is exact on the
    frame's sites): logits(residual) == logits(full forward over both frames) within float
    tolerance, at 150k-scale channel widths but a small scene."""
    from workloads.netdefs import NaiveUNet

    _, _, (vox, base) = _frames(32)
    rng = np.random.default_rng(33)
    a = vox[:7000]
    b = vox[rng.permutation(len(vox))]
    f_a = base[:7000]
    f_b = rng.uniform(0, 1, (len(b), 3)).astype(np.float32)
    model = NaiveUNet(m=32, levels=5, seed=10).cuda()
    with torch.no_grad():
        model(_inp(a, f_a), increment=False)
        res = model(_inp(b, f_b), increment="residual")
        full = model(_inp(np.concatenate([a, b]), np.concatenate([f_a, f_b])), increment=False)
    ref = full[len(a):]
    parity.check("residual frame covering the scene vs full forward", res.cpu().numpy(), ref.cpu().numpy())


def test_increment_true_follows_set_mode():
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    f0, f1, _ = _frames(34)
    model = NaiveUNet(m=16, levels=3, seed=11).cuda()
    with torch.no_grad():
        model(_inp(*f0), increment=False)
        want = model(_inp(*f1), increment="residual")
        scn.set_incremental_mode("residual")
        try:
            got = model(_inp(*f1), increment=True)
        finally:
            scn.set_incremental_mode("exact")
    assert scn.get_incremental_mode() == "exact"
    assert torch.equal(got, want)
    with pytest.raises(ValueError):
        model(_inp(*f1), increment="approximate")


@pytest.mark.parametrize("levels,m", [(3, 16), (7, 32)])
def test_compiled_residual_frames_equal_module_tree(levels, m):
    """The executor's residual frame (one C call) against the module tree's: same kernels on the
    same rows, so the same bits.  With residual=True the executor also keeps the inputs of the
    batch norms; full and exact incremental frames must not change because of that, and a
    residual frame must leave the saved state as it was."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    f0, f1, _ = _frames(35)
    model = NaiveUNet(m=m, levels=levels, seed=12).cuda()
    ref_model = copy.deepcopy(model)
    net = scn.compile(model.sparseModel, capacity_sites=4096, residual=True)
    plain = scn.compile(copy.deepcopy(model).sparseModel, capacity_sites=4096)
    with torch.no_grad():
        full = net(_inp(*f0), increment=False)
        assert torch.equal(full, ref_model.sparseModel(_inp(*f0), False))
        want = ref_model.sparseModel(_inp(*f1), "residual")
        got = net(_inp(*f1), increment="residual")
        assert got.shape == want.shape == (len(f1[0]), m)
        assert torch.equal(got, want), "max diff %.3e" % (got - want).abs().max().item()
        assert net.n_sites_frame == len(np.unique(f1[0], axis=0))
        # a smaller frame right after a larger one (the frame's buffers are reused)
        half = (f1[0][:700], f1[1][:700])
        assert torch.equal(net(_inp(*half), increment="residual"), ref_model.sparseModel(_inp(*half), "residual"))
        # the saved state is intact: an exact incremental frame equals a full forward over both
        exact = net(_inp(*f1), increment=True, all_points=True)
        both = ref_model.sparseModel(_inp(np.concatenate([f0[0], f1[0]]), np.concatenate([f0[1], f1[1]])), False)
        assert torch.equal(exact, both)
        # and residual frames now refer to the state after that exact frame
        want2 = ref_model.sparseModel(_inp(*half), "residual")
        assert torch.equal(net(_inp(*half), increment="residual"), want2)
        with pytest.raises(RuntimeError):
            plain(_inp(*f0), increment=False)
            plain(_inp(*f1), increment="residual")
