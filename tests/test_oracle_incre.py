"""Pins the oracle's restatement of the reference's residual operators (Incre_*).

The reference holds no test or golden vector for them, so each is pinned by the identity
that defines it: for a saved scene A and a frame B (some voxels of A observed again, some new
ones), with the frame's features being differences for voxels of A and plain values for new
voxels,

    saved output + residual output == the plain operator applied to the merged scene,

at every site of the frame.  The right-hand side comes from a library routine (dense torch
conv3d in float64) or from the plain oracle operator that tests/test_oracle_ops.py pins
against one.  A dropped saved term, a wrong sign, a swapped existing/new case or a wrong
neighbour direction fails here.  The input layer's non-mean modes, for which the reference's
formula does not satisfy the identity, are pinned by hand-computed values instead.

Tolerance 1e-4 relative / 1e-5 absolute on values of order one.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

RTOL, ATOL = 1e-4, 1e-5
G = 16


def _scene(seed, n_a=900, n_old=200, n_new=250):
    """(coords of A, coords of the frame B, pre_exist of B): B = n_old sites of A + n_new others."""
    rng = np.random.default_rng(seed)
    allc = np.stack(np.meshgrid(np.arange(1, G - 1), np.arange(1, G - 1), np.arange(1, G - 1), indexing="ij"), -1)
    allc = allc.reshape(-1, 3)[rng.permutation((G - 2) ** 3)].astype(np.int32)
    a = allc[:n_a]
    new = allc[n_a:n_a + n_new]
    old = a[rng.choice(n_a, n_old, replace=False)]
    b = np.concatenate([old, new])[rng.permutation(n_old + n_new)]
    return a, b


def _dense(coords, feats):
    d = torch.zeros(1, feats.shape[1], G, G, G, dtype=torch.float64)
    c = torch.from_numpy(coords.astype(np.int64))
    d[0, :, c[:, 0], c[:, 1], c[:, 2]] = torch.from_numpy(feats.astype(np.float64)).t()
    return d


def _at(d, coords):
    c = torch.from_numpy(coords.astype(np.int64))
    return d[0, :, c[:, 0], c[:, 1], c[:, 2]].t().numpy()


def _merge(orc, a, b, x_a, r):
    """Merged scene: sites of A then the new sites of B; features x_a (+ r where observed again), r."""
    pe = orc.incre_pre_exist(a, b)
    new = pe < 0
    m = np.concatenate([a, b[new]])
    x = np.concatenate([x_a, r[new]]).astype(np.float32)
    np.add.at(x, pe[~new], r[~new])
    id_in_m = np.where(new, len(a) + np.cumsum(new) - 1, pe)
    return pe, m, x, id_in_m


def test_pre_exist(orc):
    a, b = _scene(0)
    pe = orc.incre_pre_exist(a, b)
    look = {tuple(c): i for i, c in enumerate(a.tolist())}
    assert pe.tolist() == [look.get(tuple(c), -1) for c in b.tolist()]
    assert (pe >= 0).sum() == 200


def test_incre_ssc_identity_vs_conv3d(orc):
    a, b = _scene(1)
    rng = np.random.default_rng(2)
    Cin, Cout = 5, 6
    x_a = rng.normal(size=(len(a), Cin)).astype(np.float32)
    r = rng.normal(size=(len(b), Cin)).astype(np.float32)
    W = (rng.normal(size=(27, Cin, Cout)) * 0.2).astype(np.float32)
    pe, m, x_m, _ = _merge(orc, a, b, x_a, r)
    _, counts, pairs = orc.ssc_rules(b)
    rules_pre = orc.incre_ssc_rules(b, a, pe)
    # only new sites gather saved features, and never from themselves
    assert set(rules_pre[1][:, 1].tolist()) <= set(np.nonzero(pe < 0)[0].tolist())
    assert rules_pre[0][13] == 0
    y = orc.incre_ssc_forward(r, x_a, W, None, (counts, pairs), rules_pre, len(b))
    w = torch.from_numpy(W.astype(np.float64)).reshape(3, 3, 3, Cin, Cout).permute(4, 3, 0, 1, 2)
    full_m = _at(F.conv3d(_dense(m, x_m), w, padding=1), b)
    full_a = _at(F.conv3d(_dense(a, x_a), w, padding=1), b)  # zero... not used for new sites
    ref = np.where((pe >= 0)[:, None], full_m - full_a, full_m)
    np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)
    # the saved-feature term matters: without it the new sites come out wrong
    y0 = orc.incre_ssc_forward(r, x_a, W, None, (counts, pairs), (np.zeros(27, np.int32), np.zeros((0, 2), np.int32)),
                               len(b))
    assert np.abs(y0 - ref)[pe < 0].max() > 0.1


def test_incre_bn_identity(orc):
    a, b = _scene(3)
    rng = np.random.default_rng(4)
    C = 7
    x_a = rng.normal(size=(len(a), C)).astype(np.float32)
    r = rng.normal(size=(len(b), C)).astype(np.float32)
    mean, var = rng.normal(size=C).astype(np.float32) * 0.3, rng.uniform(0.5, 2, C).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, C).astype(np.float32), rng.normal(size=C).astype(np.float32) * 0.2
    pe = orc.incre_pre_exist(a, b)
    for leak in (0.0, 0.3):
        y_a = orc.bn_forward(x_a, mean, var, gamma, beta, 1e-4, leak)
        y = orc.incre_bn_forward(r, mean, var, gamma, beta, 1e-4, leak, pe, x_a, y_a)

        def bn64(x):
            o = (x.astype(np.float64) - mean) / np.sqrt(var.astype(np.float64) + 1e-4) * gamma + beta
            return np.where(o > 0, o, o * leak)

        old = pe >= 0
        ref = np.empty_like(y, dtype=np.float64)
        ref[old] = bn64(x_a[pe[old]].astype(np.float64) + r[old]) - bn64(x_a[pe[old]])
        ref[~old] = bn64(r[~old])
        np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)


def test_incre_conv_and_deconv_identity(orc):
    a, b = _scene(5)
    rng = np.random.default_rng(6)
    Cin, Cout = 6, 4
    x_a = rng.normal(size=(len(a), Cin)).astype(np.float32)
    r = rng.normal(size=(len(b), Cin)).astype(np.float32)
    W = (rng.normal(size=(8, Cin, Cout)) * 0.3).astype(np.float32)
    pe, m, x_m, _ = _merge(orc, a, b, x_a, r)

    def conv(c, x):
        parent, off, cc = orc.down2_rules(c)
        counts, pairs = orc.down2_pairs(parent, off)
        y, _ = orc.conv_forward(x, W, None, pairs, counts, len(cc))
        return y, cc, parent, off

    # strided convolution: the plain operator on the frame's own sites (Incre_Convolution_updateOutput)
    y_b, cc_b, parent_b, off_b = conv(b, r)
    y_m, cc_m, _, _ = conv(m, x_m)
    y_a, cc_a, _, _ = conv(a, x_a)
    in_m = orc.grid_query(cc_m, cc_b)
    pe_c = orc.incre_pre_exist(cc_a, cc_b)
    assert (in_m >= 0).all()
    ref = y_m[in_m].copy()
    ref[pe_c >= 0] -= y_a[pe_c[pe_c >= 0]]
    np.testing.assert_allclose(y_b, ref, rtol=RTOL, atol=ATOL)

    # deconvolution back to the fine scale: coarse features z (saved z_a on A's coarse sites,
    # residual rz on the frame's), Cout -> Cin
    Wd = (rng.normal(size=(8, Cout, Cin)) * 0.3).astype(np.float32)
    z_a = rng.normal(size=(len(cc_a), Cout)).astype(np.float32)
    rz = rng.normal(size=(len(cc_b), Cout)).astype(np.float32)
    z_m = np.zeros((len(cc_m), Cout), np.float32)
    z_m[orc.grid_query(cc_m, cc_a)] = z_a
    z_m[in_m] += rz

    def deconv(c, z):
        parent, off, cc = orc.down2_rules(c)
        counts, pairs = orc.down2_pairs(parent, off)
        y, _ = orc.conv_forward(z, Wd, None, pairs, counts, len(c), swap=True)
        return y

    d_m, d_a = deconv(m, z_m), deconv(a, z_a)
    fine_in_m = orc.grid_query(m, b)
    ref = d_m[fine_in_m].copy()
    ref[pe >= 0] -= d_a[pe[pe >= 0]]
    y = orc.incre_deconv_forward(rz, z_a, Wd, None, parent_b, off_b, pe_c, pe)
    np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)
    # there are new fine sites under coarse sites that existed (the case the extra term is for)
    assert ((pe < 0) & (pe_c[parent_b] >= 0)).sum() > 20


def test_incre_input_mean_and_output_identity(orc):
    a, b = _scene(7)
    rng = np.random.default_rng(8)
    C = 3
    pts_a = np.concatenate([a, a[rng.integers(0, len(a), 300)]])[rng.permutation(len(a) + 300)]
    pts_b = np.concatenate([b, b[rng.integers(0, len(b), 200)]])[rng.permutation(len(b) + 200)]
    f_a = rng.uniform(0, 1, (len(pts_a), C)).astype(np.float32)
    f_b = rng.uniform(0, 1, (len(pts_b), C)).astype(np.float32)
    sop_a, sc_a, cnt_a = orc.grid_build(pts_a)
    sop_b, sc_b, cnt_b = orc.grid_build(pts_b)
    pre_out = orc.input_forward(f_a, sop_a, cnt_a, mode=4)
    pe = orc.incre_pre_exist(sc_a, sc_b)
    res = orc.incre_input_forward(f_b, sop_b, cnt_b, 4, pe, pre_out, cnt_a)
    # mean over every point of both frames, straight from numpy
    sop_m, sc_m, cnt_m = orc.grid_build(np.concatenate([pts_a, pts_b]))
    s = np.zeros((len(sc_m), C), np.float64)
    np.add.at(s, sop_m, np.concatenate([f_a, f_b]).astype(np.float64))
    mean_m = s / cnt_m[:, None]
    ref = mean_m[orc.grid_query(sc_m, sc_b)]
    ref[pe >= 0] -= pre_out[pe[pe >= 0]]
    np.testing.assert_allclose(res, ref, rtol=RTOL, atol=ATOL)
    # output layer: residual + saved value, one row per point of the frame
    out = orc.incre_output_forward(res, sop_b, pe, pre_out)
    np.testing.assert_allclose(out, mean_m[orc.grid_query(sc_m, pts_b)], rtol=RTOL, atol=ATOL)


def test_incre_input_other_modes_by_hand(orc):
    # saved frame: voxel (1,1,1) seen twice (rows 0, 2), voxel (2,2,2) once
    pts_a = np.array([[1, 1, 1], [2, 2, 2], [1, 1, 1]], np.int32)
    f_a = np.array([[1.0, 10.0], [5.0, 50.0], [3.0, 30.0]], np.float32)
    # frame: (1,1,1) twice (rows 0, 1), a new voxel (3,3,3) once
    pts_b = np.array([[1, 1, 1], [1, 1, 1], [3, 3, 3]], np.int32)
    f_b = np.array([[2.0, 20.0], [4.0, 40.0], [7.0, 70.0]], np.float32)
    sop_a, sc_a, cnt_a = orc.grid_build(pts_a)
    sop_b, sc_b, cnt_b = orc.grid_build(pts_b)
    pe = orc.incre_pre_exist(sc_a, sc_b)
    assert pe.tolist() == [0, -1]
    # mode 3 (sum): out = sum_new + pre*(pn - 1), pn = 2 saved rows -> [6,60] + [4,40]*1
    pre3 = orc.input_forward(f_a, sop_a, cnt_a, mode=3)
    assert pre3[0].tolist() == [4.0, 40.0]
    r3 = orc.incre_input_forward(f_b, sop_b, cnt_b, 3, pe, pre3, cnt_a)
    assert r3.tolist() == [[10.0, 100.0], [7.0, 70.0]]
    # mode 1 (first row): rule length 1 on both sides -> pre*(1-1) = 0, the first new row remains
    pre1 = np.array([[1.0, 10.0], [5.0, 50.0]], np.float32)
    r1 = orc.incre_input_forward(f_b, sop_b, cnt_b, 1, pe, pre1, cnt_a)
    assert r1.tolist() == [[2.0, 20.0], [7.0, 70.0]]
    r2 = orc.incre_input_forward(f_b, sop_b, cnt_b, 2, pe, pre1, cnt_a)
    assert r2.tolist() == [[4.0, 40.0], [7.0, 70.0]]
    # mode 4 (mean): m = 1/(2+2): (2+4)/4 + 2*(2/4 - 1) = 1.5 - 1 = 0.5 ; new voxel: 7
    pre4 = orc.input_forward(f_a, sop_a, cnt_a, mode=4)
    assert pre4[0].tolist() == [2.0, 20.0]
    r4 = orc.incre_input_forward(f_b, sop_b, cnt_b, 4, pe, pre4, cnt_a)
    np.testing.assert_allclose(r4, [[0.5, 5.0], [7.0, 70.0]], rtol=1e-6)


@pytest.mark.parametrize("levels", [2, 3])
def test_residual_net_exact_when_frame_covers_scene(orc, levels):
    """Every operator is exact on the frame's sites, so a frame that observes every saved voxel
    again (plus new ones) must reproduce a full forward over all points of both frames."""
    from oracle import oracle_net
    from workloads import scenes
    from workloads.netdefs import NaiveUNet

    vox = scenes.boxes_scene(seed=11, n=1500, grid=48, n_boxes=3, lo_rng=(4, 24), size_rng=(8, 18))
    rng = np.random.default_rng(12)
    a = vox[:1100]
    b = np.concatenate([a, vox[1100:]])[rng.permutation(len(vox))]
    f_a = rng.uniform(0, 1, (len(a), 3)).astype(np.float32)
    f_b = rng.uniform(0, 1, (len(b), 3)).astype(np.float32)
    model = NaiveUNet(m=8, levels=levels, full_scale=64, seed=5)
    save = {}
    oracle_net.forward(model.sparseModel, [a[:, :3], f_a, 1], save)
    res = oracle_net.forward_residual(model.sparseModel, [b[:, :3], f_b, 1], save)
    full = oracle_net.forward(model.sparseModel, [np.concatenate([a, b])[:, :3], np.concatenate([f_a, f_b]), 1])
    ref = full[len(a):]
    scale = np.abs(ref).max()
    np.testing.assert_allclose(res, ref, rtol=1e-3, atol=1e-4 * max(1.0, scale))
    # and a frame that leaves most of the scene out is only an approximation of it
    part = vox[900:]
    f_p = rng.uniform(0, 1, (len(part), 3)).astype(np.float32)
    res_p = oracle_net.forward_residual(model.sparseModel, [part[:, :3], f_p, 1], save)
    full_p = oracle_net.forward(model.sparseModel, [np.concatenate([a, part])[:, :3], np.concatenate([f_a, f_p]), 1])
    assert res_p.shape == full_p[len(a):].shape
    assert np.abs(res_p - full_p[len(a):]).max() > 1e-3
