"""Edge cases of the path on the GPU: several scenes in one batch, sites on the border of the
coordinate range, empty and duplicate-only increments, residual frames that share nothing or
everything with the saved scene."""
import copy

import numpy as np
import pytest
import torch

import parity

from workloads import scenes

pytestmark = pytest.mark.gpu


def _inp(pts, rgb, bs=1):
    return [torch.from_numpy(pts.astype(np.int64)), torch.from_numpy(rgb).cuda(), bs]


def _scene(seed, n=5000):
    vox = scenes.indoor_scene(seed=seed, n=n, dims=(60, 50, 20), n_boxes=5, side_rng=(6, 14))
    rgb = np.random.default_rng(seed).uniform(0, 1, (len(vox), 3)).astype(np.float32)
    return vox, rgb


def test_batch_of_scenes_equals_scenes_run_alone():
    """Two scenes with batch indices 0 and 1 (overlapping coordinates): nothing may leak across the
    batch index - each scene's logits equal those of the scene run alone, bit for bit - and the
    whole batch matches the oracle."""
    from oracle import oracle_net
    from workloads.netdefs import NaiveUNet

    (va, fa), (vb, fb) = _scene(41), _scene(42, 4000)
    vb = vb.copy()
    vb[:, 3] = 1
    rng = np.random.default_rng(43)
    perm = rng.permutation(len(va) + len(vb))
    pts, rgb = np.concatenate([va, vb])[perm], np.concatenate([fa, fb])[perm]
    model = NaiveUNet(m=16, levels=4, seed=13).cuda()
    cpu = copy.deepcopy(model).cpu()
    with torch.no_grad():
        both = model.sparseModel(_inp(pts, rgb, 2))
        alone_a = model.sparseModel(_inp(va, fa))
        alone_b = model.sparseModel(_inp(vb[:, :3], fb))
    inv = np.argsort(perm)
    assert torch.equal(both[inv[:len(va)]], alone_a)
    assert torch.equal(both[inv[len(va):]], alone_b)
    ref = oracle_net.forward(cpu.sparseModel, [pts, rgb, 2])
    parity.check("two samples in one batch, 4-level U-Net", both.cpu().numpy(), ref)


def test_sites_on_the_border_of_the_coordinate_range(orc):
    """Voxels at 0 and 65535: their neighbours outside the range do not exist (and must not alias
    voxels on the other side)."""
    from sparseconvnet import SCN

    rng = np.random.default_rng(44)
    lo = np.stack(np.meshgrid(np.arange(0, 6), np.arange(0, 6), np.arange(0, 3), indexing="ij"), -1).reshape(-1, 3)
    hi = 65535 - lo
    mid = np.array([[65535, 0, 7], [0, 65535, 7], [32768, 32768, 32768]])
    pts = np.concatenate([lo, hi, mid]).astype(np.int32)
    pts = np.concatenate([pts, np.zeros((len(pts), 1), np.int32)], 1)[rng.permutation(len(pts))]
    f = rng.normal(size=(len(pts), 16)).astype(np.float32)
    size = torch.LongTensor([65536] * 3)
    m = SCN.Metadata_3()
    feats = torch.empty(0, device="cuda")
    SCN.InputLayer_updateOutput(m, size, torch.from_numpy(pts.astype(np.int64)), torch.from_numpy(f).cuda(), feats, 0, 0)
    W = (rng.normal(size=(27, 16, 16)) * 0.1).astype(np.float32)
    out = torch.empty(0, device="cuda")
    SCN.SubmanifoldConvolution_updateOutput(size, torch.LongTensor([3, 3, 3]), m, feats, out,
                                            torch.from_numpy(W).cuda(), torch.Tensor(), 1)
    nbr, counts, pairs = orc.ssc_rules(pts)
    assert (m.ssc_rulebook(size).nbr.t[:len(pts)].cpu().numpy() == nbr).all()
    ref, _ = orc.conv_forward(f, W, None, pairs, counts, len(pts))
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=1e-4, atol=1e-5)
    # the stride-2 scale of the corner voxels
    out2 = torch.empty(0, device="cuda")
    W2 = (rng.normal(size=(8, 16, 16)) * 0.2).astype(np.float32)
    SCN.Convolution_updateOutput(size, torch.LongTensor([32768] * 3), torch.LongTensor([2] * 3),
                                 torch.LongTensor([2] * 3), m, feats, out2, torch.from_numpy(W2).cuda(), torch.Tensor())
    parent, off, cc = orc.down2_rules(pts)
    c2, p2 = orc.down2_pairs(parent, off)
    ref2, _ = orc.conv_forward(f, W2, None, p2, c2, len(cc))
    np.testing.assert_allclose(out2.cpu().numpy(), ref2, rtol=1e-4, atol=1e-5)


def test_empty_and_duplicate_only_increments():
    """An increment of zero points, one that only repeats points already seen, and one that only
    re-observes old voxels with new colours: the executor must stay equal to a full forward."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    vox, rgb = _scene(45)
    model = NaiveUNet(m=16, levels=4, seed=14).cuda()
    ref_model = copy.deepcopy(model)
    net = scn.compile(model.sparseModel, capacity_sites=8192)
    n0 = 3500
    with torch.no_grad():
        base = net(_inp(vox[:n0], rgb[:n0]), increment=False)
        out = net(_inp(vox[:0], rgb[:0]), increment=True, all_points=True)
        assert torch.equal(out, base)
        assert net(_inp(vox[:0], rgb[:0]), increment=True).shape == (0, 16)
        # the same points again: means unchanged, no new sites
        out = net(_inp(vox[:500], rgb[:500]), increment=True, all_points=True)
        allp, allf = np.concatenate([vox[:n0], vox[:500]]), np.concatenate([rgb[:n0], rgb[:500]])
        assert torch.equal(out, ref_model.sparseModel(_inp(allp, allf)))
        assert net.sites_per_level()[0] == n0
        # old voxels, new colours
        rng = np.random.default_rng(46)
        idx = rng.integers(0, n0, 300)
        f2 = rng.uniform(0, 1, (300, 3)).astype(np.float32)
        out = net(_inp(vox[idx], f2), increment=True, all_points=True)
        allp, allf = np.concatenate([allp, vox[idx]]), np.concatenate([allf, f2])
        assert torch.equal(out, ref_model.sparseModel(_inp(allp, allf)))
        # and finally new voxels
        out = net(_inp(vox[n0:], rgb[n0:]), increment=True, all_points=True)
        allp, allf = np.concatenate([allp, vox[n0:]]), np.concatenate([allf, rgb[n0:]])
        assert torch.equal(out, ref_model.sparseModel(_inp(allp, allf)))


def test_residual_frames_disjoint_from_and_inside_the_saved_scene():
    """A residual frame far away from the saved scene is a plain forward over its own points; one
    made only of saved voxels with unchanged colours has residual zero, so it returns the saved
    rows."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    vox, rgb = _scene(47)
    model = NaiveUNet(m=16, levels=4, seed=15).cuda()
    ref_model = copy.deepcopy(model)
    net = scn.compile(model.sparseModel, capacity_sites=8192, residual=True)
    far = vox[:1500].copy()
    far[:, :3] += 1500
    with torch.no_grad():
        saved = net(_inp(vox, rgb), increment=False)
        got = net(_inp(far, rgb[:1500]), increment="residual")
        alone = ref_model.sparseModel(_inp(far, rgb[:1500]))
        # (not the same bits: a residual frame's convolutions use the launch shape for small row
        # counts, which adds the terms of a row in another order)
        parity.check("residual frame away from the saved scene vs plain forward", got.cpu().numpy(), alone.cpu().numpy())
        # saved voxels, same colours, one point per voxel: mean unchanged -> residual 0
        idx = np.random.default_rng(48).permutation(len(vox))[:1200]
        got = net(_inp(vox[idx], rgb[idx]), increment="residual")
    np.testing.assert_allclose(got.cpu().numpy(), saved[idx].cpu().numpy(), rtol=0, atol=2e-5)


def test_a_frame_with_a_bad_coordinate_is_dropped_whole():
    """One coordinate outside the representable range: the executor and the module tree reject the
    frame and keep the state of the previous frame, so that the next valid frame still equals a
    full forward over the valid points; after a full frame that fails, an incremental frame is
    refused until a full frame succeeded."""
    import sparseconvnet as scn
    from sparseconvnet._lib import InscError
    from workloads.netdefs import NaiveUNet

    vox, rgb = _scene(49)
    model = NaiveUNet(m=16, levels=4, seed=16).cuda()
    ref_model = copy.deepcopy(model)
    mod_model = copy.deepcopy(model)
    for mod in mod_model.modules():
        if isinstance(mod, scn.OutputLayer):
            mod.all_points = True
    net = scn.compile(model.sparseModel, capacity_sites=8192)
    n0, n1 = 3000, 4000
    bad = vox[n0:n1].copy()
    bad[17, 1] = 70000
    neg = vox[n0:n1].copy()
    neg[3, 2] = -1
    with torch.no_grad():
        net(_inp(vox[:n0], rgb[:n0]), increment=False)
        mod_model.sparseModel(_inp(vox[:n0], rgb[:n0]), False)
        for frame in (bad, neg):
            with pytest.raises(InscError) as e:
                net(_inp(frame, rgb[n0:n1]), increment=True)
            assert e.value.code == -5
            with pytest.raises(InscError):
                mod_model.sparseModel(_inp(frame, rgb[n0:n1]), True)
        assert net.sites_per_level()[0] == n0
        out = net(_inp(vox[n0:], rgb[n0:]), increment=True, all_points=True)
        out_mod = mod_model.sparseModel(_inp(vox[n0:], rgb[n0:]), True)
        ref = ref_model.sparseModel(_inp(vox, rgb))
        assert torch.equal(out, ref)
        assert torch.equal(out_mod, ref)
        # a full frame that fails leaves no state behind
        with pytest.raises(InscError):
            net(_inp(bad, rgb[n0:n1]), increment=False)
        with pytest.raises(InscError) as e:
            net(_inp(vox[:10], rgb[:10]), increment=True)
        assert e.value.code == -4
        assert torch.equal(net(_inp(vox, rgb), increment=False), ref)


def test_frames_of_more_than_16k_points_full_incremental_and_dropped():
    """Frames beyond 16 384 points rank their new cells with a device-wide prefix sum instead of one
    workgroup per scale: a full frame and an incremental frame of that size (the latter with points
    that fall on old cells, on new cells, and twice on the same new cell) must equal the module tree
    bit for bit, and such a frame with one bad coordinate must leave nothing behind."""
    import sparseconvnet as scn
    from sparseconvnet._lib import InscError
    from workloads.netdefs import NaiveUNet

    vox = scenes.indoor_scene(seed=51, n=60000, dims=(200, 160, 60), n_boxes=12, side_rng=(10, 40))
    rng = np.random.default_rng(51)
    rgb = rng.uniform(0, 1, (len(vox), 3)).astype(np.float32)
    n0 = 30000
    # second frame: 30k new voxels, 3k of the old ones again, 2k of the new ones twice
    idx = np.concatenate([np.arange(n0, len(vox)), rng.integers(0, n0, 3000), rng.integers(n0, len(vox), 2000)])
    idx = idx[rng.permutation(len(idx))]
    p1, f1 = vox[idx], rng.uniform(0, 1, (len(idx), 3)).astype(np.float32)
    assert n0 > 16384 and len(p1) > 16384
    model = NaiveUNet(m=16, levels=5, seed=17).cuda()
    mod_model = copy.deepcopy(model)
    for mod in mod_model.modules():
        if isinstance(mod, scn.OutputLayer):
            mod.all_points = True
    net = scn.compile(model.sparseModel, capacity_sites=1 << 16)
    with torch.no_grad():
        a = net(_inp(vox[:n0], rgb[:n0]), increment=False)
        b = mod_model.sparseModel(_inp(vox[:n0], rgb[:n0]), False)
        assert torch.equal(a, b)
        bad = p1.copy()
        bad[12345, 0] = 1 << 20
        with pytest.raises(InscError) as e:
            net(_inp(bad, f1), increment=True)
        assert e.value.code == -5
        assert net.sites_per_level()[0] == n0
        a = net(_inp(p1, f1), increment=True, all_points=True)
        b = mod_model.sparseModel(_inp(p1, f1), True)
        assert torch.equal(a, b)
        assert net.sites_per_level()[0] == len(vox)
        # and against a full forward over all points (the mean of a voxel's points is formed in row order)
        pts_all, f_all = np.concatenate([vox[:n0], p1]), np.concatenate([rgb[:n0], f1])
        full = copy.deepcopy(model).sparseModel(_inp(pts_all, f_all))
        assert torch.equal(a, full)
        # a full frame of that size that fails leaves no state behind; the next full frame is sound
        with pytest.raises(InscError) as e:
            net(_inp(bad, f1), increment=False)
        assert e.value.code == -5
        with pytest.raises(InscError) as e:
            net(_inp(vox[:10], rgb[:10]), increment=True)
        assert e.value.code == -4
        assert torch.equal(net(_inp(pts_all, f_all), increment=False), full)


def test_grid_reports_a_bad_coordinate_once_and_stays_usable():
    import ctypes

    from sparseconvnet._lib import InscError, ensure_init, lib, ptr, stream_ptr

    ensure_init(0)
    I64 = ctypes.c_int64
    g = ctypes.c_void_p()
    lib.insc_grid_create(I64(4096), ctypes.byref(g))
    c = torch.tensor([[1, 2, 3, 0], [70000, 0, 0, 0], [4, 5, 6, 0], [1, 2, 3, 0]], dtype=torch.int32, device="cuda")
    sop = torch.empty(4, dtype=torch.int32, device="cuda")
    n = I64(0)
    with pytest.raises(InscError) as e:
        lib.insc_grid_insert(g, ptr(c), I64(4), ptr(sop), ctypes.byref(n), stream_ptr())
    assert e.value.code == -5
    assert sop.tolist() == [0, -1, 1, 0]
    c2 = torch.tensor([[9, 9, 9, 0], [4, 5, 6, 0]], dtype=torch.int32, device="cuda")
    lib.insc_grid_insert(g, ptr(c2), I64(2), ptr(sop), ctypes.byref(n), stream_ptr())
    assert n.value == 3 and sop[:2].tolist() == [2, 1]
    lib.insc_grid_destroy(g)
