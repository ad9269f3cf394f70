"""The native network executor (one C call per frame) against the per-layer module path:
bit-identical outputs for full frames, incremental frames, and full recomputes."""
import copy

import numpy as np
import pytest
import torch

from test_gpu_incremental import _frames, _inp

pytestmark = pytest.mark.gpu


@pytest.fixture(params=[(512, 896, 4096, 2000), (1, 1 << 40, 4096, 1 << 40), (512, 1, 4096, 2000), (512, 896, 1, 2000),
                        (512, 1 << 40, 4096, 1)],
                ids=["default-launch-policy", "persistent-kernel-forced", "shared-weights-kernel-forced",
                     "filter-in-lds-kernel-forced", "wavefront-per-unit-kernel-forced"])
def persistent_min_units(request):
    """The 3^3 layers of these small scenes stay below the thresholds of the three persistent
    kernels; the second, third and fifth run force the wide layers onto one of them, the fourth the
    narrow layers (at most 32 channels) onto the kernel that keeps its filter in LDS - each with the
    fused batch norm / residual epilogues and the dirty-tile flags of the executor."""
    from sparseconvnet._lib import lib

    lib.insc_conv_set_persistent_min_units(request.param[0])
    lib.insc_conv_set_shared_weights_min_units(request.param[1])
    lib.insc_conv_set_filter_lds_min_tiles(request.param[2])
    lib.insc_conv_set_wavefront_per_unit_min_units(request.param[3])
    yield request.param
    lib.insc_conv_set_persistent_min_units((1 << 63) - 1)
    lib.insc_conv_set_shared_weights_min_units(896)
    lib.insc_conv_set_filter_lds_min_tiles(4096)
    lib.insc_conv_set_wavefront_per_unit_min_units(2400)


@pytest.mark.parametrize("levels,m", [(3, 16), (7, 32)])
def test_compiled_full_and_incremental(levels, m, persistent_min_units):
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    frames = _frames(6, seed=31)
    model = NaiveUNet(m=m, levels=levels, seed=9).cuda()
    ref_model = copy.deepcopy(model)
    net = scn.compile(model.sparseModel, capacity_sites=4096)  # small: forces growth on later frames
    all_pts, all_rgb = frames[0]
    with torch.no_grad():
        out = net(_inp(*frames[0]), increment=False)
        ref = ref_model.sparseModel(_inp(all_pts, all_rgb), False)
        assert out.shape == ref.shape
        assert torch.equal(out, ref)
        for f in range(1, len(frames)):
            pts, rgb = frames[f]
            out = net(_inp(pts, rgb), increment=True, all_points=True)
            inc = net  # keep name for the error message below
            all_pts = np.concatenate([all_pts, pts], 0)
            all_rgb = np.concatenate([all_rgb, rgb], 0)
            ref = ref_model.sparseModel(_inp(all_pts, all_rgb), False)
            assert out.shape == ref.shape
            assert torch.equal(out, ref), "frame %d: max diff %.3e" % (f, (out - ref).abs().max().item())
        # increment rows only
        pts, rgb = frames[1]
        out = net(_inp(pts, rgb), increment=True)
        all_pts = np.concatenate([all_pts, pts], 0)
        all_rgb = np.concatenate([all_rgb, rgb], 0)
        ref = ref_model.sparseModel(_inp(all_pts, all_rgb), False)
        assert torch.equal(out, ref[-len(pts):])
        # a new full frame forgets the scene
        out = net(_inp(*frames[2]), increment=False)
        ref = ref_model.sparseModel(_inp(*frames[2]), False)
        assert torch.equal(out, ref)


def test_compiled_rejects_incremental_without_state():
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet
    from sparseconvnet._lib import InscError

    model = NaiveUNet(m=16, levels=2, seed=1).cuda()
    net = scn.compile(model.sparseModel)
    pts, rgb = _frames(2, seed=32)[0]
    with pytest.raises(InscError):
        net(_inp(pts, rgb), increment=True)


def test_dirty_set_rows_of_a_frame():
    """The dirty sets the executor reports: the input's set is the frame's touched voxels, every
    derived set contains its source (sets only grow along the program), none exceeds its scale,
    and at the finest scale they stay a fraction of the scene for a local increment."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    frames = _frames(3, seed=33)
    model = NaiveUNet(m=16, levels=4, seed=2).cuda()
    net = scn.compile(model.sparseModel)
    with torch.no_grad():
        net(_inp(*frames[0]), increment=False)
        pts, rgb = frames[1]
        net(_inp(pts, rgb), increment=True)
    sets = net.dirty_rows()
    sites = net.sites_per_level()
    assert len(sets) == 4
    assert sets[0][0][0] == "input"
    touched = len(np.unique(np.asarray(pts)[:, :3], axis=0))
    assert sets[0][0][1] == touched
    for l, ss in enumerate(sets):
        assert ss, "scale %d has no dirty set" % l
        for kind, rows in ss:
            assert 0 < rows <= sites[l], (l, kind, rows, sites[l])
    rows0 = [r for _, r in sets[0]]
    assert min(rows0) == touched and max(rows0) >= touched
    # dilation by 3^3 layers grows a set; a frame here touches one end of the scene
    assert [r for k, r in sets[0] if k == "dilate"][0] > touched


def test_order_refresh_leaves_every_bit_alone():
    """An incremental frame that re-sorts the processing orders of its scales (the input scale of this
    sweep holds 37k..50k sites, so the appended share passes 1 % with every frame) gives the bits of one
    that keeps appending, and of a full forward over all points so far."""
    import sparseconvnet as scn
    from workloads import scenes
    from workloads.netdefs import NaiveUNet

    seq = scenes.sweep_sequence()[:6]
    model = NaiveUNet(m=32, levels=7, seed=5).cuda()
    nets = [scn.compile(copy.deepcopy(model).sparseModel, capacity_sites=60000) for _ in range(3)]
    nets[0].set_order_refresh(0)   # never
    nets[1].set_order_refresh(1)   # every frame
    nets[2].set_order_refresh(12)  # once or twice in this sequence
    all_p, all_c = seq[0]
    with torch.no_grad():
        outs = [n(_inp(*seq[0]), increment=False) for n in nets]
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
        for f in range(1, len(seq)):
            p, c = seq[f]
            outs = [n(_inp(p, c), increment=True, all_points=True) for n in nets]
            assert torch.equal(outs[0], outs[1]), "frame %d" % f
            assert torch.equal(outs[0], outs[2]), "frame %d" % f
            all_p = np.concatenate([all_p, p], 0)
            all_c = np.concatenate([all_c, c], 0)
        full = scn.compile(copy.deepcopy(model).sparseModel, capacity_sites=60000)(_inp(all_p, all_c), increment=False)
        assert torch.equal(outs[1], full)
        assert [int(v) for v in nets[1].sites_per_level()] == [int(v) for v in nets[0].sites_per_level()]


def test_whole_network_sequential_runs_through_the_executor_by_itself(auto_compile):
    """The reference's own loop, unchanged (model.py:23-26, demo.py:26-38): `model(x, increment=False)`
    then `model(x, increment=True)` on the module tree, coordinates as int64 on the host or on the
    GPU.  With the switch on, the whole-network Sequential traces itself at the first frame; the
    outputs equal the layer-by-layer path bit for bit."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    frames = _frames(4, seed=35)
    model = NaiveUNet(m=16, levels=4, seed=9).cuda()
    ref_model = copy.deepcopy(model)
    assert scn.get_auto_compile()
    with torch.no_grad():
        out = model(_inp(*frames[0]), increment=False)
        assert model.sparseModel.__dict__["_exec"][0] is not None and model.sparseModel.why_not_compiled() is None
        scn.set_auto_compile(False)
        ref = ref_model(_inp(*frames[0]), increment=False)
        scn.set_auto_compile(True)
        assert torch.equal(out, ref)
        for f in range(1, len(frames)):
            pts, rgb = frames[f]
            x = _inp(pts, rgb)
            if f == 2:
                x[0] = x[0].cuda()  # int64 coordinates on the GPU, as in the reference's demo
            out = model(x, increment=True)
            scn.set_auto_compile(False)
            ref = ref_model(_inp(pts, rgb), increment=True)
            scn.set_auto_compile(True)
            assert out.shape == ref.shape == (len(pts), 20)
            assert torch.equal(out, ref), "frame %d" % f
    # a copy of the model traces its own executor
    twin = copy.deepcopy(model)
    assert "_exec" not in twin.sparseModel.__dict__
    with torch.no_grad():
        assert torch.equal(twin(_inp(*frames[0])), ref_model(_inp(*frames[0])))


def test_sequential_falls_back_to_the_layer_path(auto_compile):
    """Trees the tracer does not take run layer by layer, with the tracer's reason kept: here a
    ConcatTable of three branches joined by one JoinTable."""
    import sparseconvnet as scn

    torch.manual_seed(3)
    net = scn.Sequential().add(scn.InputLayer(3, 4096, mode=4)).add(
        scn.SubmanifoldConvolution(3, 3, 16, 3, False)).add(
        scn.ConcatTable().add(scn.Identity()).add(scn.SubmanifoldConvolution(3, 16, 16, 3, False)).add(
            scn.NetworkInNetwork(16, 16, False))).add(
        scn.JoinTable()).add(scn.BatchNormReLU(48)).add(scn.OutputLayer(3)).cuda().eval()
    pts, rgb = _frames(2, seed=36)[0]
    with torch.no_grad():
        out = net(_inp(pts, rgb))
        assert "JoinTable" in net.why_not_compiled()
        scn.set_auto_compile(False)
        ref = net(_inp(pts, rgb))
    assert out.shape == (len(pts), 48) and torch.equal(out, ref)


def test_sequential_residual_frames_through_the_executor(auto_compile):
    """With the reference's kind of incremental forward in force (set_incremental_mode("residual")),
    `model(x, increment=True)` is a residual frame; traced at the first frame, it equals the module
    tree's Incre_* operators bit for bit."""
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    frames = _frames(3, seed=37)
    model = NaiveUNet(m=16, levels=3, seed=9).cuda()
    ref_model = copy.deepcopy(model)
    scn.set_incremental_mode("residual")
    try:
        with torch.no_grad():
            model(_inp(*frames[0]), increment=False)
            got = model(_inp(*frames[1]), increment=True)
            assert model.sparseModel.__dict__["_exec"][0].residual
            scn.set_auto_compile(False)
            ref_model(_inp(*frames[0]), increment=False)
            ref = ref_model(_inp(*frames[1]), increment=True)
        assert torch.equal(got, ref)
    finally:
        scn.set_incremental_mode("exact")
    # an executor traced for exact frames says how to get residual ones
    scn.set_auto_compile(True)
    other = NaiveUNet(m=16, levels=3, seed=9).cuda()
    with torch.no_grad():
        other(_inp(*frames[0]), increment=False)
        with pytest.raises(RuntimeError, match="set_incremental_mode"):
            other(_inp(*frames[1]), increment="residual")
