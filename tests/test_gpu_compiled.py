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
