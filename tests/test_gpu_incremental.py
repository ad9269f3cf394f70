"""Incremental forward == full recompute.

Frame 0 is a full forward; each later frame appends new surface voxels and re-observes some
old ones (which changes their mean colour).  After every incremental frame the logits of ALL
points seen so far must equal a full forward over the concatenated point list.  Because a
row's result does not depend on which rows share its tile and nothing on the path uses float
atomics, the match is bit-exact, which is stronger than the stated 1e-4 / 1e-5 tolerance."""
import copy

import numpy as np
import pytest
import torch

from workloads import scenes

pytestmark = pytest.mark.gpu


def _frames(n_frames, seed):
    vox = scenes.indoor_scene(seed=seed, n=9000, dims=(70, 60, 24), n_boxes=6, side_rng=(6, 16))
    rng = np.random.default_rng(seed)
    pose = vox[:, :3].min(0).astype(np.float64)
    order = np.argsort(np.linalg.norm(vox[:, :3] - pose, axis=1), kind="stable")
    base = rng.uniform(0, 1, (len(vox), 3)).astype(np.float32)
    n0 = len(vox) // 3
    step = (len(vox) - n0) // (n_frames - 1)
    out = [(vox[order[:n0]], base[order[:n0]])]
    seen = n0
    for f in range(1, n_frames):
        new = order[seen:seen + step]
        old = order[rng.integers(0, seen, 150)]
        idx = np.concatenate([new, old])
        rgb = base[idx].copy()
        rgb[len(new):] += rng.uniform(-0.1, 0.1, (len(old), 3)).astype(np.float32)
        perm = rng.permutation(len(idx))
        out.append((vox[idx][perm], rgb[perm]))
        seen += step
    return out


def _inp(pts, rgb):
    return [torch.from_numpy(pts[:, :3].astype(np.int64)), torch.from_numpy(rgb).cuda(), 1]


@pytest.mark.parametrize("levels,m", [(3, 16), (5, 32)])
def test_incremental_equals_full_recompute(levels, m):
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    frames = _frames(5, seed=21)
    model = NaiveUNet(m=m, levels=levels, seed=7).cuda()
    ref_model = copy.deepcopy(model)
    for mod in model.modules():
        if isinstance(mod, scn.OutputLayer):
            mod.all_points = True
    all_pts, all_rgb = frames[0]
    with torch.no_grad():
        out = model(_inp(*frames[0]), increment=False)
        ref = ref_model(_inp(all_pts, all_rgb), increment=False)
        assert torch.equal(out, ref)
        for f in range(1, len(frames)):
            pts, rgb = frames[f]
            out = model(_inp(pts, rgb), increment=True)
            all_pts = np.concatenate([all_pts, pts], 0)
            all_rgb = np.concatenate([all_rgb, rgb], 0)
            ref = ref_model(_inp(all_pts, all_rgb), increment=False)
            assert out.shape == ref.shape == (len(all_pts), 20)
            err = (out - ref).abs().max().item()
            assert torch.equal(out, ref), "frame %d: max |incremental - full| = %.3e" % (f, err)


def test_incremental_default_output_is_the_increment_rows():
    from workloads.netdefs import NaiveUNet

    frames = _frames(3, seed=22)
    model = NaiveUNet(m=16, levels=3, seed=8).cuda()
    ref_model = copy.deepcopy(model)
    with torch.no_grad():
        model(_inp(*frames[0]), increment=False)
        out = model(_inp(*frames[1]), increment=True)
        all_pts = np.concatenate([frames[0][0], frames[1][0]], 0)
        all_rgb = np.concatenate([frames[0][1], frames[1][1]], 0)
        ref = ref_model(_inp(all_pts, all_rgb), increment=False)
    assert out.shape == (len(frames[1][0]), 20)
    assert torch.equal(out, ref[len(frames[0][0]):])


def test_dirty_sets_stay_local_at_fine_levels():
    """One new voxel far from everything else: the dirty set of the first layers is tiny."""
    import sparseconvnet as scn
    from sparseconvnet import incremental

    pts, rgb = _frames(2, seed=23)[0]
    size = torch.LongTensor([4096] * 3)
    inp = scn.InputLayer(3, size, mode=4)
    conv = scn.SubmanifoldConvolution(3, 3, 16, 3, False).cuda()
    with torch.no_grad():
        x = inp(_inp(pts, rgb))
        y = conv(x)
        one = pts[:1].copy()
        one[0, :3] = pts[0, :3]  # re-observe an existing voxel
        x2 = inp(_inp(one, rgb[:1] * 0.5), increment=True)
        assert x2.dirty.count() == 1
        y2 = conv(x2, increment=True)
        k = y2.dirty.count()
        assert 1 <= k <= 27
    sc = x2.metadata.scale(size)
    nbr = sc.nbr.t[:sc.n].cpu().numpy()
    site = int(x2.metadata.site_of_point[0].item())
    assert k == int((nbr[site] >= 0).sum())
