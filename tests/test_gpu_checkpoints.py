"""Checkpoints and weights trained elsewhere, through the HIP path: a state_dict saved with
checkpoint_save and restored into a fresh model on the GPU gives the same bits (module tree and
network executor, which must notice that the parameters moved); a state_dict whose 3^3 filters
follow the z-major offset numbering of the reference's CPU rule generator
(Metadata/SubmanifoldConvolutionRules.h:39-52), converted with convert_zmajor_state_dict, gives on
the HIP path what the oracle gives with the original weights on z-major rules (1e-4 / 1e-5)."""
import copy

import numpy as np
import pytest
import torch

import parity

from workloads import scenes

pytestmark = pytest.mark.gpu


def _scene(n, seed):
    vox = scenes.indoor_scene(seed=seed, n=n, dims=(60, 50, 24), n_boxes=6, side_rng=(6, 16))
    rng = np.random.default_rng(seed)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), len(vox) // 10)]], 0)
    pts = pts[rng.permutation(len(pts))]
    return pts, rng.uniform(0, 1, (len(pts), 3)).astype(np.float32)


def _inp(pts, rgb):
    return [torch.from_numpy(pts[:, :3].astype(np.int64)), torch.from_numpy(rgb).cuda(), 1]


def test_checkpoint_round_trip_through_the_hip_path(tmp_path):
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    pts, rgb = _scene(6000, seed=51)
    src = NaiveUNet(m=16, levels=4, seed=3).cuda()
    dst = NaiveUNet(m=16, levels=4, seed=99).cuda()  # other weights, other batch-norm statistics
    net = scn.compile(dst.sparseModel, capacity_sites=8192)
    with torch.no_grad():
        want = src(_inp(pts, rgb)).clone()
        before = dst(_inp(pts, rgb)).clone()
        net_before = dst.linear(net(_inp(pts, rgb), increment=False)).clone()
    assert not torch.equal(want, before)
    assert torch.equal(before, net_before)
    exp = str(tmp_path / "run")
    scn.checkpoint_save(src, exp, "unet", 7, use_cuda=True)
    assert scn.checkpoint_restore(dst, exp, "unet", use_cuda=True) == 8  # model.cpu() ... model.cuda(): new storage
    with torch.no_grad():
        after = dst(_inp(pts, rgb))
        net_after = dst.linear(net(_inp(pts, rgb), increment=False))  # the executor follows the moved parameters
    assert torch.equal(after, want)
    assert torch.equal(net_after, want)
    # new values in the same storage (load_state_dict copies in place): noticed as well
    with torch.no_grad():
        dst.load_state_dict(NaiveUNet(m=16, levels=4, seed=5).state_dict())
        again = dst(_inp(pts, rgb))
        net_again = dst.linear(net(_inp(pts, rgb), increment=False))
    assert not torch.equal(again, want)
    assert torch.equal(net_again, again)


def test_incremental_frame_after_a_reload_is_refused():
    """Rows cached by earlier frames were computed with the old parameters.  After the parameters
    change - all of them (load_state_dict) or a single tensor in the middle of the network (copy_) -
    an incremental frame must not mix old and new rows: the executor raises until a full frame has
    run, and that full frame plus an increment equals a full forward with the new parameters."""
    import sparseconvnet as scn
    from sparseconvnet._lib import InscError
    from workloads.netdefs import NaiveUNet

    pts, rgb = _scene(5000, seed=52)
    a, b = (pts[:4000], rgb[:4000]), (pts[4000:], rgb[4000:])
    model = NaiveUNet(m=16, levels=3, seed=3).cuda()
    net = scn.compile(model.sparseModel, capacity_sites=8192)

    def change_all():
        model.load_state_dict(NaiveUNet(m=16, levels=3, seed=5).state_dict())

    def change_one():
        convs = [m for m in model.modules() if isinstance(m, scn.SubmanifoldConvolution)]
        mid = convs[len(convs) // 2]  # neither the first nor the last op with parameters
        mid.weight.copy_(mid.weight * 1.5)

    for change in (change_all, change_one):
        with torch.no_grad():
            net(_inp(*a), increment=False)
            net(_inp(*b), increment=True)  # fine: state and parameters agree
            change()
            with pytest.raises(RuntimeError) as err:  # noticed by the wrapper ...
                net(_inp(*b), increment=True)
            assert "full frame" in str(err.value)
            with pytest.raises(InscError) as err:  # ... and the library has dropped its cached rows
                net(_inp(*b), increment=True)
            assert "full frame" in str(err.value)
            net(_inp(*a), increment=False)
            got = net(_inp(*b), increment=True, all_points=True)
            want = model.sparseModel(_inp(pts, rgb))
        assert torch.equal(got, want)


def test_zmajor_weights_through_the_hip_path():
    """Weights trained against the z-major offset numbering: the oracle runs the ORIGINAL weights on
    z-major rules; the HIP path runs the converted state_dict."""
    import sparseconvnet as scn
    from oracle import oracle as orc
    from oracle import oracle_net
    from workloads.netdefs import NaiveUNet

    pts, rgb = _scene(5000, seed=52)
    zmodel = NaiveUNet(m=16, levels=3, seed=6)  # stands for a model trained elsewhere, z-major filters
    hip = NaiveUNet(m=16, levels=3, seed=1)
    hip.load_state_dict(scn.convert_zmajor_state_dict(zmodel.state_dict()))
    hip = hip.cuda()
    net = scn.compile(hip.sparseModel, capacity_sites=8192)
    with torch.no_grad():
        feats = hip.sparseModel(_inp(pts, rgb))
        feats_net = net(_inp(pts, rgb), increment=False)
    assert torch.equal(feats, feats_net)
    real = orc.ssc_rules
    try:
        orc.ssc_rules = lambda sc, zmajor=False: real(sc, zmajor=True)
        ref = oracle_net.forward(zmodel.sparseModel, [pts, rgb, 1])
    finally:
        orc.ssc_rules = real
    plain = oracle_net.forward(zmodel.sparseModel, [pts, rgb, 1])
    assert np.abs(plain - ref).max() > 1e-2, "the two numberings must differ for unconverted weights"
    parity.check("converted z-major checkpoint, 3-level U-Net", feats.cpu().numpy(), ref)
