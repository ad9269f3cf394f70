"""Whole-network parity: the U-Net of the reference's example (model.py) on the HIP path
against the same module tree evaluated with the CPU oracle."""
import numpy as np
import pytest
import torch

import parity
from workloads import scenes

pytestmark = pytest.mark.gpu


def _scene(n, seed, dup=0.1):
    vox = scenes.indoor_scene(seed=seed, n=n, dims=(60, 50, 24), n_boxes=6, side_rng=(6, 16))
    rng = np.random.default_rng(seed)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), int(dup * len(vox)))]], 0)
    pts = pts[rng.permutation(len(pts))]
    rgb = rng.uniform(0, 1, (len(pts), 3)).astype(np.float32)
    return pts, rgb




@pytest.mark.parametrize("levels,m", [(3, 16), (7, 32)])
def test_unet_full_forward_matches_oracle(orc, levels, m):
    from oracle import oracle_net
    from workloads.netdefs import NaiveUNet

    pts, rgb = _scene(6000, seed=11)
    model = NaiveUNet(m=m, levels=levels, seed=4).cuda()
    coords = torch.from_numpy(pts[:, :3].astype(np.int64))
    with torch.no_grad():
        feats = model.sparseModel([coords, torch.from_numpy(rgb).cuda(), 1])
        logits = model.linear(feats)
    ref_feats = oracle_net.forward(model.sparseModel, [pts, rgb, 1])
    with orc.double_precision():
        ref64 = oracle_net.forward(model.sparseModel, [pts, rgb, 1])
    assert feats.shape == ref_feats.shape == (len(pts), m)
    parity.check("U-Net features, %d levels, m=%d, 6000 voxels" % (levels, m), feats.cpu().numpy(), ref_feats, ref64)
    w, b = model.linear.weight.detach().cpu().numpy(), model.linear.bias.detach().cpu().numpy()
    parity.check("logits, %d levels" % levels, logits.cpu().numpy(), ref_feats @ w.T + b,
                 ref64 @ w.T.astype(np.float64) + b)


def test_unet_is_deterministic():
    from workloads.netdefs import NaiveUNet

    pts, rgb = _scene(5000, seed=12)
    model = NaiveUNet(m=16, levels=4, seed=5).cuda()
    coords = torch.from_numpy(pts[:, :3].astype(np.int64))
    with torch.no_grad():
        a = model([coords, torch.from_numpy(rgb).cuda(), 1]).clone()
        b = model([coords, torch.from_numpy(rgb).cuda(), 1])
    assert torch.equal(a, b)  # no float atomics anywhere on the path
