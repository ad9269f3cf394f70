"""Whole-network parity: the U-Net of the reference's example (model.py) on the HIP path
against the same module tree evaluated with the CPU oracle."""
import numpy as np
import pytest
import torch

from workloads import scenes

pytestmark = pytest.mark.gpu


def _scene(n, seed, dup=0.1):
    vox = scenes.indoor_scene(seed=seed, n=n, dims=(60, 50, 24), n_boxes=6, side_rng=(6, 16))
    rng = np.random.default_rng(seed)
    pts = np.concatenate([vox, vox[rng.integers(0, len(vox), int(dup * len(vox)))]], 0)
    pts = pts[rng.permutation(len(pts))]
    rgb = rng.uniform(0, 1, (len(pts), 3)).astype(np.float32)
    return pts, rgb


def _check(a, b, what):
    """1e-4 relative / 1e-5 absolute, the tolerance stated for float32 outputs; for a deep
    network the absolute term is taken relative to the tensor's scale (max |value|)."""
    scale = max(1.0, float(np.abs(b).max()))
    err = np.abs(a - b)
    tol = 1e-5 * scale + 1e-4 * np.abs(b)
    assert (err <= tol).all(), "%s: max err %.3e (scale %.3e), worst excess %.3e" % (
        what, err.max(), scale, (err - tol).max())


@pytest.mark.parametrize("levels,m", [(3, 16), (7, 32)])
def test_unet_full_forward_matches_oracle(levels, m):
    from oracle import oracle_net
    from workloads.netdefs import NaiveUNet

    pts, rgb = _scene(6000, seed=11)
    model = NaiveUNet(m=m, levels=levels, seed=4).cuda()
    coords = torch.from_numpy(pts[:, :3].astype(np.int64))
    with torch.no_grad():
        feats = model.sparseModel([coords, torch.from_numpy(rgb).cuda(), 1])
        logits = model.linear(feats)
    ref_feats = oracle_net.forward(model.sparseModel, [pts, rgb, 1])
    assert feats.shape == ref_feats.shape == (len(pts), m)
    _check(feats.cpu().numpy(), ref_feats, "U-Net features")
    w, b = model.linear.weight.detach().cpu().numpy(), model.linear.bias.detach().cpu().numpy()
    _check(logits.cpu().numpy(), ref_feats @ w.T + b, "logits")


def test_unet_is_deterministic():
    from workloads.netdefs import NaiveUNet

    pts, rgb = _scene(5000, seed=12)
    model = NaiveUNet(m=16, levels=4, seed=5).cuda()
    coords = torch.from_numpy(pts[:, :3].astype(np.int64))
    with torch.no_grad():
        a = model([coords, torch.from_numpy(rgb).cuda(), 1]).clone()
        b = model([coords, torch.from_numpy(rgb).cuda(), 1])
    assert torch.equal(a, b)  # no float atomics anywhere on the path
