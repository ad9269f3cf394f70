"""Pins the whole-network oracle (oracle/oracle_net.py walking the module tree, and with it the
wiring of the UNet builder) against a dense-grid PyTorch model written by hand from the
reference's architecture text (sparseconvnet/networkArchitectures.py:202-300 with residual
blocks, model.py:8-26): conv3d / conv_transpose3d / per-channel affine on [1, C, G, G, G] float64
volumes with activity masks (a site is active at a coarse scale iff one of its eight children
is).  The dense model takes its parameters from the module tree in registration order, which is
also the order this hand-written forward consumes them in; a block wired differently, a skip
joined on the wrong side or a scale's mask handled differently shows as a mismatch.

Tolerance 1e-4 relative / 1e-5 absolute times the output's scale (float32 oracle against a
float64 library result through ~30 layers)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

G = 32


class _Params(object):
    """Hands out the layers of the sparse model in registration order, by kind."""

    def __init__(self, sparse_model):
        import sparseconvnet as scn

        self.q = {"ssc": [], "conv": [], "deconv": [], "nin": [], "bn": []}
        for m in sparse_model.modules():
            if isinstance(m, scn.SubmanifoldConvolution):
                self.q["ssc"].append(m)
            elif isinstance(m, scn.Convolution):
                self.q["conv"].append(m)
            elif isinstance(m, scn.Deconvolution):
                self.q["deconv"].append(m)
            elif isinstance(m, scn.NetworkInNetwork):
                self.q["nin"].append(m)
            elif isinstance(m, scn.BatchNormalization):
                self.q["bn"].append(m)

    def take(self, kind):
        return self.q[kind].pop(0)

    def empty(self):
        return all(len(v) == 0 for v in self.q.values())


def _t(x):
    return x.detach().double()


def _ssc(p, x, mask):
    m = p.take("ssc")
    nin, nout = m.nIn, m.nOut
    w = _t(m.weight).reshape(3, 3, 3, nin, nout).permute(4, 3, 0, 1, 2)
    assert x.shape[1] == nin
    return F.conv3d(x, w, padding=1) * mask


def _bnrelu(p, x, mask):
    m = p.take("bn")
    assert x.shape[1] == m.nPlanes and m.leakiness == 0
    w = _t(m.weight) / torch.sqrt(_t(m.running_var) + m.eps)
    b = _t(m.bias) - _t(m.running_mean) * w
    return torch.relu(x * w.view(1, -1, 1, 1, 1) + b.view(1, -1, 1, 1, 1)) * mask


def _block(p, x, mask, a, b):
    """Residual block a -> b: (identity | 1x1) + BNReLU-SSC-BNReLU-SSC."""
    assert x.shape[1] == a
    if a == b:
        skip = x
    else:
        m = p.take("nin")
        skip = torch.einsum("bcxyz,co->boxyz", x, _t(m.weight)) * mask
    # registration order inside the ConcatTable: the skip branch first, then BN, SSC, BN, SSC
    y = _ssc(p, _bnrelu(p, x, mask), mask)
    y = _ssc(p, _bnrelu(p, y, mask), mask)
    return skip + y


def _U(p, x, masks, level, planes, reps):
    n0 = planes[0]
    for _ in range(reps):
        x = _block(p, x, masks[level], x.shape[1], n0)
    if len(planes) > 1:
        y = _bnrelu(p, x, masks[level])
        m = p.take("conv")
        w = _t(m.weight).reshape(2, 2, 2, m.nIn, m.nOut).permute(4, 3, 0, 1, 2)
        y = F.conv3d(y, w, stride=2) * masks[level + 1]
        y = _U(p, y, masks, level + 1, planes[1:], reps)
        y = _bnrelu(p, y, masks[level + 1])
        m = p.take("deconv")
        w = _t(m.weight).reshape(2, 2, 2, m.nIn, m.nOut).permute(3, 4, 0, 1, 2)
        y = F.conv_transpose3d(y, w, stride=2) * masks[level]
        x = torch.cat([x, y], 1)
        for i in range(reps):
            x = _block(p, x, masks[level], n0 * (2 if i == 0 else 1), n0)
    return x


@pytest.mark.parametrize("levels,m", [(3, 4), (4, 3)])
def test_oracle_network_vs_dense_torch_model(levels, m):
    from oracle import oracle_net
    from workloads import scenes
    from workloads.netdefs import NaiveUNet

    vox = scenes.boxes_scene(seed=21, n=2500, grid=G, n_boxes=3, lo_rng=(2, 12), size_rng=(8, 18))
    rng = np.random.default_rng(22)
    dup = vox[rng.integers(0, len(vox), 300)]
    pts = np.concatenate([vox, dup])[rng.permutation(len(vox) + 300)]
    rgb = rng.uniform(0, 1, (len(pts), 3)).astype(np.float32)
    model = NaiveUNet(m=m, levels=levels, full_scale=G, seed=6)
    out = oracle_net.forward(model.sparseModel, [pts[:, :3], rgb, 1])

    # dense model: per-voxel mean of the input rows (InputLayer mode 4) ...
    c = torch.from_numpy(pts[:, :3].astype(np.int64))
    s = torch.zeros(1, 3, G, G, G, dtype=torch.float64)
    cnt = torch.zeros(1, 1, G, G, G, dtype=torch.float64)
    s.index_put_((torch.zeros(len(c), dtype=torch.long).unsqueeze(1).expand(-1, 3), torch.arange(3).expand(len(c), -1),
                  c[:, 0:1].expand(-1, 3), c[:, 1:2].expand(-1, 3), c[:, 2:3].expand(-1, 3)),
                 torch.from_numpy(rgb.astype(np.float64)), accumulate=True)
    cnt.index_put_((torch.zeros(len(c), dtype=torch.long), torch.zeros(len(c), dtype=torch.long), c[:, 0], c[:, 1],
                    c[:, 2]), torch.ones(len(c), dtype=torch.float64), accumulate=True)
    masks = [(cnt > 0).double()]
    for _ in range(levels - 1):
        masks.append(F.max_pool3d(masks[-1], 2))
    x = s / cnt.clamp(min=1)
    # ... stem convolution, the U-Net, BN+ReLU, one row per input point (model.py:8-26)
    p = _Params(model.sparseModel)
    x = _ssc(p, x, masks[0])
    x = _U(p, x, masks, 0, [m * (i + 1) for i in range(levels)], 2)
    x = _bnrelu(p, x, masks[0])
    assert p.empty(), "the dense model did not consume every layer of the module tree"
    ref = x[0, :, c[:, 0], c[:, 1], c[:, 2]].t().numpy()
    assert out.shape == ref.shape == (len(pts), m)
    scale = max(1.0, float(np.abs(ref).max()))
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-5 * scale)
    assert np.abs(ref).max() > 0.1
