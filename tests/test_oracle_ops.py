"""Pins the floating-point half of the CPU oracle against library routines: the rulebook
convolutions against dense torch conv3d / conv_transpose3d on a small grid (float64), the
batch norm against torch.nn.functional.batch_norm, the input/output layers against numpy
unique/bincount, NiN against a matmul.  A transposed weight, a wrong offset order, a
swapped rule role or a dropped eps all fail here.

Tolerance: the oracle computes in float32 like the reference; it is compared with a float64
library result at 1e-4 relative / 1e-5 absolute (the tolerance the north star states)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

RTOL, ATOL = 1e-4, 1e-5


def scene(seed, n, grid):
    rng = np.random.default_rng(seed)
    c = rng.integers(1, grid - 1, (n, 3)).astype(np.int32)
    return np.unique(c, axis=0)[rng.permutation(len(np.unique(c, axis=0)))]


def to_dense(coords, feats, grid):
    d = torch.zeros(1, feats.shape[1], grid, grid, grid, dtype=torch.float64)
    c = torch.from_numpy(coords.astype(np.int64))
    d[0, :, c[:, 0], c[:, 1], c[:, 2]] = torch.from_numpy(feats.astype(np.float64)).t()
    return d


def test_ssc_conv_vs_conv3d(orc):
    G, Cin, Cout = 16, 5, 7
    c = scene(0, 1500, G)
    rng = np.random.default_rng(1)
    x = rng.normal(size=(len(c), Cin)).astype(np.float32)
    W = rng.normal(size=(27, Cin, Cout)).astype(np.float32) * 0.2
    b = rng.normal(size=Cout).astype(np.float32)
    _, counts, pairs = orc.ssc_rules(c)
    y, flops = orc.conv_forward(x, W, b, pairs, counts, len(c))
    assert flops == len(pairs) * Cin * Cout
    # dense cross-correlation, dims ordered (x,y,z): w[co,ci,a,b,c] = W[a*9+b*3+c][ci][co]
    w = torch.from_numpy(W.astype(np.float64)).reshape(3, 3, 3, Cin, Cout).permute(4, 3, 0, 1, 2)
    d = F.conv3d(to_dense(c, x, G), w, bias=torch.from_numpy(b.astype(np.float64)), padding=1)
    ci = torch.from_numpy(c.astype(np.int64))
    ref = d[0, :, ci[:, 0], ci[:, 1], ci[:, 2]].t().numpy()
    np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)


def test_down2_conv_and_deconv_vs_torch(orc):
    G, Cin, Cout = 16, 6, 4
    c = scene(2, 1200, G)
    rng = np.random.default_rng(3)
    x = rng.normal(size=(len(c), Cin)).astype(np.float32)
    W = rng.normal(size=(8, Cin, Cout)).astype(np.float32) * 0.3
    parent, off, cc = orc.down2_rules(c)
    counts, pairs = orc.down2_pairs(parent, off)
    y, flops = orc.conv_forward(x, W, None, pairs, counts, len(cc))
    assert flops == len(c) * Cin * Cout
    w = torch.from_numpy(W.astype(np.float64)).reshape(2, 2, 2, Cin, Cout).permute(4, 3, 0, 1, 2)
    d = F.conv3d(to_dense(c, x, G), w, stride=2)
    ci = torch.from_numpy(cc.astype(np.int64))
    ref = d[0, :, ci[:, 0], ci[:, 1], ci[:, 2]].t().numpy()
    np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)
    # every coarse cell outside the coarse active set would be exactly zero in the dense result
    mask = torch.zeros(G // 2, G // 2, G // 2, dtype=torch.bool)
    mask[ci[:, 0], ci[:, 1], ci[:, 2]] = True
    assert float(d[0][:, ~mask].abs().max()) == 0.0

    # deconvolution: coarse [Nc,Cout'] -> fine sites, same rules with roles swapped
    Ci2, Co2 = 4, 5
    xc = rng.normal(size=(len(cc), Ci2)).astype(np.float32)
    W2 = rng.normal(size=(8, Ci2, Co2)).astype(np.float32) * 0.3
    yf, _ = orc.conv_forward(xc, W2, None, pairs, counts, len(c), swap=True)
    wt = torch.from_numpy(W2.astype(np.float64)).reshape(2, 2, 2, Ci2, Co2).permute(3, 4, 0, 1, 2)
    dd = F.conv_transpose3d(to_dense(cc, xc, G // 2), wt, stride=2)
    fi = torch.from_numpy(c.astype(np.int64))
    ref2 = dd[0, :, fi[:, 0], fi[:, 1], fi[:, 2]].t().numpy()
    np.testing.assert_allclose(yf, ref2, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("leak", [0.0, 0.333, 1.0])
def test_bn_vs_torch(orc, leak):
    rng = np.random.default_rng(4)
    N, C = 777, 24
    x = rng.normal(size=(N, C)).astype(np.float32) * 3
    mean = rng.normal(size=C).astype(np.float32)
    var = rng.uniform(0.5, 2, C).astype(np.float32)
    g = rng.uniform(0.5, 1.5, C).astype(np.float32)
    b = rng.normal(size=C).astype(np.float32) * 0.1
    y = orc.bn_forward(x, mean, var, g, b, eps=1e-4, leakiness=leak)
    t = lambda a: torch.from_numpy(a.astype(np.float64))
    ref = F.leaky_relu(F.batch_norm(t(x), t(mean), t(var), t(g), t(b), training=False, eps=1e-4), leak).numpy()
    np.testing.assert_allclose(y, ref, rtol=RTOL, atol=ATOL)
    y2 = orc.bn_forward(x, mean, var, None, None, eps=1e-4, leakiness=leak)
    ref2 = F.leaky_relu(F.batch_norm(t(x), t(mean), t(var), None, None, training=False, eps=1e-4), leak).numpy()
    np.testing.assert_allclose(y2, ref2, rtol=RTOL, atol=ATOL)


def test_input_mean_and_output(orc):
    rng = np.random.default_rng(5)
    pts = rng.integers(0, 9, (3000, 3)).astype(np.int32)
    f = rng.normal(size=(3000, 3)).astype(np.float32)
    sop, sc, cnt = orc.grid_build(pts)
    mean = orc.input_forward(f, sop, cnt, mode=4)
    ssum = orc.input_forward(f, sop, cnt, mode=3)
    ref = np.zeros((len(sc), 3))
    np.add.at(ref, sop, f.astype(np.float64))
    np.testing.assert_allclose(ssum, ref, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(mean, ref / np.bincount(sop)[:, None], rtol=RTOL, atol=ATOL)
    out = orc.output_forward(mean, sop)
    assert (out == mean[sop]).all()
    # no duplicates => identity up to the row permutation
    u = np.unique(pts, axis=0)
    fu = rng.normal(size=(len(u), 4)).astype(np.float32)
    sop2, _, cnt2 = orc.grid_build(u)
    assert (sop2 == np.arange(len(u))).all() and (cnt2 == 1).all()
    assert (orc.input_forward(fu, sop2, cnt2, mode=4) == fu).all()


def test_nin(orc):
    rng = np.random.default_rng(6)
    x = rng.normal(size=(500, 12)).astype(np.float32)
    W = rng.normal(size=(12, 6)).astype(np.float32)
    b = rng.normal(size=6).astype(np.float32)
    np.testing.assert_allclose(orc.nin_forward(x, W, b), x.astype(np.float64) @ W + b, rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(orc.nin_forward(x, W), x.astype(np.float64) @ W, rtol=RTOL, atol=ATOL)
