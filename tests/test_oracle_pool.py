"""Pins the oracle's pooling / unpooling / dense-copy restatements against torch library
routines on dense tensors (float64): avg_pool3d, max_pool3d, nearest upsampling and
sparse_coo_tensor(...).to_dense().  The reference's max pooling starts from a zeroed output,
so its result is max(0, max over the active children); the dense counterpart is max_pool3d over
the zero-filled volume wherever a cell has an inactive child or a positive value, and the
remaining case (eight active children, all negative) is checked by hand."""
import numpy as np
import torch
import torch.nn.functional as F

G = 16


def _scene(seed, n):
    rng = np.random.default_rng(seed)
    c = np.unique(rng.integers(0, G, (n, 3)).astype(np.int32), axis=0)
    return c[rng.permutation(len(c))]


def _dense(coords, feats, g=G):
    d = torch.zeros(1, feats.shape[1], g, g, g, dtype=torch.float64)
    c = torch.from_numpy(coords.astype(np.int64))
    d[0, :, c[:, 0], c[:, 1], c[:, 2]] = torch.from_numpy(feats.astype(np.float64)).t()
    return d


def _at(d, coords):
    c = torch.from_numpy(coords.astype(np.int64))
    return d[0, :, c[:, 0], c[:, 1], c[:, 2]].t().numpy()


def test_pooling_vs_torch(orc):
    c = _scene(0, 1500)
    rng = np.random.default_rng(1)
    x = rng.normal(size=(len(c), 6)).astype(np.float32)
    parent, off, cc = orc.down2_rules(c)
    avg = orc.avg_pool_forward(x, parent, off, len(cc), drop=1)
    ref = _at(F.avg_pool3d(_dense(c, x[:, 1:]), 2), cc)
    np.testing.assert_allclose(avg, ref, rtol=1e-6, atol=1e-7)
    mx = orc.max_pool_forward(x, parent, len(cc))
    ref = _at(F.max_pool3d(_dense(c, x), 2), cc)
    full = np.bincount(parent, minlength=len(cc)) == 8
    assert (~full).sum() > 100
    assert (mx[~full] == ref[~full].astype(np.float32)).all()
    assert (mx >= 0).all() and (mx[full] == np.maximum(ref[full], 0).astype(np.float32)).all()
    # eight active children, all negative: the zero the output started from stays
    cube = np.array([[2 + (k >> 2), 4 + ((k >> 1) & 1), 6 + (k & 1)] for k in range(8)], np.int32)
    p, o, c2 = orc.down2_rules(cube)
    assert len(c2) == 1
    assert orc.max_pool_forward(-np.ones((8, 2), np.float32), p, 1).tolist() == [[0.0, 0.0]]
    assert orc.avg_pool_forward(-np.ones((8, 2), np.float32), p, o, 1).tolist() == [[-1.0, -1.0]]


def test_unpooling_vs_nearest_upsampling(orc):
    c = _scene(2, 1200)
    rng = np.random.default_rng(3)
    parent, off, cc = orc.down2_rules(c)
    z = rng.normal(size=(len(cc), 5)).astype(np.float32)
    up = orc.unpool_forward(z, parent, drop=2)
    ref = _at(F.interpolate(_dense(cc, z[:, 2:], G // 2), scale_factor=2, mode="nearest"), c)
    assert (up == ref.astype(np.float32)).all()


def test_sparse_to_dense_vs_torch_sparse(orc):
    rng = np.random.default_rng(4)
    c = np.unique(np.concatenate([rng.integers(0, [5, 6, 7], (150, 3)), rng.integers(0, 3, (150, 1))], 1), axis=0)
    c = c[rng.permutation(len(c))].astype(np.int32)
    x = rng.normal(size=(len(c), 4)).astype(np.float32)
    d = orc.sparse_to_dense(x, c, (5, 6, 7), 3)
    idx = torch.from_numpy(c[:, [3, 0, 1, 2]].astype(np.int64)).t()
    ref = torch.sparse_coo_tensor(idx, torch.from_numpy(x), (3, 5, 6, 7, 4)).to_dense().permute(0, 4, 1, 2, 3)
    assert d.shape == (3, 4, 5, 6, 7)
    assert (d == ref.numpy()).all()
