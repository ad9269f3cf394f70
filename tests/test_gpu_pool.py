"""GPU parity of size-2 stride-2 max / average pooling, unpooling and the dense copy against the
CPU oracle, through the reference's op names and module classes.  These are selections, copies
and sums of at most eight terms in a fixed order: compared bit for bit."""
import numpy as np
import pytest
import torch

from workloads import scenes

pytestmark = pytest.mark.gpu
SZ = torch.LongTensor([128, 128, 128])
SZ2 = torch.LongTensor([64, 64, 64])
TWO = torch.LongTensor([2, 2, 2])


@pytest.fixture(scope="module")
def S():
    from sparseconvnet import SCN
    from sparseconvnet._lib import ensure_init

    ensure_init(0)
    return SCN


def cu(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _sites(S, pts, C, seed):
    rng = np.random.default_rng(seed)
    f = rng.normal(size=(len(pts), C)).astype(np.float32)
    m = S.Metadata_3()
    out = torch.empty(0, device="cuda")
    S.InputLayer_updateOutput(m, SZ, torch.from_numpy(pts.astype(np.int64)), cu(f), out, 0, 0)
    return m, f, out


@pytest.mark.parametrize("C,drop", [(32, 0), (7, 2), (96, 0)])
def test_pooling_and_unpooling(S, orc, C, drop):
    pts = scenes.boxes_scene(seed=3, n=20000)
    m, f, feats = _sites(S, pts, C, seed=C)
    parent, off, cc = orc.down2_rules(pts)
    out = torch.empty(0, device="cuda")
    S.MaxPooling_updateOutput(SZ, SZ2, TWO, TWO, m, feats, out, drop)
    assert (out.cpu().numpy() == orc.max_pool_forward(f, parent, len(cc), drop)).all()
    S.AveragePooling_updateOutput(SZ, SZ2, TWO, TWO, m, feats, out, drop)
    avg = orc.avg_pool_forward(f, parent, off, len(cc), drop)
    assert (out.cpu().numpy() == avg).all()
    assert out.shape == (len(cc), C - drop)
    up = torch.empty(0, device="cuda")
    S.UnPooling_updateOutput(SZ2, SZ, TWO, TWO, m, out, up, 1 if C - drop > 1 else 0)
    d2 = 1 if C - drop > 1 else 0
    assert (up.cpu().numpy() == orc.unpool_forward(avg, parent, d2)).all()
    assert up.shape == (len(pts), C - drop - d2)


def test_sparse_to_dense(S, orc):
    rng = np.random.default_rng(5)
    c = np.unique(np.concatenate([rng.integers(0, [20, 24, 28], (6000, 3)), rng.integers(0, 3, (6000, 1))], 1), axis=0)
    c = c[rng.permutation(len(c))].astype(np.int32)
    x = rng.normal(size=(len(c), 5)).astype(np.float32)
    size = torch.LongTensor([20, 24, 28])
    m = S.Metadata_3()
    feats = torch.empty(0, device="cuda")
    S.InputLayer_updateOutput(m, size, torch.from_numpy(c.astype(np.int64)), cu(x), feats, 3, 0)
    out = torch.empty(0, device="cuda")
    S.SparseToDense_updateOutput(size, m, feats, out, 5)
    ref = orc.sparse_to_dense(x, c, (20, 24, 28), 3)
    assert tuple(out.shape) == ref.shape
    assert (out.cpu().numpy() == ref).all()


def test_pooling_modules_in_a_network(orc):
    """InputLayer -> SSC -> MaxPooling -> SSC -> UnPooling -> SparseToDense through the module
    classes, against the same chain on the oracle."""
    import sparseconvnet as scn

    pts = scenes.boxes_scene(seed=6, n=8000, grid=64, n_boxes=4, lo_rng=(4, 30), size_rng=(8, 24))
    rng = np.random.default_rng(7)
    f = rng.normal(size=(len(pts), 3)).astype(np.float32)
    torch.manual_seed(3)
    net = scn.Sequential().add(scn.InputLayer(3, 64, mode=0)).add(scn.SubmanifoldConvolution(3, 3, 16, 3, False)).add(
        scn.MaxPooling(3, 2, 2)).add(scn.SubmanifoldConvolution(3, 16, 8, 3, True)).add(scn.UnPooling(3, 2, 2)).add(
        scn.SparseToDense(3, 8)).cuda()
    with torch.no_grad():
        net[3].bias.normal_()
        out = net([torch.from_numpy(pts[:, :3].astype(np.int64)), cu(f), 1])
    assert tuple(out.shape) == (1, 8, 64, 64, 64)
    sop, sc, cnt = orc.grid_build(pts)
    x = orc.input_forward(f, sop, cnt, mode=3)
    _, counts, pairs = orc.ssc_rules(sc)
    x, _ = orc.conv_forward(x, net[1].weight.detach().cpu().numpy(), None, pairs, counts, len(sc))
    parent, off, cc = orc.down2_rules(sc)
    x = orc.max_pool_forward(x, parent, len(cc))
    _, counts, pairs = orc.ssc_rules(cc)
    x, _ = orc.conv_forward(x, net[3].weight.detach().cpu().numpy(), net[3].bias.detach().cpu().numpy(), pairs,
                            counts, len(cc))
    x = orc.unpool_forward(x, parent)
    ref = orc.sparse_to_dense(x, sc, (64, 64, 64), 1)
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=1e-4, atol=1e-5)
    with pytest.raises(NotImplementedError):
        net[2](None, increment=True)
