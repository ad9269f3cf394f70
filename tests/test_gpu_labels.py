"""Label fusion on the GPU against the oracle: random frames with repeated voxels, both table
kinds, queries, export, finalize and growth.  Labels are compared exactly; confidences and
scores are float32 sums of the same terms in the same order, compared exactly as well."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _frames(rng, n_frames, P, C, span):
    for _ in range(n_frames):
        ps = rng.integers(0, span, (P, 3))
        ps[P // 2:] = ps[rng.integers(0, P // 2, P - P // 2)]  # half of the rows repeat earlier voxels
        sc = rng.uniform(0, 1, (P, C)).astype(np.float32)
        yield ps, sc


@pytest.mark.parametrize("maximum", [0.7, 2.5])
def test_result_matches_oracle(orc, maximum):
    from sparseconvnet import SCN

    rng = np.random.default_rng(7)
    ref, got = orc.ResultOracle(maximum), SCN.Result_3(maximum)
    ps0 = rng.integers(0, 12, (300, 3))
    sc0 = rng.uniform(0, 1, (300, 20)).astype(np.float32)
    ref.set(ps0, sc0)
    got.set(torch.from_numpy(ps0), torch.from_numpy(sc0))
    for ps, sc in _frames(rng, 6, 4000, 20, 14):
        ref.update(ps, sc)
        got.update(torch.from_numpy(ps), torch.from_numpy(sc).cuda())
    assert len(got) == len(ref.result)
    pts, conf = got.get_all_points_labels(with_confidence=True)
    assert np.array_equal(pts.numpy(), ref.all_points_labels())       # same voxels, same order, same labels
    assert np.array_equal(conf.numpy(), ref.confidences())
    q = rng.integers(-2, 16, (5000, 3))
    q = q[(q >= 0).all(1)]
    assert np.array_equal(got.multiQuery(torch.from_numpy(q)).numpy(), ref.multi_query(q))
    assert got.query(torch.from_numpy(q[0])) == int(ref.multi_query(q[:1])[0])
    keep = np.concatenate([ref.all_points_labels()[::3, :3], rng.integers(20, 30, (10, 3))])
    ref.finalize(keep)
    got.finalize(torch.from_numpy(keep))
    assert np.array_equal(got.get_all_points_labels().numpy(), ref.all_points_labels())
    for ps, sc in _frames(rng, 2, 3000, 20, 14):  # the table keeps working after finalize
        ref.update(ps, sc)
        got.update(torch.from_numpy(ps), torch.from_numpy(sc))
    pts, conf = got.get_all_points_labels(with_confidence=True)
    assert np.array_equal(pts.numpy(), ref.all_points_labels()) and np.array_equal(conf.numpy(), ref.confidences())
    got.clear()
    assert len(got) == 0 and got.query(torch.from_numpy(q[0])) == -1


def test_result_of_weight_matches_oracle_and_grows(orc):
    from sparseconvnet import SCN

    rng = np.random.default_rng(8)
    ref, got = orc.ResultOfWeightOracle(), SCN.ResultOfWeight()
    for ps, sc in _frames(rng, 5, 40000, 8, 100):  # ~100k distinct voxels: outgrows the initial 64k rows
        ref.update(ps, sc)
        got.update(torch.from_numpy(ps), torch.from_numpy(sc))
    assert len(got) == len(ref.result) > (1 << 16)
    assert np.array_equal(got.get_all_points_labels().numpy(), ref.all_points_labels())
    q = rng.integers(0, 104, (4000, 3))
    assert np.array_equal(got.multiQuery(torch.from_numpy(q)).numpy(), ref.multi_query(q))
    keep = ref.all_points_labels()[1::2, :3]
    ref.finalize(keep)
    got.finalize(torch.from_numpy(keep))
    assert np.array_equal(got.get_all_points_labels().numpy(), ref.all_points_labels())
    with pytest.raises(Exception):
        got.update(torch.from_numpy(q[:4]), torch.zeros(4, 5))  # width differs from the table's
