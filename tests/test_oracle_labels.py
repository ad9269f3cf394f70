"""Pins of the label-fusion oracle: a hand-worked sequence for one voxel (every branch of
Result::update, Metadata/resultHash.h:78-99) and the closed form of ResultOfWeight's running
scores (x_n + x_{n-1}/2 + ... + x_1/2^(n-1), resultHash.h:158-170)."""
import numpy as np


def _row(label, p, C=4):
    r = np.zeros(C, np.float32)
    r[label] = p
    return r[None]


def test_result_update_known_sequence(orc):
    P = [[5, 6, 7]]
    r = orc.ResultOracle(maximum=3.9)  # ceiling int(3.9) = 3
    r.update(P, _row(2, 0.6))
    assert r.result[(5, 6, 7)] == [2, np.float32(0.6)]          # new voxel: (argmax, max)
    r.update(P, _row(2, 0.5))
    assert r.result[(5, 6, 7)][0] == 2 and abs(r.result[(5, 6, 7)][1] - 1.1) < 1e-6   # agree: gain
    r.update(P, _row(1, 0.4))
    assert r.result[(5, 6, 7)][0] == 2 and abs(r.result[(5, 6, 7)][1] - 0.7) < 1e-6   # disagree: lose
    r.update(P, _row(1, 0.9))
    assert r.result[(5, 6, 7)][0] == 1 and abs(r.result[(5, 6, 7)][1] - 0.2) < 1e-6   # below zero: flip
    for _ in range(5):
        r.update(P, _row(1, 0.9))
    assert r.result[(5, 6, 7)] == [1, np.float32(3.0)]           # ceiling
    assert r.multi_query([[5, 6, 7], [0, 0, 0]]).tolist() == [1, -1]


def test_result_default_maximum_truncates_to_zero(orc):
    r = orc.ResultOracle()  # 0.7 stored in an int member
    r.update([[1, 1, 1]], _row(3, 0.8))
    r.update([[1, 1, 1]], _row(3, 0.8))
    assert r.result[(1, 1, 1)] == [3, np.float32(0.0)]


def test_result_duplicates_in_one_call_apply_in_row_order(orc):
    r = orc.ResultOracle(maximum=5)
    ps = [[1, 2, 3], [1, 2, 3], [9, 9, 9], [1, 2, 3]]
    sc = np.concatenate([_row(0, 0.5), _row(1, 0.7), _row(2, 0.3), _row(1, 0.1)])
    r.update(ps, sc)
    # (0,0.5) -> disagree: 0.5-0.7 < 0 -> (1,0.2) -> agree: 0.3
    assert r.result[(1, 2, 3)][0] == 1 and abs(r.result[(1, 2, 3)][1] - 0.3) < 1e-6
    assert r.all_points_labels().tolist() == [[1, 2, 3, 1], [9, 9, 9, 2]]
    r.set([[9, 9, 9], [9, 9, 9]], np.concatenate([_row(3, 1.0), _row(0, 1.0)]))
    assert r.result[(9, 9, 9)] == [0, np.float32(0)]             # set: last row wins, confidence 0
    r.finalize([[9, 9, 9], [4, 4, 4]])
    assert list(r.result) == [(9, 9, 9)]


def test_result_of_weight_closed_form(orc):
    rng = np.random.default_rng(0)
    xs = rng.normal(size=(6, 5)).astype(np.float32)
    r = orc.ResultOfWeightOracle()
    for x in xs:
        r.update([[3, 3, 3]], x[None])
    want = sum(xs[i].astype(np.float64) / 2 ** (len(xs) - 1 - i) for i in range(len(xs)))
    np.testing.assert_allclose(r.result[(3, 3, 3)], want, rtol=1e-5)
    assert r.multi_query([[3, 3, 3], [0, 0, 0]]).tolist() == [int(np.argmax(want)), -1]
