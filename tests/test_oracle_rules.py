"""Pins the integer half of the CPU oracle (grid, submanifold and stride-2 rulebooks)
against numpy set operations, brute force with a Python dict, and structural invariants.
The reference holds no golden vectors for this path, so these checks are what anchors the
oracle; each one fails for a plausible mistake (wrong offset order, swapped in/out,
dropped neighbour, wrong parity bit)."""
import numpy as np
import pytest

from workloads import scenes


def small_scene(seed, n=1500, grid=24):
    rng = np.random.default_rng(seed)
    c = rng.integers(0, grid, (n, 3)).astype(np.int32)
    b = rng.integers(0, 2, (n, 1)).astype(np.int32)
    return np.concatenate([c, b], 1)


def test_grid_matches_numpy_unique(orc):
    pts = small_scene(0, 4000, 12)  # many duplicates
    sop, sc, cnt = orc.grid_build(pts)
    uniq, inv, counts = np.unique(pts, axis=0, return_inverse=True, return_counts=True)
    assert len(sc) == len(uniq)
    # same set
    assert (orc.canonical_sites(sc) == orc.canonical_sites(uniq)).all()
    # every point maps to the site holding its own coordinates
    assert (sc[sop] == pts).all()
    # first-appearance numbering: site ids appear in increasing order of first use
    first = np.full(len(sc), len(pts))
    np.minimum.at(first, sop, np.arange(len(pts)))
    assert (np.diff(first) > 0).all()
    # duplicate counts
    key = {tuple(u): c for u, c in zip(uniq.tolist(), counts.tolist())}
    assert [key[tuple(s)] for s in sc.tolist()] == cnt.tolist()


def test_grid_query_vs_dict(orc):
    pts = small_scene(1)
    _, sc, _ = orc.grid_build(pts)
    d = {tuple(s): i for i, s in enumerate(sc.tolist())}
    q = small_scene(2, 3000, 26)
    got = orc.grid_query(sc, q)
    exp = np.array([d.get(tuple(x), -1) for x in q.tolist()], np.int32)
    assert (got == exp).all()
    assert (got == -1).any() and (got >= 0).any()


@pytest.mark.parametrize("seed", [3, 4])
def test_ssc_rules_brute_force(orc, seed):
    _, sc, _ = orc.grid_build(small_scene(seed, 2000, 14))
    nbr, counts, pairs = orc.ssc_rules(sc)
    d = {tuple(s): i for i, s in enumerate(sc.tolist())}
    exp = np.full((len(sc), 27), -1, np.int32)
    for o, (x, y, z, b) in enumerate(sc.tolist()):
        k = 0
        for dx in (-1, 0, 1):  # x outermost, z innermost: offset = (dx+1)*9+(dy+1)*3+(dz+1)
            for dy in (-1, 0, 1):
                for dz in (-1, 0, 1):
                    exp[o, k] = d.get((x + dx, y + dy, z + dz, b), -1)
                    k += 1
    assert (nbr == exp).all()
    assert counts.tolist() == (exp >= 0).sum(0).tolist()
    # pair lists: offset k holds (nbr[o,k], o) in ascending o
    base = 0
    for k in range(27):
        o = np.nonzero(exp[:, k] >= 0)[0]
        assert (pairs[base:base + len(o), 1] == o).all()
        assert (pairs[base:base + len(o), 0] == exp[o, k]).all()
        base += len(o)
    assert base == len(pairs)


def test_ssc_rules_invariants(orc):
    sc = scenes.boxes_scene(seed=7, n=5000, grid=64, lo_rng=(4, 30))
    nbr, counts, pairs = orc.ssc_rules(sc)
    N = len(sc)
    # centre offset is the identity on all sites
    assert (nbr[:, 13] == np.arange(N)).all()
    # symmetry: (k, i, o) in RB  <=>  (26-k, o, i) in RB
    for k in range(27):
        o = np.nonzero(nbr[:, k] >= 0)[0]
        assert (nbr[nbr[o, k], 26 - k] == o).all()
    assert counts.sum() == (nbr >= 0).sum() == len(pairs)
    # each output at most once per offset; input = output + delta
    base = 0
    for k in range(27):
        p = pairs[base:base + counts[k]]
        assert len(np.unique(p[:, 1])) == len(p)
        delta = np.array([k // 9 - 1, (k // 3) % 3 - 1, k % 3 - 1])
        assert (sc[p[:, 0], :3] - sc[p[:, 1], :3] == delta).all()
        base += counts[k]


def test_ssc_offset_order_permutation(orc):
    """The CPU rewrite's z-major numbering is the x-major one under k <-> (k%3)*9+((k/3)%3)*3+k/9."""
    _, sc, _ = orc.grid_build(small_scene(5, 1500, 12))
    nx, _, _ = orc.ssc_rules(sc, zmajor=False)
    nz, _, _ = orc.ssc_rules(sc, zmajor=True)
    perm = np.array([(k % 3) * 9 + ((k // 3) % 3) * 3 + k // 9 for k in range(27)])
    assert (nz == nx[:, perm]).all()
    assert not (nz == nx).all()


def test_batches_do_not_mix(orc):
    a = np.array([[5, 5, 5, 0], [5, 5, 6, 1], [5, 6, 5, 0]], np.int32)
    nbr, counts, _ = orc.ssc_rules(a)
    assert nbr[0, 14] == -1 and nbr[1, 12] == -1  # z+-1 neighbour lives in the other sample
    assert nbr[0, 16] == 2 and nbr[2, 10] == 0


def test_down2_rules_closed_form(orc):
    _, sc, _ = orc.grid_build(small_scene(6, 3000, 20))
    parent, off, cc = orc.down2_rules(sc)
    half = sc.copy()
    half[:, :3] >>= 1
    uniq = np.unique(half, axis=0)
    assert len(cc) == len(uniq)
    assert (orc.canonical_sites(cc) == orc.canonical_sites(uniq)).all()
    assert (cc[parent] == half).all()
    assert (off == (sc[:, 0] & 1) * 4 + (sc[:, 1] & 1) * 2 + (sc[:, 2] & 1)).all()
    # first-appearance numbering of the coarse sites
    first = np.full(len(cc), len(sc))
    np.minimum.at(first, parent, np.arange(len(sc)))
    assert (np.diff(first) > 0).all()
    counts, pairs = orc.down2_pairs(parent, off)
    assert counts.sum() == len(sc) and len(np.unique(pairs[:, 0])) == len(sc)  # every input exactly once


def test_canonical_rules_is_numbering_independent(orc):
    pts = small_scene(8, 1200, 10)
    _, sc, _ = orc.grid_build(pts)
    _, c1, p1 = orc.ssc_rules(sc)
    perm = np.random.default_rng(0).permutation(len(sc))
    sc2 = sc[perm]
    _, c2, p2 = orc.ssc_rules(sc2)
    assert (orc.canonical_rules(c1, p1, sc, sc) == orc.canonical_rules(c2, p2, sc2, sc2)).all()
