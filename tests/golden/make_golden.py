"""Writes tests/golden/small_scene.npz: inputs and expected outputs of every operator of the
path on one tiny scene, computed by the CPU oracle (oracle/insc_oracle.c), which is itself
pinned against torch conv3d / conv_transpose3d / batch_norm and numpy in tests/test_oracle_*.py.
The reference ships no fixtures for this path and cannot be built or imported here, so these
vectors come from the oracle, not from the reference.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import oracle as orc  # noqa: E402


def main():
    rng = np.random.default_rng(20240607)
    pts = np.concatenate([rng.integers(0, 7, (160, 3)), rng.integers(0, 2, (160, 1))], 1).astype(np.int32)
    feats = rng.normal(size=(160, 4)).astype(np.float32)
    sop, sc, cnt = orc.grid_build(pts)
    x = orc.input_forward(feats, sop, cnt, mode=4)
    nbr, counts, pairs = orc.ssc_rules(sc)
    W = (rng.normal(size=(27, 4, 8)) * 0.2).astype(np.float32)
    b = rng.normal(size=8).astype(np.float32)
    y, _ = orc.conv_forward(x, W, b, pairs, counts, len(sc))
    mean, var = rng.normal(size=8).astype(np.float32), rng.uniform(0.5, 2, 8).astype(np.float32)
    gamma, beta = rng.uniform(0.5, 1.5, 8).astype(np.float32), (rng.normal(size=8) * 0.1).astype(np.float32)
    z = orc.bn_forward(y, mean, var, gamma, beta, 1e-4, 0.0)
    parent, off, cc = orc.down2_rules(sc)
    dcounts, dpairs = orc.down2_pairs(parent, off)
    Wd = (rng.normal(size=(8, 8, 6)) * 0.3).astype(np.float32)
    c, _ = orc.conv_forward(z, Wd, None, dpairs, dcounts, len(cc))
    Wu = (rng.normal(size=(8, 6, 8)) * 0.3).astype(np.float32)
    u, _ = orc.conv_forward(c, Wu, None, dpairs, dcounts, len(sc), swap=True)
    Wn = (rng.normal(size=(8, 5)) * 0.4).astype(np.float32)
    v = orc.nin_forward(u, Wn, None)
    out = orc.output_forward(v, sop)
    np.savez_compressed(os.path.join(HERE, "small_scene.npz"), pts=pts, feats=feats, site_of_point=sop,
                        site_coords=sc, count=cnt, x=x, nbr=nbr, ssc_counts=counts, ssc_pairs=pairs, W=W, b=b, y=y,
                        mean=mean, var=var, gamma=gamma, beta=beta, z=z, parent=parent, offset=off,
                        coarse_coords=cc, Wd=Wd, c=c, Wu=Wu, u=u, Wn=Wn, v=v, out=out)
    print("wrote small_scene.npz:", len(pts), "points,", len(sc), "sites,", len(pairs), "rules")


if __name__ == "__main__":
    main()
