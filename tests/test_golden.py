"""Committed golden vectors (tests/golden/small_scene.npz, written by make_golden.py from the
CPU oracle): the oracle must keep reproducing them (CPU test), and the HIP path must reproduce
them through the reference's op names (GPU test) - bit-exact for the integer structures,
1e-4 / 1e-5 for float32 outputs."""
import os

import numpy as np
import pytest

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "small_scene.npz"))
RTOL, ATOL = 1e-4, 1e-5


def test_oracle_reproduces_golden(orc):
    sop, sc, cnt = orc.grid_build(G["pts"])
    assert (sop == G["site_of_point"]).all() and (sc == G["site_coords"]).all() and (cnt == G["count"]).all()
    x = orc.input_forward(G["feats"], sop, cnt, mode=4)
    assert (x == G["x"]).all()
    nbr, counts, pairs = orc.ssc_rules(sc)
    assert (nbr == G["nbr"]).all() and (counts == G["ssc_counts"]).all() and (pairs == G["ssc_pairs"]).all()
    y, _ = orc.conv_forward(x, G["W"], G["b"], pairs, counts, len(sc))
    np.testing.assert_allclose(y, G["y"], rtol=RTOL, atol=ATOL)
    parent, off, cc = orc.down2_rules(sc)
    assert (parent == G["parent"]).all() and (off == G["offset"]).all() and (cc == G["coarse_coords"]).all()


@pytest.mark.gpu
def test_hip_reproduces_golden():
    import torch

    from sparseconvnet import SCN

    cu = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    SZ, two, three = torch.LongTensor([8, 8, 8]), torch.LongTensor([2, 2, 2]), torch.LongTensor([3, 3, 3])
    m = SCN.Metadata_3()
    x = torch.empty(0, device="cuda")
    SCN.InputLayer_updateOutput(m, SZ, torch.from_numpy(G["pts"].astype(np.int64)), cu(G["feats"]), x, 2, 4)
    assert (m.site_of_point.cpu().numpy() == G["site_of_point"]).all()
    assert (m.getSpatialLocations(SZ).numpy() == G["site_coords"]).all()
    np.testing.assert_allclose(x.cpu().numpy(), G["x"], rtol=RTOL, atol=ATOL)
    sc = m.ssc_rulebook(SZ)
    assert (sc.nbr.t[:sc.n].cpu().numpy() == G["nbr"]).all()
    counts, pairs = SCN.ssc_rulebook_lists(m, SZ)
    assert (counts.numpy() == G["ssc_counts"]).all() and (pairs.numpy() == G["ssc_pairs"]).all()
    y = torch.empty(0, device="cuda")
    SCN.SubmanifoldConvolution_updateOutput(SZ, three, m, cu(G["x"]), y, cu(G["W"]), cu(G["b"]), 1)
    np.testing.assert_allclose(y.cpu().numpy(), G["y"], rtol=RTOL, atol=ATOL)
    z = torch.empty(0, device="cuda")
    SCN.BatchNormalization_updateOutput(cu(G["y"]), z, None, None, cu(G["mean"]), cu(G["var"]), cu(G["gamma"]),
                                        cu(G["beta"]), 1e-4, 0.9, False, 0.0)
    np.testing.assert_allclose(z.cpu().numpy(), G["z"], rtol=RTOL, atol=ATOL)
    c = torch.empty(0, device="cuda")
    SCN.Convolution_updateOutput(SZ, SZ // 2, two, two, m, cu(G["z"]), c, cu(G["Wd"]), torch.Tensor())
    fine, coarse, d = m.down_rulebook(SZ, SZ // 2)
    assert (d.parent.t[:fine.n].cpu().numpy() == G["parent"]).all()
    assert (d.offset.t[:fine.n].cpu().numpy() == G["offset"]).all()
    assert (coarse.coords_view().cpu().numpy() == G["coarse_coords"]).all()
    np.testing.assert_allclose(c.cpu().numpy(), G["c"], rtol=RTOL, atol=ATOL)
    u = torch.empty(0, device="cuda")
    SCN.Deconvolution_updateOutput(SZ // 2, SZ, two, two, m, cu(G["c"]), u, cu(G["Wu"]), torch.Tensor())
    np.testing.assert_allclose(u.cpu().numpy(), G["u"], rtol=RTOL, atol=ATOL)
    v = torch.empty(0, device="cuda")
    SCN.NetworkInNetwork_updateOutput(cu(G["u"]), v, cu(G["Wn"]), torch.Tensor())
    np.testing.assert_allclose(v.cpu().numpy(), G["v"], rtol=RTOL, atol=ATOL)
    o = torch.empty(0, device="cuda")
    SCN.OutputLayer_updateOutput(m, cu(G["v"]), o)
    assert (o.cpu().numpy() == G["out"]).all()
