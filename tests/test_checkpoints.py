"""Checkpoint helpers and the offset-numbering conversion for weights trained against the
reference's CPU rule generator (no GPU needed: modules are only constructed, the numerical
check runs on the CPU oracle), and the state_dict keys of the reference's module tree for its usage
example (model.py:15-21 over networkArchitectures.py:202-300)."""
import os

import numpy as np
import torch

from workloads import scenes


def test_checkpoint_round_trip(tmp_path):
    import sparseconvnet as scn
    from workloads.netdefs import NaiveUNet

    a, b = NaiveUNet(m=8, levels=3, seed=1), NaiveUNet(m=8, levels=3, seed=2)
    exp = str(tmp_path / "exp")
    for epoch in (1, 2, 3, 4, 5):
        scn.checkpoint_save(a, exp, "unet", epoch, use_cuda=False)
    left = sorted(os.listdir(tmp_path))
    # epochs whose number is a power of two survive, plus the latest (utils.py:228-233)
    assert left == ["exp-0001-unet.pth", "exp-0002-unet.pth", "exp-0004-unet.pth", "exp-0005-unet.pth"]
    nxt = scn.checkpoint_restore(b, exp, "unet", use_cuda=False)
    assert nxt == 6
    for (ka, va), (kb, vb) in zip(a.state_dict().items(), b.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)
    assert scn.checkpoint_restore(b, exp, "unet", use_cuda=False, epoch=2) == 3
    # parameter names and shapes are the reference's: [27|8, nIn, nOut] filters, BN running stats
    sd = a.state_dict()
    assert any(v.dim() == 3 and v.size(0) == 27 for v in sd.values())
    assert any(v.dim() == 3 and v.size(0) == 8 for v in sd.values())
    assert any(k.endswith("running_mean") for k in sd) and any(k.endswith("running_var") for k in sd)


def test_zmajor_weights_convert_to_this_numbering(orc):
    import sparseconvnet as scn

    perm = scn.ssc_offset_permutation()
    assert torch.equal(perm[perm], torch.arange(27))
    for k in range(27):
        dx, dy, dz = k // 9 - 1, (k // 3) % 3 - 1, k % 3 - 1
        assert perm[k].item() == (dz + 1) * 9 + (dy + 1) * 3 + (dx + 1)
    pts = scenes.boxes_scene(seed=1, n=3000)
    _, sc, _ = orc.grid_build(pts)
    rng = np.random.default_rng(0)
    x = rng.normal(size=(len(sc), 8)).astype(np.float32)
    Wz = rng.normal(size=(27, 8, 12)).astype(np.float32)  # trained against the z-major numbering
    _, cz, pz = orc.ssc_rules(sc, zmajor=True)
    ref, _ = orc.conv_forward(x, Wz, None, pz, cz, len(sc))
    Wx = scn.convert_zmajor_state_dict({"w": torch.from_numpy(Wz), "b": torch.zeros(3)})["w"].numpy()
    _, cx, px = orc.ssc_rules(sc, zmajor=False)
    got, _ = orc.conv_forward(x, Wx, None, px, cx, len(sc))
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=1e-5)  # (the two runs add the 27 terms in different orders)


# The keys of `sparseModel` for m = 8, two levels, reps = 1, residual blocks, written out by hand from
# the reference's builder: Sequential indices follow the order of .add(); a residual block is
# ConcatTable(0: shortcut, 1: Sequential(0: BN, 1: SSC, 2: BN, 3: SSC)) then AddTable; a level is
# [block] [ConcatTable(0: Identity, 1: Sequential(0: BN, 1: Conv, 2: <inner>, 3: BN, 4: Deconv))]
# [JoinTable] [block with NiN shortcut].  BN contributes running_mean, running_var (buffers, listed
# after the parameters of the same module by torch), weight, bias.
def _bn(prefix):
    return [prefix + ".weight", prefix + ".bias", prefix + ".running_mean", prefix + ".running_var"]


EXPECTED_KEYS = (
    ["1.weight"]                                                       # SSC 3 -> 8 (no bias)
    + _bn("2.0.1.0") + ["2.0.1.1.weight"] + _bn("2.0.1.2") + ["2.0.1.3.weight"]            # level 0, block 0 (8 -> 8)
    + _bn("2.2.1.0") + ["2.2.1.1.weight"]                                                 # BN, Conv 8 -> 16
    + _bn("2.2.1.2.0.1.0") + ["2.2.1.2.0.1.1.weight"] + _bn("2.2.1.2.0.1.2") + ["2.2.1.2.0.1.3.weight"]  # level 1 block
    + _bn("2.2.1.3") + ["2.2.1.4.weight"]                                                 # BN, Deconv 16 -> 8
    + ["2.4.0.weight"]                                                                    # NiN 16 -> 8 shortcut
    + _bn("2.4.1.0") + ["2.4.1.1.weight"] + _bn("2.4.1.2") + ["2.4.1.3.weight"]            # block 16 -> 8
    + _bn("3")                                                                            # final BNReLU
)


def test_state_dict_keys_are_the_reference_trees():
    import sparseconvnet as scn

    model = scn.Sequential().add(scn.InputLayer(3, 4096, mode=4)).add(
        scn.SubmanifoldConvolution(3, 3, 8, 3, False)).add(
        scn.UNet(3, 1, [8, 16], True)).add(scn.BatchNormReLU(8)).add(scn.OutputLayer(3))
    sd = model.state_dict()
    assert list(sd.keys()) == EXPECTED_KEYS
    assert sd["2.2.1.1.weight"].shape == (8, 8, 16) and sd["2.2.1.4.weight"].shape == (8, 16, 8)
    assert sd["2.0.1.1.weight"].shape == (27, 8, 8) and sd["2.4.0.weight"].shape == (16, 8)
