"""The network of the reference's usage example (model.py:8-26): InputLayer(mode 4) ->
SSC 3->m -> UNet(reps 2, planes m..L*m, residual) -> BNReLU -> OutputLayer -> Linear(m, 20).
Weights follow the modules' own init laws from one seeded generator; batch-norm running
statistics are seeded random values (mean ~ N(0, 0.2), var ~ U[0.5, 2], gamma ~ U[0.5, 1.5],
beta ~ N(0, 0.1)) so that the inference path is exercised with non-trivial affine maps."""
import torch
import torch.nn as nn


class NaiveUNet(nn.Module):
    def __init__(self, m=32, levels=7, full_scale=4096, seed=4, classes=20):
        nn.Module.__init__(self)
        import sparseconvnet as scn

        torch.manual_seed(seed)
        self.sparseModel = scn.Sequential().add(
            scn.InputLayer(3, full_scale, mode=4)).add(
            scn.SubmanifoldConvolution(3, 3, m, 3, False)).add(
            scn.UNet(3, 2, [m * (i + 1) for i in range(levels)], True)).add(
            scn.BatchNormReLU(m)).add(
            scn.OutputLayer(3))
        self.linear = nn.Linear(m, classes)
        g = torch.Generator().manual_seed(seed + 1)
        for mod in self.modules():
            if isinstance(mod, scn.BatchNormalization):
                mod.running_mean.copy_(torch.randn(mod.nPlanes, generator=g) * 0.2)
                mod.running_var.copy_(torch.rand(mod.nPlanes, generator=g) * 1.5 + 0.5)
                with torch.no_grad():
                    mod.weight.copy_(torch.rand(mod.nPlanes, generator=g) + 0.5)
                    mod.bias.copy_(torch.randn(mod.nPlanes, generator=g) * 0.1)
        self.eval()

    def forward(self, x, increment=False):
        x = self.sparseModel(x, increment)
        return self.linear(x)
