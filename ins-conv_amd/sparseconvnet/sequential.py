"""Sequential container that threads the `increment` flag (reference: sparseconvnet/sequential.py:9-25)."""
import torch


class Sequential(torch.nn.Sequential):
    def input_spatial_size(self, out_size):
        for m in reversed(self._modules):
            out_size = self._modules[m].input_spatial_size(out_size)
        return out_size

    def add(self, module):
        self._modules[str(len(self._modules))] = module
        return self

    def forward(self, input, increment=False):
        for module in self:
            input = module(input, increment)
        return input
