"""Identity (reference: sparseconvnet/identity.py)."""
from torch.nn import Module


class Identity(Module):
    def forward(self, input, increment=False):
        return input

    def input_spatial_size(self, out_size):
        return out_size
