"""Small helpers with the reference's names (sparseconvnet/utils.py:13-24)."""
import torch


def toLongTensor(dimension, x):
    if isinstance(x, torch.Tensor) and x.dtype == torch.long:
        return x
    if isinstance(x, (list, tuple)):
        assert len(x) == dimension
        return torch.LongTensor(list(x))
    return torch.LongTensor(dimension).fill_(int(x))


def optionalTensor(a, b):
    return getattr(a, b) if hasattr(a, b) else torch.Tensor()


class StateBuf(object):
    """Backing store of a layer's cached output.

    A full forward allocates an exact-size output and hands it over with `adopt`; incremental
    forwards call `grow`, which returns a [n, C] view whose first `keep` rows still hold the
    cached values (the store is reallocated with headroom when the site count outgrows it).
    """

    def __init__(self):
        self.buf = None

    def adopt(self, t):
        self.buf = t
        return t

    def new(self, n, C, like):
        self.buf = torch.empty((n, C), dtype=torch.float32, device=like.device)
        return self.buf

    def grow(self, n, keep):
        if self.buf is None:
            raise RuntimeError("incremental forward before any full forward (no cached state)")
        if self.buf.size(0) < n:
            nb = torch.empty((max(n, int(1.5 * self.buf.size(0))), self.buf.size(1)), dtype=self.buf.dtype,
                             device=self.buf.device)
            nb[:keep] = self.buf[:keep]
            self.buf = nb
        return self.buf[:n]
