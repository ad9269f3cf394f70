"""Small helpers with the reference's names (sparseconvnet/utils.py:13-24, 201-233)."""
import glob
import os

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


# ---------------------------------------------------------------------------------------------
# checkpoints (sparseconvnet/utils.py:201-233) and weights trained elsewhere
# ---------------------------------------------------------------------------------------------
def is_power2(num):
    return num != 0 and ((num & (num - 1)) == 0)


def checkpoint_save(model, exp_name, name2, epoch, use_cuda=True):
    """state_dict to '<exp_name>-<epoch:04d>-<name2>.pth'; the previous epoch's file is removed
    unless its number is a power of two (utils.py:222-233)."""
    f = exp_name + "-%04d-" % epoch + name2 + ".pth"
    model.cpu()
    torch.save(model.state_dict(), f)
    if use_cuda:
        model.cuda()
    epoch = epoch - 1
    f = exp_name + "-%04d-" % epoch + name2 + ".pth"
    if os.path.isfile(f) and not is_power2(epoch):
        os.remove(f)


def checkpoint_restore(model, exp_name, name2, use_cuda=True, epoch=0):
    """Load the given epoch, or the latest '<exp_name>-*-<name2>.pth'; returns the next epoch
    number (utils.py:201-218).  Files are read with weights_only=True (tensors only)."""
    if use_cuda:
        model.cpu()
    if epoch > 0:
        f = exp_name + "-%09d-" % epoch + name2 + ".pth"  # the reference's pattern for an explicit epoch
        if not os.path.isfile(f):
            f = exp_name + "-%04d-" % epoch + name2 + ".pth"  # what checkpoint_save writes
        assert os.path.isfile(f), f
        model.load_state_dict(torch.load(f, weights_only=True))
    else:
        fs = sorted(glob.glob(exp_name + "-*-" + name2 + ".pth"))
        if len(fs) > 0:
            f = fs[-1]
            model.load_state_dict(torch.load(f, weights_only=True))
            epoch = int(f[len(exp_name) + 1:-len(name2) - 5])
    if use_cuda:
        model.cuda()
    return epoch + 1


def ssc_offset_permutation():
    """perm with perm[k_xmajor] = k_zmajor for the 27 offsets of a 3^3 filter.

    This package (and upstream SparseConvNet, and the reference's GPU path) numbers the offset
    (dx,dy,dz) as (dx+1)*9 + (dy+1)*3 + (dz+1); the reference's rewritten CPU rule generator
    numbers it (dz+1)*9 + (dy+1)*3 + (dx+1) (Metadata/SubmanifoldConvolutionRules.h:39-52).
    The permutation is its own inverse."""
    return torch.tensor([(k % 3) * 9 + ((k // 3) % 3) * 3 + k // 9 for k in range(27)], dtype=torch.long)


def convert_zmajor_state_dict(state_dict):
    """A copy of a state_dict whose 3^3 filters ([27, nIn, nOut] weights) were trained against the
    z-major offset numbering, re-indexed for this package."""
    perm = ssc_offset_permutation()
    out = {}
    for k, v in state_dict.items():
        if torch.is_tensor(v) and v.dim() == 3 and v.size(0) == 27:
            out[k] = v.index_select(0, perm.to(v.device)).contiguous()
        else:
            out[k] = v
    return out
