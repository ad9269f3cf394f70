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
    return num > 0 and bin(num).count("1") == 1


def _checkpoint_file(exp_name, name2, epoch, digits=4):
    return "%s-%0*d-%s.pth" % (exp_name, digits, epoch, name2)


def checkpoint_save(model, exp_name, name2, epoch, use_cuda=True):
    """Writes the state_dict to '<exp_name>-<epoch:04d>-<name2>.pth' and drops the file of epoch - 1
    unless that number is a power of two, so a long run keeps a logarithmic trail
    (reference: sparseconvnet/utils.py:222-233; same file names, same pruning rule).  The
    tensors are written from host memory; with use_cuda the model goes back to the GPU."""
    model.cpu()
    torch.save(model.state_dict(), _checkpoint_file(exp_name, name2, epoch))
    if use_cuda:
        model.cuda()
    stale = _checkpoint_file(exp_name, name2, epoch - 1)
    if not is_power2(epoch - 1) and os.path.isfile(stale):
        os.remove(stale)


def checkpoint_restore(model, exp_name, name2, use_cuda=True, epoch=0):
    """Loads epoch `epoch`, or with epoch == 0 the newest '<exp_name>-*-<name2>.pth', into the
    model and returns the number of the epoch to run next; without any file the model is left as
    it is and 1 is returned (reference: sparseconvnet/utils.py:201-218).  Files are read with
    weights_only=True: tensors only, nothing in the file is executed."""
    path = None
    if epoch > 0:
        # the reference asks for nine digits here although it writes four; accept both
        for digits in (9, 4):
            if os.path.isfile(_checkpoint_file(exp_name, name2, epoch, digits)):
                path = _checkpoint_file(exp_name, name2, epoch, digits)
                break
        if path is None:
            raise AssertionError("no checkpoint %s" % _checkpoint_file(exp_name, name2, epoch))
    else:
        found = sorted(glob.glob(exp_name + "-*-" + name2 + ".pth"))
        if found:
            path = found[-1]
            epoch = int(path[len(exp_name) + 1:len(path) - len(name2) - 5])
    if use_cuda:
        model.cpu()
    if path is not None:
        model.load_state_dict(torch.load(path, weights_only=True))
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
