"""Dirty-site bookkeeping of the incremental forward.

A DirtySet names the rows of one feature matrix that changed in the current frame.  Layers
map it to the rows of their output that must be recomputed:
  3x3x3 submanifold convolution : dilate by one site, restricted to active sites
  pointwise layers              : unchanged
  size-2 stride-2 convolution   : parents of the dirty sites
  size-2 stride-2 deconvolution : children of the dirty coarse sites
  add / join                    : union
Every one of these maps only grows a set, so a set derived from another contains it; the
`ancestors` record lets unions of related sets be answered without touching the GPU.

The reference's incremental path does not dilate (CUDA/Convolution.cpp:221-303) and is an
approximation; recomputing exactly the dirty rows from cached inputs makes an incremental
frame equal to a full forward over all points seen so far.

Both kinds of incremental forward are provided.  `increment=True` selects the default kind
(set_mode), `increment="exact"` / `increment="residual"` name one: "exact" is the dirty-set
path above, "residual" the reference's own (features of a frame are differences to the state
saved by the last full or exact forward, SCN.Incre_*; the saved state is left untouched).
"""
import ctypes
import itertools

import torch

from ._lib import lib, ptr, stream_ptr

I64 = ctypes.c_int64
_ids = itertools.count()
_KINDS = ("exact", "residual")
_mode = "exact"


def set_mode(mode):
    """Kind of incremental forward that `increment=True` stands for: "exact" or "residual"."""
    global _mode
    if mode not in _KINDS:
        raise ValueError("incremental mode must be one of %s" % (_KINDS,))
    _mode = mode


def get_mode():
    return _mode


def kind(increment):
    """None for a full forward, else "exact" or "residual"."""
    if isinstance(increment, str):
        if increment not in _KINDS:
            raise ValueError("increment must be a bool or one of %s" % (_KINDS,))
        return increment
    return _mode if increment else None


class DirtySet(object):
    def __init__(self, scale, mask, ancestors=()):
        self.id = next(_ids)
        self.scale = scale  # SCN._Scale the rows belong to
        self.mask = mask  # uint8 [>= n]
        self.n_upper = scale.n
        self.ancestors = frozenset(ancestors) | {self.id}
        self._rows = {}
        self._derived = {}

    def rows(self, order=None, tag="ssc"):
        """(rows int32 list, device count) of the dirty sites, taken in the given processing order."""
        if tag not in self._rows:
            dev = self.mask.device
            rows = torch.empty(max(self.n_upper, 1), dtype=torch.int32, device=dev)
            count = torch.empty(1, dtype=torch.int32, device=dev)
            lib.insc_dirty_compact(ptr(self.mask), ptr(order), None, I64(self.n_upper), ptr(rows), ptr(count), None,
                                   stream_ptr())
            self._rows[tag] = (rows, count)
        return self._rows[tag]

    def count(self):
        """Number of dirty rows (synchronises; for reporting only)."""
        return int(self.rows(self.scale.order.t)[1].item())


def _new_mask(scale, device):
    return torch.zeros(max(scale.capacity(), 1), dtype=torch.uint8, device=device)


def from_points(scale, site_of_point):
    d = DirtySet(scale, _new_mask(scale, site_of_point.device))
    lib.insc_dirty_mark(ptr(site_of_point), I64(site_of_point.numel()), ptr(d.mask), stream_ptr())
    return d


def all_rows(scale, device):
    d = DirtySet(scale, torch.ones(max(scale.capacity(), 1), dtype=torch.uint8, device=device))
    return d


def dilate(d):
    """Rows whose 3x3x3 neighbourhood contains a dirty row."""
    if "dilate" not in d._derived:
        sc = d.scale
        out = DirtySet(sc, _new_mask(sc, d.mask.device), d.ancestors)
        lib.insc_dirty_dilate3(ptr(sc.nbr.t), ptr(d.mask), ptr(out.mask), None, I64(sc.n), stream_ptr())
        d._derived["dilate"] = out
    return d._derived["dilate"]


def parents(d, coarse, down):
    key = ("parents", id(coarse))
    if key not in d._derived:
        out = DirtySet(coarse, _new_mask(coarse, d.mask.device), d.ancestors)
        lib.insc_dirty_parents(ptr(down.parent.t), ptr(d.mask), ptr(out.mask), None, I64(d.scale.n), stream_ptr())
        d._derived[key] = out
    return d._derived[key]


def children(d, fine, down):
    key = ("children", id(fine))
    if key not in d._derived:
        out = DirtySet(fine, _new_mask(fine, d.mask.device), d.ancestors)
        lib.insc_dirty_children(ptr(down.parent.t), ptr(d.mask), ptr(out.mask), None, I64(fine.n), stream_ptr())
        d._derived[key] = out
    return d._derived[key]


def union(a, b):
    if a is b or a.id in b.ancestors:
        return b
    if b.id in a.ancestors:
        return a
    if a.scale is not b.scale:
        raise RuntimeError("union of dirty sets of different scales")
    out = DirtySet(a.scale, torch.empty_like(a.mask), a.ancestors | b.ancestors)
    lib.insc_dirty_or(ptr(a.mask), ptr(b.mask), ptr(out.mask), None, I64(a.scale.n), stream_ptr())
    return out
