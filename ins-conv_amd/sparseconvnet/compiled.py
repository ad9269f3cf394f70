"""Run a sparseconvnet module tree through the native network executor (insc_net_*).

    net = scn.compile(sparse_model)          # Sequential starting with InputLayer, ending with OutputLayer
    feats = net([coords, features, batch], increment=False)     # same call shape as the module
    feats = net([new_coords, new_features, batch], increment=True)
    net = scn.compile(sparse_model, residual=True)               # also allows increment="residual"

The module path issues one C call per layer from Python; this path hands the whole frame to
one C call, so an incremental frame costs a few hundred kernel launches and no Python work.
Results are bit-identical to the module path.  Parameters are read in place (device
pointers).  A parameter that moved (`.to()`, `.cpu()` + `.cuda()`) or changed through torch
(`load_state_dict`, `checkpoint_restore`, `copy_`, an optimizer step: anything that bumps the
tensor's version counter) is noticed at the next call: the executor is pointed at the current
tensors, re-packs its weights and forgets the rows cached by earlier frames, so the next frame
must be a full one (an incremental frame raises instead of mixing rows computed with old and
new parameters).  Writes torch cannot see (a raw kernel on the parameter's memory) need
`refresh()`.  JoinTable takes two inputs (the U-Net's skip connection); wider joins run on the
module path only.
"""
import ctypes

import torch

from . import SCN
from ._lib import ensure_init, lib, ptr, stream_ptr

I64 = ctypes.c_int64
_KIND = {"ssc": 0, "conv": 2, "deconv": 3, "nin": 4}


class CompiledNet(object):
    def __init__(self, model, capacity_sites=1 << 18, residual=False):
        import sparseconvnet as scn

        mods = list(model)
        if not (isinstance(mods[0], scn.InputLayer) and isinstance(mods[-1], scn.OutputLayer)):
            raise ValueError("the model must start with an InputLayer and end with an OutputLayer")
        self.model = model
        self.input_layer, self.output_layer = mods[0], mods[-1]
        self.device = next(model.parameters()).device
        if self.device.type != "cuda":
            raise ValueError("move the model to the GPU before compiling it")
        ensure_init(self.device.index or 0)
        levels = 1 + sum(1 for m in model.modules() if isinstance(m, scn.Convolution))
        first = next(m for m in model.modules() if hasattr(m, "nIn") or hasattr(m, "nPlanes"))
        self.in_channels = getattr(first, "nIn", None) or first.nPlanes
        self.h = ctypes.c_void_p()
        lib.insc_net_create(levels, int(self.in_channels), int(self.input_layer.mode), ctypes.byref(self.h))
        self._keep = []  # tensors whose storage the executor points into
        self._bound = []  # (op index, module) of every op with parameters
        self._sig_tensors = None
        self._level = {0: 0}
        self._chan = {0: self.in_channels}
        x = 0
        for m in mods[1:-1]:
            x = self._trace(m, x)
        self.out_tensor = x
        self.out_channels = self._chan[x]
        self._n_points = 0  # points since the last full frame (rows of an all_points output)
        self.residual = bool(residual)
        if self.residual:
            lib.insc_net_enable_residual(self.h)
        lib.insc_net_finalize(self.h, int(x), I64(int(capacity_sites)), stream_ptr())
        self._sig = self._signature()

    def __del__(self):
        try:
            if self.h:
                lib.insc_net_destroy(self.h)
                self.h = ctypes.c_void_p()
        except Exception:
            pass

    # ---- tracing --------------------------------------------------------------------------
    def _new(self, level, C):
        t = ctypes.c_int(0)
        lib.insc_net_tensor(self.h, int(level), int(C), ctypes.byref(t))
        self._level[t.value], self._chan[t.value] = level, C
        return t.value

    def _dev(self, t):
        if t is None:
            return None
        t = t.detach()
        if not t.is_contiguous():
            raise ValueError("parameters must be contiguous")
        if t.device != self.device:
            raise ValueError("a parameter is on %s, the compiled net on %s" % (t.device, self.device))
        self._keep.append(t)
        return ptr(t)

    @staticmethod
    def _params(m):
        """The tensors op parameters are read from, in the order of insc_net_rebind_op."""
        import sparseconvnet as scn

        bias = getattr(m, "bias", None)
        if isinstance(m, scn.BatchNormalization):
            return (None, None, m.running_mean, m.running_var, getattr(m, "weight", None), bias)
        return (m.weight, bias, None, None, None, None)

    def _bind_op(self, m):
        self._bound.append((int(lib.insc_net_op_count(self.h)) - 1, m))

    def _signature(self):
        """(addresses, versions) of every tensor the ops read (some 330 for the 7-level U-Net).  The
        tensor objects are looked up once per binding: torch moves and reloads parameters in place
        (`.to()`, `load_state_dict`), which the address and the version counter show."""
        ts = self._sig_tensors
        if ts is None:
            ts = self._sig_tensors = [t for _, m in self._bound for t in self._params(m) if t is not None]
        return [t.data_ptr() for t in ts], [t._version for t in ts]

    def _rebind(self):
        keep, self._keep, self._sig_tensors = self._keep, [], None
        for op, m in self._bound:
            lib.insc_net_rebind_op(self.h, op, *[self._dev(t) for t in self._params(m)])
        lib.insc_net_refresh_weights(self.h, stream_ptr())
        self._sig = self._signature()
        del keep  # (the old storages stayed alive until the executor stopped pointing at them)

    def _trace(self, m, x):
        import sparseconvnet as scn

        if isinstance(m, scn.ConcatTable):
            return [self._trace(c, x) for c in m._modules.values()]
        if isinstance(m, scn.Sequential):
            for c in m:
                x = self._trace(c, x)
            return x
        if isinstance(m, scn.Identity):
            return x
        if isinstance(m, scn.AddTable):
            out = x[0]
            for t in x[1:]:
                o = self._new(self._level[out], self._chan[out])
                lib.insc_net_op_add(self.h, out, t, o)
                out = o
            return out
        if isinstance(m, scn.JoinTable):
            if len(x) != 2:
                raise NotImplementedError("JoinTable of two inputs")
            o = self._new(self._level[x[0]], self._chan[x[0]] + self._chan[x[1]])
            lib.insc_net_join(self.h, x[0], x[1], o)
            return o
        bias = getattr(m, "bias", None)
        if isinstance(m, scn.BatchNormalization):
            o = self._new(self._level[x], m.nPlanes)
            lib.insc_net_op_bn(self.h, x, o, self._dev(m.running_mean), self._dev(m.running_var),
                               self._dev(getattr(m, "weight", None)), self._dev(bias), ctypes.c_float(m.eps),
                               ctypes.c_float(m.leakiness))
            self._bind_op(m)
            return o
        if isinstance(m, scn.SubmanifoldConvolution):
            if SCN._key(m.filter_size) != (3, 3, 3) or m.dilated_rate != 1:
                raise NotImplementedError("3x3x3 submanifold convolutions with dilated_rate 1")
            kind, dl = "ssc", 0
        elif isinstance(m, scn.Convolution):
            SCN._check_down(m.filter_size, m.filter_stride)
            kind, dl = "conv", 1
        elif isinstance(m, scn.Deconvolution):
            SCN._check_down(m.filter_size, m.filter_stride)
            kind, dl = "deconv", -1
        elif isinstance(m, scn.NetworkInNetwork):
            kind, dl = "nin", 0
        else:
            raise NotImplementedError("no executor op for %s" % type(m).__name__)
        o = self._new(self._level[x] + dl, m.nOut)
        lib.insc_net_op_conv(self.h, _KIND[kind], x, o, self._dev(m.weight), self._dev(bias))
        self._bind_op(m)
        return o

    # ---- running --------------------------------------------------------------------------
    def refresh(self):
        """Point the executor at the model's current parameter tensors and re-pack the weights."""
        self._rebind()

    def _coords(self, coords):
        """int32 on the device.  The reference's callers pass int64 coordinates, on the host
        (ioLayers.py:52-69 converts to a CPU LongTensor) or on the GPU (demo.py:20): narrowed on
        the side where they are, so that the host-to-device copy carries half the bytes."""
        if coords.dtype != torch.int32:
            coords = coords.to(torch.int32)
        return coords.to(self.device).contiguous()

    def _changed(self):
        """Whether a parameter moved or changed since the weights were packed.  Looked at AFTER a
        frame has been enqueued - the walk over the tensors costs the host some 60 us, which the
        GPU then spends on the frame instead of waiting for it; the stale pointers stay valid
        memory because `_keep` holds the old storages."""
        return self._signature() != self._sig

    def __call__(self, input, increment=False, all_points=None):
        coords, feats = input[0], input[1]
        from . import incremental
        if incremental.kind(increment) == "residual":
            out = self._residual(coords, feats)
            if self._changed():
                self._rebind()
                raise RuntimeError("the model's parameters changed since the last full frame: run a full frame "
                                   "(increment=False) before the next residual frame")
            return out
        increment = bool(increment)
        if all_points is None:
            all_points = (not increment) or self.output_layer.all_points
        c = self._coords(coords)
        f = feats.detach().to(device=self.device, dtype=torch.float32).contiguous()
        P = c.size(0)
        rows = (self._n_points if increment else 0) + P if all_points else P
        out = torch.empty((rows, self.out_channels), dtype=torch.float32, device=self.device)
        n = I64(0)
        for attempt in (0, 1):
            lib.insc_net_forward(self.h, ptr(c), int(c.size(1)), ptr(f), I64(P), int(increment), ptr(out),
                                 int(bool(all_points)), ctypes.byref(n), stream_ptr())
            if attempt or not self._changed():
                break
            # the frame just enqueued read parameters that have moved or changed since they were packed
            self._rebind()
            if increment:
                raise RuntimeError("the model's parameters changed since the last full frame: the cached rows "
                                   "belong to the old parameters; run a full frame (increment=False) first")
        self._n_points = (self._n_points if increment else 0) + P
        self.n_sites = int(n.value)
        self._timed = getattr(self, "_profiling", False)
        return out

    def _residual(self, coords, feats):
        """The reference's own incremental frame (SCN.Incre_* semantics) in one C call: rows of
        the frame's points only; the saved state is not touched."""
        if not self.residual:
            raise RuntimeError("compile the model with residual=True to run residual frames")
        c = self._coords(coords)
        f = feats.detach().to(device=self.device, dtype=torch.float32).contiguous()
        P = c.size(0)
        out = torch.empty((P, self.out_channels), dtype=torch.float32, device=self.device)
        n = I64(0)
        lib.insc_net_forward_residual(self.h, ptr(c), int(c.size(1)), ptr(f), I64(P), ptr(out), ctypes.byref(n),
                                      stream_ptr())
        self.n_sites_frame = int(n.value)
        return out

    def set_order_refresh(self, percent):
        """Share (in percent) of appended sites at which an incremental frame re-sorts the processing
        orders of all scales (insc_net_set_order_refresh); 0 switches the re-sorting off."""
        lib.insc_net_set_order_refresh(self.h, int(percent))

    def profile(self, enable=True):
        """Switch phase timing on/off; returns the last timed frame's phases in ms as a dict
        (structure, dirty, layers, output), or None if no frame was timed yet."""
        ms = (ctypes.c_float * 4)()
        have = getattr(self, "_profiling", False)
        lib.insc_net_profile(self.h, int(bool(enable)), ms if have and getattr(self, "_timed", False) else None)
        out = dict(zip(("structure", "dirty", "layers", "output"), [float(v) for v in ms])) if have and getattr(self, "_timed", False) else None
        self._profiling, self._timed = bool(enable), False
        return out

    def dirty_rows(self):
        """Rows of every dirty set of the last exact incremental frame, per scale: a list (one entry
        per scale) of lists of (kind, rows) in program order; kind is "input", "dilate", "parents",
        "children" or "union"."""
        n = ctypes.c_int(0)
        cap = 512
        lv, kd, rows = (ctypes.c_int * cap)(), (ctypes.c_int * cap)(), (I64 * cap)()
        lib.insc_net_dirty_counts(self.h, cap, ctypes.byref(n), lv, kd, rows, stream_ptr())
        names = ("input", "dilate", "parents", "children", "union")
        out = [[] for _ in range(max(lv[:n.value], default=-1) + 1)]
        for i in range(n.value):
            out[lv[i]].append((names[kd[i]], int(rows[i])))
        return out

    def frame_work(self):
        """What every convolution of the last frame worked on: a list of dicts (kind, level, cin, cout,
        rows, rules, slots) in program order; useful multiply-adds of a layer = rules * cin * cout, the
        matrix cores are issued slots * cin * cout (insc_net_frame_work).  Synchronises."""
        cap = 256
        n = ctypes.c_int(0)
        kd, lv, ci, co = ((ctypes.c_int * cap)() for _ in range(4))
        rows, rules, slots = ((I64 * cap)() for _ in range(3))
        lib.insc_net_frame_work(self.h, cap, ctypes.byref(n), kd, lv, ci, co, rows, rules, slots, stream_ptr())
        names = {0: "ssc", 2: "conv", 3: "deconv", 4: "nin"}
        return [dict(kind=names[kd[i]], level=lv[i], cin=ci[i], cout=co[i], rows=int(rows[i]), rules=int(rules[i]),
                     slots=int(slots[i])) for i in range(n.value)]

    def sites_per_level(self):
        a = (I64 * 16)()
        lib.insc_net_counts(self.h, a, None)
        return [int(v) for v in a]


def compile(model, capacity_sites=1 << 18, residual=False):
    return CompiledNet(model, capacity_sites, residual)
