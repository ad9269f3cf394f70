"""`sparseconvnet.SCN`: the native-extension surface of the reference, over libinsc.

The reference builds this module with pybind11 (sparseconvnet/SCN/pybind.cpp:13-33,153-258);
here it is a thin Python shim: tensors are checked, turned into raw device pointers and
handed to the C ABI (include/insc.h).  Function names, argument order and the
"caller passes an empty output tensor that the callee resizes" convention follow the
reference (sparseconvnet/SCN/sparseconvnet.h).  Only dimension 3 is provided.

PyTorch is used for device memory and streams only; every computation runs in the HIP
kernels of libinsc.so, and there is no fallback if the library is missing.
"""
import ctypes

import torch

from ._lib import InscError, ensure_init, lib, ptr, stream_ptr  # noqa: F401

I64 = ctypes.c_int64


def _key(t):
    """Hashable form of a spatial-size argument (LongTensor, list or int)."""
    if isinstance(t, torch.Tensor):
        return tuple(int(v) for v in t.tolist())
    if isinstance(t, (list, tuple)):
        return tuple(int(v) for v in t)
    return (int(t),) * 3


def _check_feats(t, name):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.float32 and t.dim() == 2):
        raise TypeError("%s must be a 2-d float32 CUDA tensor" % name)
    if t.stride(1) != 1 and t.numel():
        raise TypeError("%s must have unit stride along channels" % name)
    return t


def _opt(t):
    """Reference convention: an empty tensor stands for 'absent' (sparseconvnet/utils.py:23-24)."""
    if t is None or t.numel() == 0:
        return None
    return t.detach().contiguous()


def _ld(t):
    return t.stride(0) if t.numel() and t.size(0) > 1 else t.size(1)


class _Buf(object):
    """A device array with spare capacity along dim 0 that keeps its rows when it grows."""

    def __init__(self, cols, dtype, device, fill=None):
        self.cols, self.dtype, self.device, self.fill = cols, dtype, device, fill
        self.t = None

    def ensure(self, rows, keep=0):
        cap = 0 if self.t is None else self.t.size(0)
        if rows <= cap:
            return self.t
        new_cap = max(rows, int(cap * 1.5), 1024)
        shape = (new_cap,) if self.cols is None else (new_cap, self.cols)
        if self.fill is None:
            nt = torch.empty(shape, dtype=self.dtype, device=self.device)
        else:
            nt = torch.full(shape, self.fill, dtype=self.dtype, device=self.device)
        if self.t is not None and keep > 0:
            nt[:keep] = self.t[:keep]
        self.t = nt
        return nt


class _Down(object):
    """Size-2 stride-2 link between a fine scale and the next coarser one."""

    def __init__(self, device):
        self.parent = _Buf(None, torch.int32, device)
        self.offset = _Buf(None, torch.int32, device)
        self.child = _Buf(8, torch.int32, device, fill=-1)
        self.n_done = 0  # fine sites linked so far
        self.by_offset = _Buf(None, torch.int32, device)  # fine sites grouped by offset
        self.by_offset_n = 0


class _Scale(object):
    """Active sites of one spatial size and everything derived from them."""

    def __init__(self, device):
        self.device = device
        self.grid = ctypes.c_void_p()
        self.n = 0
        self.nbr = _Buf(27, torch.int32, device)
        self.nbr_n = 0
        self.order = _Buf(None, torch.int32, device)
        self.order_n = 0
        self.plan = None  # tile plan of the 3^3 map in processing order: (map [27*ld] int32, tmask, ld, sched)
        self.plan_n = -1
        self.n_rules = None  # cached number of (in,out) pairs of the 3^3 rulebook
        self.n_rules_at = -1
        self.downs = {}

    def create(self, capacity):
        lib.insc_grid_create(I64(int(capacity)), ctypes.byref(self.grid))

    def capacity(self):
        return int(lib.insc_grid_capacity(self.grid)) if self.grid else 0

    def destroy(self):
        if self.grid:
            lib.insc_grid_destroy(self.grid)
            self.grid = ctypes.c_void_p()

    def coords_view(self):
        """int32 [n,4] view (x,y,z,batch) of the grid's own coordinate table."""
        if self.n == 0:
            return torch.empty((0, 4), dtype=torch.int32, device=self.device)
        addr = lib.insc_grid_coords(self.grid)
        return _from_ptr(addr, (self.n, 4), torch.int32, self.device)


def _from_ptr(addr, shape, dtype, device):
    """Wrap library-owned device memory as a torch tensor (no copy, no ownership)."""
    class _Holder(object):
        pass

    h = _Holder()
    h.__cuda_array_interface__ = {
        "shape": tuple(shape),
        "typestr": {torch.int32: "<i4", torch.float32: "<f4", torch.uint8: "|u1"}[dtype],
        "data": (int(addr), False),
        "version": 2,
        "strides": None,
    }
    return torch.as_tensor(h, device=device)


class Metadata_3(object):
    """Which sites are active at each spatial size, and the rulebooks between them.

    Mirrors Metadata<3> (Metadata/Metadata.h:218-386): grids keyed by spatial size, rulebooks
    cached per size, input-layer bookkeeping.  Site numbering is by first appearance and is
    append-only, so feature rows cached from earlier frames stay valid after `append`.
    """

    def __init__(self):
        self.scales = {}
        self.device = None
        self.input_size = None
        self.clear()

    # ---- reference-visible methods ------------------------------------------------------
    def clear(self):
        for sc in self.scales.values():
            sc.destroy()
        self.scales = {}
        self.input_size = None
        self.mode = None
        self.site_of_point = None  # int32 [P] of the most recent input call
        self.site_of_all_points = None  # all input rows since the last full pass
        self.in_sum = None
        self.in_cnt = None
        self.n_points = 0
        self._pre_exist = {}  # residual frames: per spatial size, this frame's site -> saved site
        self._nbr_pre = {}

    def __del__(self):
        try:
            for sc in self.scales.values():
                sc.destroy()
        except Exception:
            pass

    def setInputSpatialSize(self, spatial_size):
        self.input_size = _key(spatial_size)

    def getSpatialLocations(self, spatial_size):
        """Long [N,4] (x,y,z,batch) on the CPU, rows in site order (Metadata.cpp:793-821)."""
        sc = self.scales.get(_key(spatial_size))
        if sc is None or sc.n == 0:
            return torch.zeros((0, 4), dtype=torch.long)
        return sc.coords_view().cpu().long()

    def getNActive(self, spatial_size):
        sc = self.scales.get(_key(spatial_size))
        return 0 if sc is None else sc.n

    # ---- internals ----------------------------------------------------------------------
    def _bind(self, device):
        if self.device is None:
            self.device = device
            ensure_init(device.index if device.index is not None else torch.cuda.current_device())
        elif self.device != device:
            raise RuntimeError("Metadata is bound to %s, got a tensor on %s" % (self.device, device))

    def scale(self, spatial_size, create_capacity=None):
        k = _key(spatial_size)
        sc = self.scales.get(k)
        if sc is None:
            if create_capacity is None:
                raise RuntimeError("no active sites recorded for spatial size %s" % (k,))
            sc = _Scale(self.device)
            sc.create(create_capacity)
            self.scales[k] = sc
        return sc

    def insert(self, sc, coords4):
        """Insert int32 [P,4] device coordinates; returns int32 [P] site ids."""
        P = coords4.size(0)
        sop = torch.empty(P, dtype=torch.int32, device=self.device)
        n = I64(0)
        lib.insc_grid_insert(sc.grid, ptr(coords4), I64(P), ptr(sop), ctypes.byref(n), stream_ptr())
        sc.n = int(n.value)
        return sop

    def ssc_rulebook(self, spatial_size):
        """Neighbour map + processing order of a scale, brought up to date with its sites."""
        sc = self.scale(spatial_size)
        if sc.nbr_n < sc.n:
            nbr = sc.nbr.ensure(sc.capacity(), keep=sc.nbr_n)
            lib.insc_rulebook_ssc3(sc.grid, I64(sc.nbr_n), I64(sc.n - sc.nbr_n), ptr(nbr), int(sc.nbr_n > 0),
                                   stream_ptr())
            order = sc.order.ensure(sc.capacity(), keep=sc.order_n)
            lib.insc_order_build(sc.grid, ptr(nbr), I64(sc.nbr_n), I64(sc.n - sc.nbr_n), ptr(order), stream_ptr())
            sc.nbr_n = sc.order_n = sc.n
        return sc

    def ssc_plan(self, sc):
        """Tile plan of the scale's 3^3 map (insc_plan_build), rebuilt when sites were added."""
        if sc.plan_n != sc.n:
            ld = (sc.n + 31) // 32 * 32
            if sc.plan is None or sc.plan[2] < ld:
                cap = max(ld, 1024)
                sc.plan = (torch.empty(27 * cap, dtype=torch.int32, device=sc.device),
                           torch.empty(cap // 32 + 1, dtype=torch.int32, device=sc.device), cap,
                           torch.empty(cap // 32 + cap // 128 + 3, dtype=torch.int32, device=sc.device))
            lib.insc_plan_build(ptr(sc.nbr.t), ptr(sc.order.t), None, I64(sc.n), I64(sc.plan[2]), ptr(sc.plan[0]),
                                ptr(sc.plan[1]), ptr(sc.plan[3]), stream_ptr())
            sc.plan_n = sc.n
        return sc.plan

    def n_ssc_rules(self, sc):
        if sc.n_rules_at != sc.n:
            # bookkeeping for the multiply-add counter only (not part of the computation)
            sc.n_rules = int((sc.nbr.t[:sc.n] >= 0).sum().item())
            sc.n_rules_at = sc.n
        return sc.n_rules

    def down_rulebook(self, fine_size, coarse_size):
        """Parent/offset/child maps between two scales (creating the coarse grid on first use)."""
        fk, ck = _key(fine_size), _key(coarse_size)
        fine = self.scale(fk)
        d = fine.downs.get(ck)
        if d is None:
            d = fine.downs[ck] = _Down(self.device)
        coarse = self.scales.get(ck)
        if coarse is None:
            coarse = self.scale(ck, create_capacity=max(fine.capacity(), 1024))
        if d.n_done < fine.n:
            n_new = fine.n - d.n_done
            if coarse.n + n_new > coarse.capacity():
                lib.insc_grid_reserve(coarse.grid, I64(max(2 * coarse.capacity(), coarse.n + n_new)), stream_ptr())
            parent = d.parent.ensure(fine.capacity(), keep=d.n_done)
            offset = d.offset.ensure(fine.capacity(), keep=d.n_done)
            child = d.child.ensure(coarse.capacity(), keep=coarse.n)
            lib.insc_rulebook_down2(fine.grid, coarse.grid, I64(d.n_done), I64(n_new), ptr(parent), ptr(offset),
                                    ptr(child), I64(child.size(0)), stream_ptr())
            n = I64(0)
            lib.insc_grid_size(coarse.grid, ctypes.byref(n), stream_ptr())
            coarse.n = int(n.value)
            d.n_done = fine.n
        return fine, self.scales[ck], d

    def deconv_order(self, fine, d):
        """Fine sites grouped by their offset inside the parent cell (stable), so that a row
        tile of the deconvolution uses one weight slice."""
        if d.by_offset_n != fine.n:
            order = self.ssc_rulebook_for(fine).order.t
            buf = d.by_offset.ensure(fine.capacity())
            lib.insc_order_by_offset(ptr(order), ptr(d.offset.t), I64(fine.n), ptr(buf), stream_ptr())
            d.by_offset_n = fine.n
        return d.by_offset.t

    def pre_exist_map(self, spatial_size, pre_m):
        """int32 [n]: id of each of this site set's sites in `pre_m`'s site set of the same
        spatial size, or -1 (getPreExistMaps, Metadata/Metadata.cpp:609-626)."""
        k = _key(spatial_size)
        hit = self._pre_exist.get(k)
        sc = self.scale(k)
        if hit is None or hit[0] is not pre_m or hit[1].numel() != sc.n:
            pe = torch.empty(max(sc.n, 1), dtype=torch.int32, device=self.device)[:sc.n]
            pre_sc = pre_m.scales.get(k)
            if pre_sc is None or pre_sc.n == 0:
                pe.fill_(-1)
            elif sc.n:
                lib.insc_grid_query(pre_sc.grid, lib.insc_grid_coords(sc.grid), I64(sc.n), ptr(pe), stream_ptr())
            hit = self._pre_exist[k] = (pre_m, pe)
        return hit[1]

    def incre_ssc_map(self, spatial_size, pre_m):
        """int32 [n,27] neighbours, in `pre_m`'s site set, of the sites that are new to it
        (insc_incre_rulebook_ssc3)."""
        k = _key(spatial_size)
        hit = self._nbr_pre.get(k)
        sc = self.scale(k)
        if hit is None or hit[0] is not pre_m or hit[1].size(0) != sc.n:
            nbr = torch.empty((max(sc.n, 1), 27), dtype=torch.int32, device=self.device)[:sc.n]
            pre_sc = pre_m.scales.get(k)
            if pre_sc is None or pre_sc.n == 0:
                nbr.fill_(-1)
            elif sc.n:
                lib.insc_incre_rulebook_ssc3(sc.grid, pre_sc.grid, ptr(self.pre_exist_map(k, pre_m)), I64(sc.n),
                                             ptr(nbr), stream_ptr())
            hit = self._nbr_pre[k] = (pre_m, nbr)
        return hit[1]

    def ssc_rulebook_for(self, sc):
        for k, v in self.scales.items():
            if v is sc:
                return self.ssc_rulebook(k)
        raise RuntimeError("scale not owned by this Metadata")


# =========================================================================================
# helpers shared by the op functions
# =========================================================================================
def _coords4(coords, device):
    """Reference input: Long [P,3] or [P,4] (last column = batch index), usually on the CPU."""
    if coords.dim() != 2 or coords.size(1) not in (3, 4):
        raise ValueError("coords must be [P,3] or [P,4]")
    c = coords.to(device=device, dtype=torch.int32, non_blocking=False)
    if c.size(1) == 3:
        c = torch.cat([c, torch.zeros((c.size(0), 1), dtype=torch.int32, device=device)], 1)
    return c.contiguous()


def _rows_args(rows, count, n_upper):
    """(d_rows, d_n_rows, n_rows) triple for the C ABI."""
    return ptr(rows), ptr(count), I64(int(n_upper))


def packed_weight(weight, K):
    """Weights in the matrix-core operand layout.  The packed copy is kept on the tensor
    object itself and reused until the tensor is modified in place or re-assigned."""
    Cin, Cout = weight.size(-2), weight.size(-1)
    if Cin % 16:
        return None
    tag = (weight._version, weight.data_ptr(), K, Cin, Cout)
    hit = getattr(weight, "_insc_packed", None)
    if hit is not None and hit[0] == tag:
        return hit[1]
    w = weight.detach()
    if not w.is_contiguous():
        w = w.contiguous()
    n = int(lib.insc_conv_packed_floats(int(K), int(Cin), int(Cout)))
    wp = torch.empty(n, dtype=torch.float32, device=weight.device)
    lib.insc_conv_pack_weights(ptr(w), int(K), int(Cin), int(Cout), ptr(wp), stream_ptr())
    try:
        weight._insc_packed = (tag, wp)
    except AttributeError:
        pass
    return wp


def conv_rows(in_f, out_f, weight, bias, nbr, K, rows, count, n_rows):
    """insc_conv_nbr on a row subset; in_f/out_f may be column slices of wider buffers."""
    Cin, Cout = weight.size(-2), weight.size(-1)
    lib.insc_conv_nbr(ptr(in_f), I64(_ld(in_f)), I64(in_f.size(0)), ptr(out_f), I64(_ld(out_f)), ptr(weight),
                      ptr(packed_weight(weight, K)), ptr(bias), ptr(nbr), int(K), ptr(rows), ptr(count),
                      I64(int(n_rows)), int(Cin), int(Cout), None, stream_ptr())


def ssc_rows_planned(in_f, out_f, weight, bias, sc, plan):
    """insc_conv_ssc_plan over all sites of a scale in its processing order."""
    Cin, Cout = weight.size(-2), weight.size(-1)
    lib.insc_conv_ssc_plan(ptr(in_f), I64(_ld(in_f)), I64(in_f.size(0)), ptr(out_f), I64(_ld(out_f)), ptr(weight),
                           ptr(packed_weight(weight, 27)), ptr(bias), ptr(sc.nbr.t), ptr(plan[0]), I64(plan[2]),
                           ptr(plan[1]), ptr(plan[3]), ptr(sc.order.t), None, I64(int(sc.n)), int(Cin), int(Cout),
                           stream_ptr())


def deconv_rows(in_f, out_f, weight, bias, parent, offset, rows, count, n_rows):
    Cin, Cout = weight.size(-2), weight.size(-1)
    lib.insc_deconv_down2(ptr(in_f), I64(_ld(in_f)), I64(in_f.size(0)), ptr(out_f), I64(_ld(out_f)), ptr(weight),
                          ptr(packed_weight(weight, 8)), ptr(bias), ptr(parent), ptr(offset), ptr(rows), ptr(count),
                          I64(int(n_rows)), int(Cin), int(Cout), stream_ptr())


def bn_rows(in_f, out_f, mean, var, gamma, beta, eps, leak, rows, count, n_rows):
    C = in_f.size(1)
    lib.insc_bn_leaky(ptr(in_f), I64(_ld(in_f)), ptr(out_f), I64(_ld(out_f)), ptr(mean), ptr(var), ptr(gamma),
                      ptr(beta), ctypes.c_float(eps), ctypes.c_float(leak), ptr(rows), ptr(count), I64(int(n_rows)),
                      int(C), stream_ptr())


def add_rows(a, b, out, rows, count, n_rows):
    C = a.size(1)
    lib.insc_add(ptr(a), I64(_ld(a)), ptr(b), I64(_ld(b)), ptr(out), I64(_ld(out)), ptr(rows), ptr(count),
                 I64(int(n_rows)), int(C), stream_ptr())


def copy_rows(src, out, rows, count, n_rows):
    C = src.size(1)
    lib.insc_copy_rows(ptr(src), I64(_ld(src)), ptr(out), I64(_ld(out)), ptr(rows), ptr(count), I64(int(n_rows)),
                       int(C), stream_ptr())


def _resize(out, n, c, like):
    """The reference's `output_features.resize_({n, c})` on a caller-created empty tensor."""
    if out.device != like.device or out.dtype != like.dtype:
        out.data = torch.empty((n, c), dtype=like.dtype, device=like.device)
    else:
        out.resize_(n, c)
    return out


# =========================================================================================
# the reference's op functions (dimension 3)
# =========================================================================================
def InputLayer_updateOutput(m, spatialSize, input_coords, input_features, output_features, batchSize, mode):
    """cuda_InputLayer_updateOutput (CUDA/IOLayers.cpp:35-96).  Starts a fresh site set."""
    input_features = _check_feats(input_features, "input_features")
    m.clear()
    m._bind(input_features.device)
    m.setInputSpatialSize(spatialSize)
    m.mode = int(mode)
    P, C = input_features.shape
    if input_coords.size(0) != P:
        raise ValueError("coords and features disagree on the number of rows")
    sc = m.scale(spatialSize, create_capacity=max(int(1.25 * P), 4096))
    _append_points(m, sc, input_coords, input_features)
    _resize(output_features, sc.n, C, input_features)
    lib.insc_input_finish(ptr(m.in_sum.t), ptr(m.in_cnt.t), int(m.mode), ptr(output_features), I64(C), None, None,
                          I64(sc.n), int(C), stream_ptr())


def _append_points(m, sc, input_coords, input_features):
    """Insert points, update per-site sums/counts; returns (site_of_point, n_before)."""
    P, C = input_features.shape
    n_before = sc.n
    c4 = _coords4(input_coords, m.device)
    # checked before anything is inserted, so that a bad frame leaves the site set as it was
    if P and bool(((c4[:, :3] < 0) | (c4[:, :3] > 65535)).any().item() or (c4[:, 3] < 0).any().item()
                  or (c4[:, 3] > 32767).any().item()):
        raise InscError(-5, "a coordinate is outside 0..65535 (batch 0..32767); nothing was inserted")
    sop = m.insert(sc, c4)
    if m.in_sum is None:
        m.in_sum = _Buf(C, torch.float32, m.device, fill=0.0)
        m.in_cnt = _Buf(None, torch.int32, m.device, fill=0)
    m.in_sum.ensure(sc.capacity(), keep=n_before)
    m.in_cnt.ensure(sc.capacity(), keep=n_before)
    feats = input_features.detach().contiguous()
    lib.insc_input_accumulate(ptr(feats), I64(P), int(C), ptr(sop), int(m.mode), ptr(m.in_sum.t), ptr(m.in_cnt.t),
                              I64(sc.n), stream_ptr())
    m.site_of_point = sop
    m.site_of_all_points = sop if m.site_of_all_points is None else torch.cat([m.site_of_all_points, sop])
    m.n_points += P
    return sop, n_before


def OutputLayer_updateOutput(m, input_features, output_features):
    """cuda_OutputLayer_updateOutput (CUDA/IOLayers.cpp:123-145): one row per original input row."""
    input_features = _check_feats(input_features, "input_features")
    sop = m.site_of_all_points
    P, C = sop.numel(), input_features.size(1)
    _resize(output_features, P, C, input_features)
    lib.insc_output_gather(ptr(input_features), I64(_ld(input_features)), ptr(sop), I64(P), int(C),
                           ptr(output_features), stream_ptr())


def SubmanifoldConvolution_updateOutput(inputSize, filterSize, m, input_features, output_features, weight, bias,
                                        dilated_rate=1):
    """cuda_SubmanifoldConvolution_updateOutput (CUDA/Convolution.cpp:152-218); returns multiply-adds."""
    if _key(filterSize) != (3, 3, 3) or int(dilated_rate) != 1:
        raise NotImplementedError("only 3x3x3 submanifold convolutions with dilated_rate 1 are provided")
    input_features = _check_feats(input_features, "input_features")
    sc = m.ssc_rulebook(inputSize)
    w, b = (weight if weight.is_contiguous() else weight.contiguous()), _opt(bias)
    if input_features.size(0) != sc.n or input_features.size(1) != w.size(1) or w.size(0) != 27:
        raise ValueError("feature / weight shapes do not match the active sites")
    _resize(output_features, sc.n, w.size(2), input_features)
    if sc.n == 0:
        return 0.0
    ssc_rows_planned(input_features, output_features, w, b, sc, m.ssc_plan(sc))
    return float(m.n_ssc_rules(sc)) * w.size(1) * w.size(2)


def _check_down(filterSize, filterStride):
    if _key(filterSize) != (2, 2, 2) or _key(filterStride) != (2, 2, 2):
        raise NotImplementedError("only size-2 stride-2 (de)convolutions are provided")


def Convolution_updateOutput(inputSize, outputSize, filterSize, filterStride, m, input_features, output_features,
                             weight, bias):
    """cuda_Convolution_updateOutput (CUDA/Convolution.cpp:52-81), size 2 / stride 2."""
    _check_down(filterSize, filterStride)
    input_features = _check_feats(input_features, "input_features")
    fine, coarse, d = m.down_rulebook(inputSize, outputSize)
    w, b = (weight if weight.is_contiguous() else weight.contiguous()), _opt(bias)
    if input_features.size(0) != fine.n or input_features.size(1) != w.size(1) or w.size(0) != 8:
        raise ValueError("feature / weight shapes do not match the active sites")
    _resize(output_features, coarse.n, w.size(2), input_features)
    if coarse.n == 0:
        return 0.0
    conv_rows(input_features, output_features, w, b, d.child.t, 8, None, None, coarse.n)
    return float(fine.n) * w.size(1) * w.size(2)


def Deconvolution_updateOutput(inputSize, outputSize, filterSize, filterStride, m, input_features, output_features,
                               weight, bias):
    """cuda_Deconvolution_updateOutput (CUDA/Deconvolution.cpp:28-58): input is the coarse scale."""
    _check_down(filterSize, filterStride)
    input_features = _check_feats(input_features, "input_features")
    fine, coarse, d = m.down_rulebook(outputSize, inputSize)
    w, b = (weight if weight.is_contiguous() else weight.contiguous()), _opt(bias)
    if input_features.size(0) != coarse.n or input_features.size(1) != w.size(1) or w.size(0) != 8:
        raise ValueError("feature / weight shapes do not match the active sites")
    _resize(output_features, fine.n, w.size(2), input_features)
    if fine.n == 0:
        return 0.0
    rows = m.deconv_order(fine, d)
    deconv_rows(input_features, output_features, w, b, d.parent.t, d.offset.t, rows, None, fine.n)
    return float(fine.n) * w.size(1) * w.size(2)


def BatchNormalization_updateOutput(input_features, output_features, saveMean, saveInvStd, runningMean, runningVar,
                                    weight, bias, eps, momentum, train, leakiness):
    """cuda_BatchNormalization_updateOutput (CUDA/BatchNormalization.cpp:39-61), inference only."""
    if train:
        raise NotImplementedError("training-mode batch norm is outside the inference path")
    input_features = _check_feats(input_features, "input_features")
    n, C = input_features.shape
    _resize(output_features, n, C, input_features)
    if n:
        ensure_init(input_features.device.index)
        bn_rows(input_features, output_features, runningMean.detach(), runningVar.detach(), _opt(weight), _opt(bias),
                float(eps), float(leakiness), None, None, n)


def NetworkInNetwork_updateOutput(input_features, output_features, weight, bias):
    """cuda_NetworkInNetwork_updateOutput (CUDA/NetworkInNetwork.cpp:9-25)."""
    input_features = _check_feats(input_features, "input_features")
    w, b = (weight if weight.is_contiguous() else weight.contiguous()), _opt(bias)
    n = input_features.size(0)
    _resize(output_features, n, w.size(1), input_features)
    if n:
        ensure_init(input_features.device.index)
        conv_rows(input_features, output_features, w, b, None, 1, None, None, n)
    return float(n) * w.size(0) * w.size(1)


# =========================================================================================
# residual frames: the reference's Incre_* operators (pybind.cpp:218-258).  `m` holds only the
# frame's own points; `pre_m` and the pre_* feature matrices are the state saved by the last
# full forward and are not modified.
# =========================================================================================
def _pre_rows(pre_m, size):
    sc = pre_m.scales.get(_key(size))
    return 0 if sc is None else sc.n


def Incre_InputLayer_updateOutput(m, spatialSize, input_coords, input_features, output_features, batchSize, mode,
                                  pre_m, pre_output_feats):
    """cuda_Incre_InputLayer_updateOutput (CUDA/IOLayers.cpp:290-337)."""
    input_features = _check_feats(input_features, "input_features")
    if m is pre_m:
        raise ValueError("a residual frame needs a Metadata of its own")
    if pre_m.mode is not None and int(mode) != pre_m.mode:
        raise ValueError("input mode differs from the saved frame's")
    m.clear()
    m._bind(input_features.device)
    m.setInputSpatialSize(spatialSize)
    m.mode = int(mode)
    P, C = input_features.shape
    if input_coords.size(0) != P:
        raise ValueError("coords and features disagree on the number of rows")
    sc = m.scale(spatialSize, create_capacity=max(int(1.25 * P), 4096))
    _append_points(m, sc, input_coords, input_features)
    _resize(output_features, sc.n, C, input_features)
    if sc.n == 0:
        return
    if m.mode == 0:  # the reference hands the rows through unchanged in mode 0 (:320-322)
        lib.insc_input_finish(ptr(m.in_sum.t), ptr(m.in_cnt.t), 0, ptr(output_features), I64(C), None, None,
                              I64(sc.n), int(C), stream_ptr())
        return
    pre = _check_feats(pre_output_feats, "pre_output_feats")
    if pre.size(1) != C or pre.size(0) < _pre_rows(pre_m, spatialSize):
        raise ValueError("saved input-layer output does not match the saved site set")
    pe = m.pre_exist_map(spatialSize, pre_m)
    lib.insc_incre_input(ptr(m.in_sum.t), ptr(m.in_cnt.t), int(m.mode), ptr(pe), ptr(pre), I64(_ld(pre)),
                         ptr(pre_m.in_cnt.t), ptr(output_features), I64(C), I64(sc.n), int(C), stream_ptr())


def Incre_OutputLayer_updateOutput(m, input_features, output_features, pre_m, pre_input_feats):
    """cuda_Incre_OutputLayer_updateOutput (CUDA/IOLayers.cpp:339-368): one row per point of the frame."""
    input_features = _check_feats(input_features, "input_features")
    pre = _check_feats(pre_input_feats, "pre_input_feats")
    sop = m.site_of_point
    P, C = sop.numel(), input_features.size(1)
    if pre.size(1) != C or pre.size(0) < _pre_rows(pre_m, m.input_size):
        raise ValueError("saved features do not match the saved site set")
    _resize(output_features, P, C, input_features)
    if P:
        pe = m.pre_exist_map(m.input_size, pre_m)
        lib.insc_incre_output(ptr(input_features), I64(_ld(input_features)), ptr(pre), I64(_ld(pre)), ptr(pe),
                              ptr(sop), I64(P), int(C), ptr(output_features), stream_ptr())


def Incre_SubmanifoldConvolution_updateOutput(inputSize, filterSize, m, input_features, output_features, weight, bias,
                                              pre_m, pre_input_feats, count_muladds=True):
    """cuda_Incre_SubmanifoldConvolution_updateOutput (CUDA/Convolution.cpp:221-303); returns the
    multiply-adds of both rulebooks (count_muladds=False skips the count and its host round trip)."""
    if _key(filterSize) != (3, 3, 3):
        raise NotImplementedError("only 3x3x3 submanifold convolutions are provided")
    input_features = _check_feats(input_features, "input_features")
    pre = _check_feats(pre_input_feats, "pre_input_feats")
    sc = m.ssc_rulebook(inputSize)
    w, b = (weight if weight.is_contiguous() else weight.contiguous()), _opt(bias)
    if input_features.size(0) != sc.n or input_features.size(1) != w.size(1) or w.size(0) != 27:
        raise ValueError("feature / weight shapes do not match the active sites")
    n_pre = _pre_rows(pre_m, inputSize)
    if pre.size(1) != w.size(1) or pre.size(0) < n_pre:
        raise ValueError("saved features do not match the saved site set")
    _resize(output_features, sc.n, w.size(2), input_features)
    if sc.n == 0:
        return 0.0
    nbr_pre = m.incre_ssc_map(inputSize, pre_m)
    Cin, Cout = w.size(1), w.size(2)
    lib.insc_incre_conv_ssc(ptr(input_features), I64(_ld(input_features)), ptr(pre), I64(_ld(pre)), I64(n_pre),
                            ptr(output_features), I64(_ld(output_features)), ptr(w), ptr(packed_weight(w, 27)),
                            ptr(b), ptr(sc.nbr.t), ptr(nbr_pre), I64(sc.n), int(Cin), int(Cout), stream_ptr())
    if not count_muladds:
        return 0.0
    return float(m.n_ssc_rules(sc) + int((nbr_pre >= 0).sum().item())) * Cin * Cout


def Incre_Convolution_updateOutput(inputSize, outputSize, filterSize, filterStride, m, input_features,
                                   output_features, weight, bias):
    """cuda_Incre_Convolution_updateOutput (CUDA/Convolution.cpp:83-113): the plain strided
    convolution on the frame's own rulebook (linear, so exact on differences)."""
    return Convolution_updateOutput(inputSize, outputSize, filterSize, filterStride, m, input_features,
                                    output_features, weight, bias)


def Incre_Deconvolution_updateOutput(inputSize, outputSize, filterSize, filterStride, m, input_features,
                                     output_features, weight, bias, pre_m, pre_input_feats):
    """cuda_Incre_Deconvolution_updateOutput (CUDA/Deconvolution.cpp:61-96): input is the coarse scale."""
    _check_down(filterSize, filterStride)
    input_features = _check_feats(input_features, "input_features")
    pre = _check_feats(pre_input_feats, "pre_input_feats")
    fine, coarse, d = m.down_rulebook(outputSize, inputSize)
    w, b = (weight if weight.is_contiguous() else weight.contiguous()), _opt(bias)
    if input_features.size(0) != coarse.n or input_features.size(1) != w.size(1) or w.size(0) != 8:
        raise ValueError("feature / weight shapes do not match the active sites")
    n_pre = _pre_rows(pre_m, inputSize)
    if pre.size(1) != w.size(1) or pre.size(0) < n_pre:
        raise ValueError("saved features do not match the saved site set")
    _resize(output_features, fine.n, w.size(2), input_features)
    if fine.n == 0:
        return 0.0
    pe_in = m.pre_exist_map(inputSize, pre_m)
    pe_out = m.pre_exist_map(outputSize, pre_m)
    lib.insc_incre_deconv_down2(ptr(input_features), I64(_ld(input_features)), I64(coarse.n), ptr(pre), I64(_ld(pre)),
                                I64(n_pre), ptr(output_features), I64(_ld(output_features)), ptr(w),
                                ptr(packed_weight(w, 8)), ptr(b), ptr(d.parent.t), ptr(d.offset.t), ptr(pe_in),
                                ptr(pe_out), I64(fine.n), int(w.size(1)), int(w.size(2)), stream_ptr())
    return float(fine.n) * w.size(1) * w.size(2)


def Incre_BatchNormalization_updateOutput(input_features, output_features, saveMean, saveInvStd, runningMean,
                                          runningVar, weight, bias, eps, momentum, train, leakiness, m, pre_m,
                                          pre_output_feats, pre_input_feats, inputSize):
    """cuda_Incre_BatchNormalization_updateOutput (CUDA/BatchNormalization.cpp:63-91), inference only."""
    if train:
        raise NotImplementedError("training-mode batch norm is outside the inference path")
    input_features = _check_feats(input_features, "input_features")
    pre_in = _check_feats(pre_input_feats, "pre_input_feats")
    pre_out = _check_feats(pre_output_feats, "pre_output_feats")
    n, C = input_features.shape
    n_pre = _pre_rows(pre_m, inputSize)
    if pre_in.size(1) != C or pre_out.size(1) != C or pre_in.size(0) < n_pre or pre_out.size(0) < n_pre:
        raise ValueError("saved features do not match the saved site set")
    if n != m.getNActive(inputSize):
        raise ValueError("features do not match the active sites")
    _resize(output_features, n, C, input_features)
    if n:
        pe = m.pre_exist_map(inputSize, pre_m)
        mean, var, g, b = runningMean.detach(), runningVar.detach(), _opt(weight), _opt(bias)
        lib.insc_incre_bn_leaky(ptr(input_features), I64(_ld(input_features)), ptr(output_features),
                                I64(_ld(output_features)), ptr(mean), ptr(var), ptr(g), ptr(b),
                                ctypes.c_float(eps), ctypes.c_float(leakiness),
                                ptr(pe), ptr(pre_in), I64(_ld(pre_in)), ptr(pre_out), I64(_ld(pre_out)), I64(n),
                                int(C), stream_ptr())


# =========================================================================================
# size-2 stride-2 pooling, unpooling and the dense copy (siblings of the strided convolution:
# they share its rulebook)
# =========================================================================================
def _pool(mode, inputSize, outputSize, poolSize, poolStride, m, input_features, output_features, nFeaturesToDrop):
    _check_down(poolSize, poolStride)
    input_features = _check_feats(input_features, "input_features")
    fine, coarse, d = m.down_rulebook(inputSize, outputSize)
    drop = int(nFeaturesToDrop)
    C = input_features.size(1) - drop
    if input_features.size(0) != fine.n or C <= 0:
        raise ValueError("features do not match the active sites / nFeaturesToDrop too large")
    _resize(output_features, coarse.n, C, input_features)
    if coarse.n:
        src = input_features[:, drop:]
        lib.insc_pool_down2(ptr(src), I64(_ld(input_features)), ptr(d.child.t), I64(coarse.n), int(C), int(mode),
                            ptr(output_features), I64(C), stream_ptr())


def MaxPooling_updateOutput(inputSize, outputSize, poolSize, poolStride, m, input_features, output_features,
                            nFeaturesToDrop):
    """cuda_MaxPooling_updateOutput (CUDA/MaxPooling.cpp:18-36), size 2 / stride 2."""
    _pool(0, inputSize, outputSize, poolSize, poolStride, m, input_features, output_features, nFeaturesToDrop)


def AveragePooling_updateOutput(inputSize, outputSize, poolSize, poolStride, m, input_features, output_features,
                                nFeaturesToDrop):
    """cuda_AveragePooling_updateOutput (CUDA/AveragePooling.cpp:19-39), size 2 / stride 2."""
    _pool(1, inputSize, outputSize, poolSize, poolStride, m, input_features, output_features, nFeaturesToDrop)


def UnPooling_updateOutput(inputSize, outputSize, poolSize, poolStride, m, input_features, output_features,
                           nFeaturesToDrop):
    """cuda_UnPooling_updateOutput (CUDA/UnPooling.cpp:17-37): input is the coarse scale; every
    fine site copies its parent's row."""
    _check_down(poolSize, poolStride)
    input_features = _check_feats(input_features, "input_features")
    fine, coarse, d = m.down_rulebook(outputSize, inputSize)
    drop = int(nFeaturesToDrop)
    C = input_features.size(1) - drop
    if input_features.size(0) != coarse.n or C <= 0:
        raise ValueError("features do not match the active sites / nFeaturesToDrop too large")
    _resize(output_features, fine.n, C, input_features)
    if fine.n:
        src = input_features[:, drop:]
        lib.insc_output_gather(ptr(src), I64(_ld(input_features)), ptr(d.parent.t), I64(fine.n), int(C),
                               ptr(output_features), stream_ptr())


def SparseToDense_updateOutput(inputSize, m, input_features, output_features, nPlanes):
    """cuda_SparseToDense_updateOutput (CUDA/SparseToDense.cpp:16-41): [batch, nPlanes, X, Y, Z]."""
    input_features = _check_feats(input_features, "input_features")
    sc = m.scale(inputSize)
    X, Y, Z = _key(inputSize)
    C = input_features.size(1)
    if input_features.size(0) != sc.n or C != int(nPlanes):
        raise ValueError("features do not match the active sites / nPlanes")
    batch = int(sc.coords_view()[:, 3].max().item()) + 1 if sc.n else 1
    if output_features.device != input_features.device or output_features.dtype != input_features.dtype:
        output_features.data = torch.empty((batch, C, X, Y, Z), dtype=input_features.dtype,
                                           device=input_features.device)
    else:
        output_features.resize_(batch, C, X, Y, Z)
    lib.insc_sparse_to_dense(sc.grid, ptr(input_features), I64(_ld(input_features)), I64(sc.n), int(C), I64(X), I64(Y),
                             I64(Z), int(batch), ptr(output_features), stream_ptr())


def n_rulebook_bits():
    return 32


# =========================================================================================
# label fusion over frames (Result_3 / ResultOfWeight, pybind.cpp:36-45,275-282)
# =========================================================================================
class _Labels(object):
    """Shared front end of the two label tables: the reference's method names and argument
    shapes (Long [P,3] points, float [P,C] scores), tensors on either device."""
    KIND = 0

    def __init__(self, maximum=0.7, device=None):
        self.device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
        ensure_init(self.device.index or 0)
        self.h = ctypes.c_void_p()
        lib.insc_labels_create(I64(1 << 16), self.KIND, ctypes.c_float(float(maximum)), ctypes.byref(self.h))

    def __del__(self):
        try:
            if self.h:
                lib.insc_labels_destroy(self.h)
                self.h = ctypes.c_void_p()
        except Exception:
            pass

    def _args(self, ps, label):
        if ps.dim() == 1:
            ps, label = ps.unsqueeze(0), label.reshape(1, -1)
        c4 = _coords4(ps[:, :3], self.device)
        x = label.detach().to(device=self.device, dtype=torch.float32).contiguous()
        if x.dim() != 2 or x.size(0) != c4.size(0):
            raise ValueError("one row of scores per point is needed")
        return c4, x

    def update(self, ps, label):
        if ps.dim() != 2:
            raise ValueError("update takes a [P,3] list of points")  # the reference asserts the same
        c4, x = self._args(ps, label)
        lib.insc_labels_update(self.h, ptr(c4), ptr(x), I64(x.size(1)), I64(x.size(0)), int(x.size(1)), stream_ptr())

    def multiQuery(self, ps):
        c4 = _coords4(ps[:, :3], self.device)
        out = torch.empty(c4.size(0), dtype=torch.int32, device=self.device)
        lib.insc_labels_query(self.h, ptr(c4), I64(c4.size(0)), ptr(out), stream_ptr())
        return out.cpu().long()

    def query(self, p):
        return int(self.multiQuery(p.reshape(1, -1))[0])

    def __len__(self):
        n = I64(0)
        lib.insc_labels_count(self.h, ctypes.byref(n), stream_ptr())
        return int(n.value)

    def get_all_points_labels(self, with_confidence=False):
        """Long [N,4] rows (x, y, z, label), in order of first appearance (the reference iterates
        its hash map, i.e. in no particular order)."""
        n = len(self)
        out = torch.empty((n, 4), dtype=torch.int32, device=self.device)
        conf = torch.empty(n, dtype=torch.float32, device=self.device) if with_confidence else None
        lib.insc_labels_export(self.h, ptr(out), ptr(conf), I64(n), stream_ptr())
        return (out.cpu().long(), conf.cpu()) if with_confidence else out.cpu().long()

    def finalize(self, points):
        c4 = _coords4(points[:, :3], self.device)
        lib.insc_labels_finalize(self.h, ptr(c4), I64(c4.size(0)), stream_ptr())

    def clear(self):
        lib.insc_labels_clear(self.h, stream_ptr())


class Result_3(_Labels):
    """Result<3> (Metadata/resultHash.h:23-150): one (label, confidence) pair per voxel."""
    KIND = 0

    def set(self, ps, label):
        c4, x = self._args(ps, label)
        lib.insc_labels_set(self.h, ptr(c4), ptr(x), I64(x.size(1)), I64(x.size(0)), int(x.size(1)), stream_ptr())


class ResultOfWeight(_Labels):
    """ResultOfWeight (Metadata/resultHash.h:153-218): running scores per voxel, new = old/2 + row."""
    KIND = 1

    def __init__(self, device=None):
        _Labels.__init__(self, 0.0, device)


# =========================================================================================
# canonical exports used by parity tests: the reference's list-form rulebooks
# =========================================================================================
def ssc_rulebook_lists(m, spatial_size):
    """(counts[27], pairs[R,2]) int32 CPU tensors: RuleBook of Metadata::getSubmanifoldRuleBook."""
    sc = m.ssc_rulebook(spatial_size)
    counts = torch.empty(27, dtype=torch.int32, device=m.device)
    cap = 27 * max(sc.n, 1)
    pairs = torch.empty((cap, 2), dtype=torch.int32, device=m.device)
    tot = I64(0)
    lib.insc_rulebook_pairs(ptr(sc.nbr.t), I64(sc.n), 27, ptr(counts), ptr(pairs), I64(cap), ctypes.byref(tot),
                            stream_ptr())
    return counts.cpu(), pairs[:int(tot.value)].cpu()


def down_rulebook_lists(m, fine_size, coarse_size):
    """(counts[8], pairs[R,2]) of (fine, coarse) pairs grouped by offset: Metadata::getRuleBook."""
    fine, coarse, d = m.down_rulebook(fine_size, coarse_size)
    counts = torch.empty(8, dtype=torch.int32, device=m.device)
    cap = 8 * max(coarse.n, 1)
    pairs = torch.empty((cap, 2), dtype=torch.int32, device=m.device)
    tot = I64(0)
    lib.insc_rulebook_pairs(ptr(d.child.t), I64(coarse.n), 8, ptr(counts), ptr(pairs), I64(cap), ctypes.byref(tot),
                            stream_ptr())
    return counts.cpu(), pairs[:int(tot.value)].cpu()
