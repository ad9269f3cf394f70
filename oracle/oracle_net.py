"""Runs a network built from the sparseconvnet mirror modules on the CPU oracle.

The module tree (Sequential / ConcatTable / AddTable / JoinTable / layers) is walked exactly
as Sequential.forward does, but every layer is evaluated with the oracle's restatement of the
reference's CPU path, on numpy arrays.  Used to check whole-network results of the HIP path.
"""
import numpy as np

from . import oracle as orc


class OTensor(object):
    def __init__(self, feats, size, ctx):
        self.features, self.spatial_size, self.ctx = feats, tuple(int(v) for v in size), ctx


class Ctx(object):
    """Sites per spatial size and the rulebooks between them (the oracle's Metadata)."""

    def __init__(self):
        self.coords = {}
        self.ssc = {}
        self.down = {}

    def ssc_rules(self, size):
        if size not in self.ssc:
            _, counts, pairs = orc.ssc_rules(self.coords[size])
            self.ssc[size] = (counts, pairs)
        return self.ssc[size]

    def down_rules(self, fine, coarse):
        if (fine, coarse) not in self.down:
            parent, off, cc = orc.down2_rules(self.coords[fine])
            self.coords[coarse] = cc
            self.down[(fine, coarse)] = orc.down2_pairs(parent, off)
        return self.down[(fine, coarse)]


def _np(t):
    return None if t is None else t.detach().cpu().numpy()


def forward(module, x, save=None):
    """Full forward.  `save` (a dict) receives, per module, the (input, output) pair that a
    residual frame refers to later (the reference's save_* attributes)."""
    y = _forward(module, x, save)
    if save is not None and not isinstance(y, list):
        save[id(module)] = (x, y)
    return y


def _forward(module, x, save):
    import sparseconvnet as scn

    name = type(module).__name__
    if isinstance(module, scn.InputLayer):
        coords, feats = x[0], x[1]
        ctx = Ctx()
        size = tuple(int(v) for v in module.spatial_size.tolist())
        sop, sc, cnt = orc.grid_build(np.asarray(coords))
        ctx.coords[size] = sc
        ctx.site_of_point = sop
        ctx.count = cnt
        f = orc.input_forward(np.asarray(feats), sop, cnt, mode=module.mode)
        return OTensor(f, size, ctx)
    if isinstance(module, scn.OutputLayer):
        return orc.output_forward(x.features, x.ctx.site_of_point)
    if isinstance(module, scn.ConcatTable):
        return [forward(m, x, save) for m in module._modules.values()]
    if isinstance(module, scn.AddTable):
        f = x[0].features
        for t in x[1:]:
            f = f + t.features
        return OTensor(f.astype(x[0].features.dtype), x[0].spatial_size, x[0].ctx)
    if isinstance(module, scn.JoinTable):
        return OTensor(np.concatenate([t.features for t in x], 1), x[0].spatial_size, x[0].ctx)
    if isinstance(module, scn.Sequential):
        for m in module:
            x = forward(m, x, save)
        return x
    if isinstance(module, scn.Identity):
        return x
    bias = _np(getattr(module, "bias", None))
    if isinstance(module, scn.SubmanifoldConvolution):
        counts, pairs = x.ctx.ssc_rules(x.spatial_size)
        f, _ = orc.conv_forward(x.features, _np(module.weight), bias, pairs, counts, len(x.features))
        return OTensor(f, x.spatial_size, x.ctx)
    if isinstance(module, scn.Convolution):
        coarse = tuple(s // 2 for s in x.spatial_size)
        counts, pairs = x.ctx.down_rules(x.spatial_size, coarse)
        f, _ = orc.conv_forward(x.features, _np(module.weight), bias, pairs, counts, len(x.ctx.coords[coarse]))
        return OTensor(f, coarse, x.ctx)
    if isinstance(module, scn.Deconvolution):
        fine = tuple(s * 2 for s in x.spatial_size)
        counts, pairs = x.ctx.down_rules(fine, x.spatial_size)
        f, _ = orc.conv_forward(x.features, _np(module.weight), bias, pairs, counts, len(x.ctx.coords[fine]), swap=True)
        return OTensor(f, fine, x.ctx)
    if isinstance(module, scn.BatchNormalization):
        f = orc.bn_forward(x.features, _np(module.running_mean), _np(module.running_var),
                           _np(getattr(module, "weight", None)), bias, module.eps, module.leakiness)
        return OTensor(f, x.spatial_size, x.ctx)
    if isinstance(module, scn.NetworkInNetwork):
        return OTensor(orc.nin_forward(x.features, _np(module.weight), bias), x.spatial_size, x.ctx)
    raise NotImplementedError(name)


# ---------------------------------------------------------------------------------------------
# residual frame (the reference's increment=True): every layer evaluated with the oracle's
# restatement of the Incre_* operators against the state saved by `forward(..., save)`
# ---------------------------------------------------------------------------------------------
def _pre_exist(x, pre, size=None):
    size = x.spatial_size if size is None else size
    key = ("pre_exist", size)
    if not hasattr(x.ctx, "cache"):
        x.ctx.cache = {}
    if key not in x.ctx.cache:
        if size not in pre.ctx.coords:
            x.ctx.cache[key] = np.full(len(x.ctx.coords[size]), -1, np.int32)
        else:
            x.ctx.cache[key] = orc.incre_pre_exist(pre.ctx.coords[size], x.ctx.coords[size])
    return x.ctx.cache[key]


def forward_residual(module, x, save):
    import sparseconvnet as scn

    if isinstance(module, scn.InputLayer):
        pre_in, pre_out = save[id(module)]
        coords, feats = x[0], x[1]
        ctx = Ctx()
        size = tuple(int(v) for v in module.spatial_size.tolist())
        sop, sc, cnt = orc.grid_build(np.asarray(coords))
        ctx.coords[size] = sc
        ctx.site_of_point = sop
        ctx.count = cnt
        t = OTensor(None, size, ctx)
        pe = _pre_exist(t, pre_out)
        t.features = orc.incre_input_forward(np.asarray(feats, np.float32), sop, cnt, module.mode, pe,
                                             pre_out.features, pre_out.ctx.count)
        return t
    if isinstance(module, scn.OutputLayer):
        pre_in, _ = save[id(module)]
        return orc.incre_output_forward(x.features, x.ctx.site_of_point, _pre_exist(x, pre_in), pre_in.features)
    if isinstance(module, scn.ConcatTable):
        return [forward_residual(m, x, save) for m in module._modules.values()]
    if isinstance(module, scn.Sequential) and not isinstance(module, (scn.AddTable, scn.JoinTable)):
        for m in module:
            x = forward_residual(m, x, save)
        return x
    bias = _np(getattr(module, "bias", None))
    if isinstance(module, scn.SubmanifoldConvolution):
        pre_in, _ = save[id(module)]
        pe = _pre_exist(x, pre_in)
        rules = x.ctx.ssc_rules(x.spatial_size)
        key = ("ssc_pre", x.spatial_size)
        if key not in x.ctx.cache:
            x.ctx.cache[key] = orc.incre_ssc_rules(x.ctx.coords[x.spatial_size], pre_in.ctx.coords[x.spatial_size], pe)
        f = orc.incre_ssc_forward(x.features, pre_in.features, _np(module.weight), bias, rules, x.ctx.cache[key],
                                  len(x.features))
        return OTensor(f, x.spatial_size, x.ctx)
    if isinstance(module, scn.BatchNormalization):
        pre_in, pre_out = save[id(module)]
        f = orc.incre_bn_forward(x.features, _np(module.running_mean), _np(module.running_var),
                                 _np(getattr(module, "weight", None)), bias, module.eps, module.leakiness,
                                 _pre_exist(x, pre_in), pre_in.features, pre_out.features)
        return OTensor(f, x.spatial_size, x.ctx)
    if isinstance(module, scn.Deconvolution):
        pre_in, pre_out = save[id(module)]
        fine = tuple(s * 2 for s in x.spatial_size)
        x.ctx.down_rules(fine, x.spatial_size)
        parent, off, _ = orc.down2_rules(x.ctx.coords[fine])
        f = orc.incre_deconv_forward(x.features, pre_in.features, _np(module.weight), bias, parent, off,
                                     _pre_exist(x, pre_in), _pre_exist(x, pre_out, fine))
        return OTensor(f, fine, x.ctx)
    # Convolution, NetworkInNetwork, AddTable, JoinTable, Identity: the plain operator on the frame's rows
    return _forward(module, x, None)
