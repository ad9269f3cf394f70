"""Sequential container that threads the `increment` flag (reference: sparseconvnet/sequential.py:9-25).

A Sequential that is a whole network - it starts with an InputLayer and ends with an OutputLayer,
like `sparseModel` of the reference's example (model.py:15-26) - hands its frames to the native
network executor: the first forward traces the module tree once (compiled.CompiledNet), every
later `model(x, increment)` is one C call instead of one per layer.  The caller's loop stays
what it is with the reference (demo.py:26-38); results are bit-identical to the layer-by-layer
path, which remains in use for every other Sequential, for trees the tracer does not take (a
JoinTable of three inputs, filter sizes other than 3 / 2, a layer type it does not know) and when
switched off with `set_auto_compile(False)`.  The tree is traced at the first full forward;
modules added to an inner container afterwards are not seen (`add` on this Sequential is), and
the per-layer `save_*` attributes of the reference's modules are not filled in on this path.
"""
import torch

from . import incremental

_AUTO = True
_CAPACITY = 1 << 18


def set_auto_compile(flag, capacity_sites=None):
    """Whether whole-network Sequentials run through the network executor (default) or layer by
    layer.  `capacity_sites`: sites at the input scale that an executor traced from now on is sized
    for at the start (default 262 144; it grows by half whenever a frame does not fit, which costs
    that frame a reallocation).  Returns the previous setting of the switch."""
    global _AUTO, _CAPACITY
    prev, _AUTO = _AUTO, bool(flag)
    if capacity_sites is not None:
        _CAPACITY = int(capacity_sites)
    return prev


def get_auto_compile():
    return _AUTO


class Sequential(torch.nn.Sequential):
    def input_spatial_size(self, out_size):
        for m in reversed(self._modules):
            out_size = self._modules[m].input_spatial_size(out_size)
        return out_size

    def add(self, module):
        self._modules[str(len(self._modules))] = module
        self.__dict__.pop("_exec", None)  # the tree changed: trace again
        return self

    def forward(self, input, increment=False):
        net = self._executor(input, increment) if _AUTO else None
        if net is not None:
            return net(input, increment=increment)
        for module in self:
            input = module(input, increment)
        return input

    # ---- the executor behind a whole-network Sequential --------------------------------------
    def _executor(self, input, increment):
        """The CompiledNet that serves this call, or None for the layer-by-layer path."""
        from .ioLayers import InputLayer, OutputLayer

        mods = self._modules
        if len(mods) < 3 or not isinstance(input, (list, tuple)) or len(input) < 2:
            return None
        first, last = mods[next(iter(mods))], mods[next(reversed(mods))]
        if not (isinstance(first, InputLayer) and isinstance(last, OutputLayer)):
            return None
        feats = input[1]
        if not (torch.is_tensor(feats) and feats.is_cuda):
            return None
        kind = incremental.kind(increment)
        state = self.__dict__.get("_exec")
        if state is not None and state[2] != feats.device:
            state = None  # traced (or refused) for another device
        if state is None:
            if kind is not None:
                return None  # no executor holds the scene of the earlier frames: layer by layer
            try:
                from .compiled import CompiledNet

                # residual frames need the raw input of every batch norm kept; asked for when that
                # is the kind of incremental forward in force as the first frame arrives
                net = CompiledNet(self, capacity_sites=max(_CAPACITY, 2 * int(feats.size(0))),
                                  residual=incremental.get_mode() == "residual")
                state = (net, None, feats.device)
            except (NotImplementedError, ValueError) as e:
                state = (None, str(e), feats.device)  # not a tree the tracer takes: layer by layer
            self.__dict__["_exec"] = state
        net = state[0]
        if net is None:
            return None
        if kind == "residual" and not net.residual:
            raise RuntimeError(
                "this network was traced for exact incremental frames; for the reference's residual frames call "
                "sparseconvnet.set_incremental_mode('residual') before the first forward (or use "
                "sparseconvnet.compile(model, residual=True))")
        return net

    def __getstate__(self):
        # the executor is a handle into the native library: a copy (copy.deepcopy, pickle) of the
        # module tree traces its own at its first forward
        d = self.__dict__.copy()
        d.pop("_exec", None)
        return d

    def why_not_compiled(self):
        """None if this Sequential runs through the executor (or has not run yet), else the tracer's reason."""
        state = self.__dict__.get("_exec")
        return None if state is None else state[1]
