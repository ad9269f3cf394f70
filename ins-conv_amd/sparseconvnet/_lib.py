"""ctypes binding of libinsc.so (the C ABI declared in include/insc.h).

There is no CPU or PyTorch fallback: if the shared library is missing or a call fails, an
exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libinsc.so")

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_f32 = ctypes.c_float
vp = ctypes.c_void_p

_SIGS = {
    "insc_init": [c_int],
    "insc_grid_create": [c_i64, ctypes.POINTER(vp)],
    "insc_grid_destroy": [vp],
    "insc_grid_clear": [vp, vp],
    "insc_grid_reserve": [vp, c_i64, vp],
    "insc_grid_insert": [vp, vp, c_i64, vp, ctypes.POINTER(c_i64), vp],
    "insc_grid_insert_noalloc": [vp, vp, c_i64, vp, ctypes.POINTER(c_i64), vp],
    "insc_grid_insert_scales": [ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), ctypes.POINTER(vp), c_int,
                                vp, c_int, c_i64, vp, ctypes.POINTER(c_i64), vp],
    "insc_grid_query": [vp, vp, c_i64, vp, vp],
    "insc_grid_size": [vp, ctypes.POINTER(c_i64), vp],
    "insc_rulebook_ssc3": [vp, c_i64, c_i64, vp, c_int, vp],
    "insc_rulebook_pairs": [vp, c_i64, c_int, vp, vp, c_i64, ctypes.POINTER(c_i64), vp],
    "insc_rulebook_down2": [vp, vp, c_i64, c_i64, vp, vp, vp, c_i64, vp],
    "insc_order_build": [vp, vp, c_i64, c_i64, vp, vp],
    "insc_order_by_offset": [vp, vp, c_i64, vp, vp],
    "insc_order_build_scales": [vp, vp, vp, vp, c_int, vp, vp, vp, vp, vp],
    "insc_order_append": [vp, vp, vp, vp, vp, vp, vp, c_i64, vp],
    "insc_conv_nbr": [vp, c_i64, c_i64, vp, c_i64, vp, vp, vp, vp, c_int, vp, vp, c_i64, c_int, c_int,
                      ctypes.POINTER(ctypes.c_double), vp],
    "insc_conv_pack_weights": [vp, c_int, c_int, c_int, vp, vp],
    "insc_plan_build": [vp, vp, vp, c_i64, c_i64, vp, vp, vp, vp],
    "insc_conv_ssc_plan": [vp, c_i64, c_i64, vp, c_i64, vp, vp, vp, vp, vp, c_i64, vp, vp, vp, vp, c_i64, c_int, c_int,
                           vp],
    "insc_conv_set_persistent_min_units": [c_i64],
    "insc_conv_set_shared_weights_min_units": [c_i64],
    "insc_conv_set_filter_lds_min_tiles": [c_i64],
    "insc_conv_set_wavefront_per_unit_min_units": [c_i64],
    "insc_deconv_down2": [vp, c_i64, c_i64, vp, c_i64, vp, vp, vp, vp, vp, vp, vp, c_i64, c_int, c_int, vp],
    "insc_bn_leaky": [vp, c_i64, vp, c_i64, vp, vp, vp, vp, c_f32, c_f32, vp, vp, c_i64, c_int, vp],
    "insc_add": [vp, c_i64, vp, c_i64, vp, c_i64, vp, vp, c_i64, c_int, vp],
    "insc_copy_rows": [vp, c_i64, vp, c_i64, vp, vp, c_i64, c_int, vp],
    "insc_input_accumulate": [vp, c_i64, c_int, vp, c_int, vp, vp, c_i64, vp],
    "insc_input_finish": [vp, vp, c_int, vp, c_i64, vp, vp, c_i64, c_int, vp],
    "insc_output_gather": [vp, c_i64, vp, c_i64, c_int, vp, vp],
    "insc_pool_down2": [vp, c_i64, vp, c_i64, c_int, c_int, vp, c_i64, vp],
    "insc_sparse_to_dense": [vp, vp, c_i64, c_i64, c_int, c_i64, c_i64, c_i64, c_int, vp, vp],
    "insc_fill_u8": [vp, c_i64, c_int, vp],
    "insc_fill_i32": [vp, c_i64, ctypes.c_int32, vp],
    "insc_dirty_mark": [vp, c_i64, vp, vp],
    "insc_dirty_dilate3": [vp, vp, vp, vp, c_i64, vp],
    "insc_dirty_parents": [vp, vp, vp, vp, c_i64, vp],
    "insc_dirty_children": [vp, vp, vp, vp, c_i64, vp],
    "insc_dirty_or": [vp, vp, vp, vp, c_i64, vp],
    "insc_dirty_compact": [vp, vp, vp, c_i64, vp, vp, ctypes.POINTER(c_i64), vp],
    "insc_net_create": [c_int, c_int, c_int, ctypes.POINTER(vp)],
    "insc_net_destroy": [vp],
    "insc_net_tensor": [vp, c_int, c_int, ctypes.POINTER(c_int)],
    "insc_net_join": [vp, c_int, c_int, c_int],
    "insc_net_op_conv": [vp, c_int, c_int, c_int, vp, vp],
    "insc_net_op_bn": [vp, c_int, c_int, vp, vp, vp, vp, c_f32, c_f32],
    "insc_net_op_add": [vp, c_int, c_int, c_int],
    "insc_net_finalize": [vp, c_int, c_i64, vp],
    "insc_net_refresh_weights": [vp, vp],
    "insc_net_rebind_op": [vp, c_int, vp, vp, vp, vp, vp, vp],
    "insc_net_forward": [vp, vp, c_int, vp, c_i64, c_int, vp, c_int, ctypes.POINTER(c_i64), vp],
    "insc_net_enable_residual": [vp],
    "insc_net_set_order_refresh": [vp, ctypes.c_int],
    "insc_net_forward_residual": [vp, vp, c_int, vp, c_i64, vp, ctypes.POINTER(c_i64), vp],
    "insc_net_tensor_view": [vp, c_int, ctypes.POINTER(vp), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64),
                             ctypes.POINTER(c_int)],
    "insc_net_counts": [vp, ctypes.POINTER(c_i64), ctypes.POINTER(c_i64)],
    "insc_net_dirty_counts": [vp, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int), ctypes.POINTER(c_int),
                              ctypes.POINTER(c_i64), vp],
    "insc_net_profile": [vp, c_int, ctypes.POINTER(ctypes.c_float)],
    "insc_net_frame_work": [vp, c_int, ctypes.POINTER(c_int), ctypes.POINTER(c_int), ctypes.POINTER(c_int),
                            ctypes.POINTER(c_int), ctypes.POINTER(c_int), ctypes.POINTER(c_i64), ctypes.POINTER(c_i64),
                            ctypes.POINTER(c_i64), vp],
    "insc_labels_create": [c_i64, c_int, c_f32, ctypes.POINTER(vp)],
    "insc_labels_destroy": [vp],
    "insc_labels_clear": [vp, vp],
    "insc_labels_set": [vp, vp, vp, c_i64, c_i64, c_int, vp],
    "insc_labels_update": [vp, vp, vp, c_i64, c_i64, c_int, vp],
    "insc_labels_query": [vp, vp, c_i64, vp, vp],
    "insc_labels_count": [vp, ctypes.POINTER(c_i64), vp],
    "insc_labels_export": [vp, vp, vp, c_i64, vp],
    "insc_labels_finalize": [vp, vp, c_i64, vp],
    "insc_incre_rulebook_ssc3": [vp, vp, vp, c_i64, vp, vp],
    "insc_incre_input": [vp, vp, c_int, vp, vp, c_i64, vp, vp, c_i64, c_i64, c_int, vp],
    "insc_incre_conv_ssc": [vp, c_i64, vp, c_i64, c_i64, vp, c_i64, vp, vp, vp, vp, vp, c_i64, c_int, c_int, vp],
    "insc_incre_bn_leaky": [vp, c_i64, vp, c_i64, vp, vp, vp, vp, c_f32, c_f32, vp, vp, c_i64, vp, c_i64, c_i64,
                            c_int, vp],
    "insc_incre_deconv_down2": [vp, c_i64, c_i64, vp, c_i64, c_i64, vp, c_i64, vp, vp, vp, vp, vp, vp, vp, c_i64,
                                c_int, c_int, vp],
    "insc_incre_output": [vp, c_i64, vp, c_i64, vp, vp, c_i64, c_int, vp, vp],
    "insc_scan_exclusive_i32": [vp, vp, c_i64, vp, vp],
    "insc_sort_pairs_u64": [vp, vp, c_i64, c_int, vp],
}
# functions that return something other than a status code
_OTHER = {
    "insc_last_error": (ctypes.c_char_p, []),
    "insc_version": (ctypes.c_char_p, []),
    "insc_grid_coords": (vp, [vp]),
    "insc_grid_count_ptr": (vp, [vp]),
    "insc_grid_capacity": (c_i64, [vp]),
    "insc_conv_packed_floats": (c_i64, [c_int, c_int, c_int]),
    "insc_net_op_count": (c_int, [vp]),
}

EXPORTS = sorted(list(_SIGS) + list(_OTHER))


class InscError(RuntimeError):
    def __init__(self, code, msg):
        RuntimeError.__init__(self, "libinsc error %d: %s" % (code, msg))
        self.code = code


_cdll = None


def cdll():
    """The raw ctypes handle (no GPU is touched by loading it)."""
    global _cdll
    if _cdll is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "libinsc.so not found at %s - build it with `make -C ins-conv_amd/csrc` "
                "(there is no fallback implementation)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, args in _SIGS.items():
            f = getattr(L, name)
            f.argtypes = args
            f.restype = c_int
        for name, (res, args) in _OTHER.items():
            f = getattr(L, name)
            f.argtypes = args
            f.restype = res
        _cdll = L
    return _cdll


class _Checked(object):
    """Attribute access returns a wrapper that raises InscError on a non-zero status."""

    def __getattr__(self, name):
        L = cdll()
        f = getattr(L, name)
        if name in _OTHER:
            return f

        def call(*a):
            rc = f(*a)
            if rc != 0:
                raise InscError(rc, L.insc_last_error().decode())
            return rc

        call.__name__ = name
        setattr(self, name, call)
        return call


lib = _Checked()
_inited = set()


def ensure_init(device_index):
    if device_index not in _inited:
        lib.insc_init(int(device_index))
        _inited.add(device_index)


def ptr(t):
    """Device (or host) address of a torch tensor, None -> NULL."""
    if t is None:
        return None
    return t.data_ptr() if t.numel() else None


def stream_ptr():
    import torch

    return torch.cuda.current_stream().cuda_stream
