"""The C ABI: every function declared in include/insc.h is exported by libinsc.so and bound by
the Python loader, and nothing here needs a GPU (loading the library touches no device)."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared():
    text = open(os.path.join(ROOT, "include", "insc.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(insc_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from sparseconvnet import _lib

    names = declared()
    assert len(names) >= 45
    lib = _lib.cdll()
    for n in names:
        assert hasattr(lib, n), "libinsc.so does not export %s" % n
    assert sorted(_lib.EXPORTS) == names, set(names) ^ set(_lib.EXPORTS)


def test_no_unexpected_exports():
    out = subprocess.check_output(["nm", "-D", "--defined-only", _so()]).decode()
    exported = sorted(l.split()[-1] for l in out.splitlines() if " T insc_" in l)
    assert exported == declared()


def _so():
    from sparseconvnet import _lib

    return _lib.LIB_PATH


def test_error_reporting_without_gpu():
    from sparseconvnet import _lib

    lib = _lib.cdll()
    assert lib.insc_version().startswith(b"insc")
    # argument validation happens before any device call
    assert lib.insc_scan_exclusive_i32(None, None, -1, None, None) == -1
    assert b"insc_scan_exclusive_i32" in lib.insc_last_error()
    assert lib.insc_conv_packed_floats(27, 32, 32) == 27 * 1024
    assert lib.insc_conv_packed_floats(27, 48, 224) == 27 * 2 * 8 * 1024
    # the thresholds between the kernels of wide 3^3 layers: host state only
    import ctypes

    for name in ("insc_conv_set_persistent_min_units", "insc_conv_set_shared_weights_min_units"):
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = [ctypes.c_int64], ctypes.c_int
        assert fn(0) == -1 and name.encode() in lib.insc_last_error()
        assert fn(512 if "persistent" in name else 896) == 0
    # a plan whose leading dimension does not cover the rows is refused before any launch
    lib.insc_plan_build.restype = ctypes.c_int
    lib.insc_plan_build.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int64] * 2 + [ctypes.c_void_p] * 4
    assert lib.insc_plan_build(None, None, None, 100, 96, None, None, None, None) == -1
    assert b"plan_ld" in lib.insc_last_error()


def test_module_api_surface():
    """Names and constructor signatures the reference's users rely on (sparseconvnet/__init__.py)."""
    import inspect

    import sparseconvnet as scn

    for name in ["InputLayer", "OutputLayer", "SubmanifoldConvolution", "ValidConvolution", "Convolution",
                 "Deconvolution", "BatchNormalization", "BatchNormReLU", "BatchNormLeakyReLU", "NetworkInNetwork",
                 "Sequential", "ConcatTable", "AddTable", "JoinTable", "Identity", "UNet", "SparseConvNetTensor",
                 "Metadata"]:
        assert hasattr(scn, name), name
    assert list(inspect.signature(scn.SubmanifoldConvolution.__init__).parameters)[1:] == [
        "dimension", "nIn", "nOut", "filter_size", "bias", "dilated_rate"]
    assert list(inspect.signature(scn.Convolution.__init__).parameters)[1:] == [
        "dimension", "nIn", "nOut", "filter_size", "filter_stride", "bias"]
    assert list(inspect.signature(scn.InputLayer.__init__).parameters)[1:4] == ["dimension", "spatial_size", "mode"]
    for cls in (scn.Sequential, scn.SubmanifoldConvolution, scn.BatchNormalization, scn.InputLayer, scn.OutputLayer):
        assert list(inspect.signature(cls.forward).parameters)[1:] == ["input", "increment"]
    net = scn.UNet(3, 2, [32, 64, 96], True)
    n_ssc = sum(isinstance(m, scn.SubmanifoldConvolution) for m in net.modules())
    assert n_ssc == 4 * 3 + 4 * 2  # 4 per level on the way down, 4 per non-bottom level on the way up
    w = scn.SubmanifoldConvolution(3, 16, 24, 3, False).weight
    assert tuple(w.shape) == (27, 16, 24)


def test_scn_function_surface():
    """The native-extension functions of the reference that this path covers
    (sparseconvnet/SCN/pybind.cpp:153-258) exist with the reference's argument counts."""
    import inspect

    from sparseconvnet import SCN

    expect = {
        "InputLayer_updateOutput": 7, "OutputLayer_updateOutput": 3, "SubmanifoldConvolution_updateOutput": 8,
        "Convolution_updateOutput": 9, "Deconvolution_updateOutput": 9, "BatchNormalization_updateOutput": 12,
        "NetworkInNetwork_updateOutput": 4, "Incre_InputLayer_updateOutput": 9, "Incre_OutputLayer_updateOutput": 5,
        "Incre_SubmanifoldConvolution_updateOutput": 9, "Incre_Convolution_updateOutput": 9,
        "Incre_Deconvolution_updateOutput": 11, "Incre_BatchNormalization_updateOutput": 17,
        "MaxPooling_updateOutput": 8, "AveragePooling_updateOutput": 8, "UnPooling_updateOutput": 8,
        "SparseToDense_updateOutput": 5,
    }
    for name, n in expect.items():
        params = [p for p in inspect.signature(getattr(SCN, name)).parameters.values()
                  if p.default is inspect.Parameter.empty or p.name == "dilated_rate"]
        assert len(params) == n, (name, [p.name for p in params])
    for name in ("Metadata_3", "Result_3", "ResultOfWeight", "n_rulebook_bits"):
        assert hasattr(SCN, name)


def test_residual_entry_points_validate_before_touching_the_device():
    from sparseconvnet import _lib

    lib = _lib.cdll()
    assert lib.insc_incre_input(None, None, 7, None, None, 0, None, None, 0, 1, 1, None) == -1
    assert b"insc_incre_input" in lib.insc_last_error()
    assert lib.insc_incre_bn_leaky(None, 1, None, 1, None, None, None, None, 0.0, 0.0, None, None, 1, None, 1, -1, 1,
                                   None) == -1
    assert lib.insc_incre_conv_ssc(None, 4, None, 4, 0, None, 4, None, None, None, None, None, 5, 4, 4, None) == -1
    assert b"null pointer" in lib.insc_last_error()
    assert lib.insc_pool_down2(None, 4, None, 3, 4, 2, None, 4, None) == -1
    assert lib.insc_incre_rulebook_ssc3(None, None, None, 0, None, None) == -1
    assert lib.insc_net_forward_residual(None, None, 3, None, 0, None, None, None) == -4
    assert lib.insc_net_enable_residual(None) == -4


def test_incremental_mode_switch():
    import pytest

    import sparseconvnet as scn
    from sparseconvnet import incremental

    assert scn.get_incremental_mode() == "exact"
    assert incremental.kind(False) is None and incremental.kind(True) == "exact"
    assert incremental.kind("residual") == "residual"
    scn.set_incremental_mode("residual")
    try:
        assert incremental.kind(True) == "residual" and incremental.kind(0) is None
        assert incremental.kind("exact") == "exact"
    finally:
        scn.set_incremental_mode("exact")
    with pytest.raises(ValueError):
        scn.set_incremental_mode("fast")
    with pytest.raises(ValueError):
        incremental.kind("yes")
