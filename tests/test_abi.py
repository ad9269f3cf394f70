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
