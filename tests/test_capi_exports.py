"""The C-ABI library loads without a GPU and exports every symbol include/zant_hip.h declares."""
import ctypes
import os
import re

from conftest import ROOT

LIB = os.path.join(ROOT, "z-ant_amd", "libzant_hip.so")
HEADER = os.path.join(ROOT, "include", "zant_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(zant_hip_\w+|zant_model_\w+|setLogFunctionC|setLogFunction|predict_batched|predict)\s*\(", text)
    return sorted(set(names))


def test_library_is_built():
    assert os.path.exists(LIB), "run `python z-ant_amd/build.py` first"


def test_every_declared_symbol_is_exported():
    lib = ctypes.CDLL(LIB)
    names = declared_symbols()
    assert len(names) >= 30
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_python_binding_covers_the_header():
    import __graft_entry__ as ge
    za = ge.load_package()
    from zant_amd import capi
    assert sorted(capi.PROTOTYPES) == declared_symbols()
    assert za.status_name(-1) == "InvalidDimensions"
    assert za.status_name(-100) == "HipError"


def test_host_only_shape_functions():
    """Shape / check entry points take no device memory and must agree with the oracle's."""
    import __graft_entry__ as ge
    ge.load_package()
    from zant_amd import tensor_math as tm, ZantError
    from oracle import oracle as zo
    import pytest
    cases = [((1, 1, 5, 5), (1, 1, 3, 3), [1], [0, 0, 0, 0], None, None),
             ((1, 1, 5, 5), (1, 1, 3, 3), [1], None, None, "SAME_UPPER"),
             ((2, 3, 9, 7), (4, 3, 3, 2), [2, 1], [1, 0, 2, 1], [1, 1], "NOTSET"),
             ((2, 3, 9, 7), (4, 3, 3, 2), [2, 1], [1, 0, 2, 1], [2, 1], None),
             ((1, 2, 8, 8), (4, 2, 3, 3), [2, 2], None, None, "VALID")]
    for xs, ws, s, p, d, ap in cases:
        assert tm.get_convolution_output_shape(xs, ws, s, p, d, ap) == zo.conv_out_shape(xs, ws, s, p, d, None, ap)
    with pytest.raises(ZantError) as e:
        tm.get_convolution_output_shape((1, 1, 5, 5), (1, 1, 3, 3), [1], None, None, "BOGUS")
    assert e.value.name == "InvalidPadding"
    for k, s, d, p, ap, ceil in [([2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET", False),
                                 ([2, 2], [1, 1], [1, 1], [0, 0, 0, 0], "SAME_UPPER", False),
                                 ([2, 2], [2, 2], [1, 1], [0, 0, 0, 0], "NOTSET", True),
                                 ([3, 3], [2, 2], [2, 1], [1, 1, 1, 1], "NOTSET", False)]:
        assert tm.get_onnx_maxpool_output_shape((1, 1, 9, 9), k, s, d, p, ap, ceil) == \
            zo.maxpool_out_shape((1, 1, 9, 9), k, s, d, p, ap, ceil)
