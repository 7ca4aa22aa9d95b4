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


def _split_params(s):
    """Top-level comma split of a parameter list (function-pointer parameters carry their own parentheses)."""
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([":
            depth += 1
        elif ch in ")]":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip() and cur.strip() != "void":
        out.append(cur.strip())
    return out


def _header_prototypes():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    protos = {}
    for m in re.finditer(r"\b(zant_hip_\w+|zant_model_\w+|setLogFunctionC|setLogFunction|predict_batched|predict)\s*\(((?:[^()]|\([^()]*\))*)\)\s*;", text):
        protos[m.group(1)] = _split_params(m.group(2))
    return protos


def test_zig_binding_mirrors_the_header():
    """bindings/zant_hip.zig (no Zig compiler here: a text check): one `extern fn` per function of the header with
    the same number of parameters in the same order of names, and the reference's lean signatures verbatim."""
    zig = open(os.path.join(ROOT, "bindings", "zant_hip.zig")).read()
    externs = {m.group(1): _split_params(m.group(2))
               for m in re.finditer(r"pub extern fn (\w+)\(((?:[^()]|\([^()]*\))*)\)", zig)}
    protos = _header_prototypes()
    assert sorted(protos) == declared_symbols()
    assert sorted(externs) == sorted(protos)
    rename = {"var": "variance"}  # `var` is a Zig keyword
    for name, params in protos.items():
        assert len(externs[name]) == len(params), name
        for c_param, z_param in zip(params, externs[name]):
            if "(*" in c_param:   # a function pointer: void (*func)(char *)
                c_name = re.search(r"\(\*(\w+)\)", c_param).group(1)
            else:
                c_name = re.search(r"(\w+)(\[\d*\])?$", c_param).group(1)
            assert z_param.split(":")[0].strip() == rename.get(c_name, c_name), (name, c_param, z_param)
    lean = [  # tensor_math_standard.zig name, then the parameter list as the reference writes it
        "pub fn conv_lean(comptime T: type, input: *Tensor(T), kernel: *Tensor(T), output: *Tensor(T), bias: ?*const Tensor(T), stride: []const usize, pads: ?[]const usize, dilations: ?[]const usize, group: ?usize, auto_pad: ?[]const u8) !void",
        "pub fn gemm_lean(comptime T: anytype, A: *Tensor(T), B: *Tensor(T), C: ?*Tensor(T), alpha: T, beta: T, transA: bool, transB: bool, result: *Tensor(T)) !void",
        "pub fn mat_mul_lean(comptime T: anytype, A: *const Tensor(T), B: *const Tensor(T), Y: *Tensor(T)) !void",
        "pub fn onnx_maxpool_lean(comptime T: type, input: *Tensor(T), output: *Tensor(T), kernel_shape: []const usize, strides: []const usize, dilations: []const usize, pads: []const usize, auto_pad: AutoPadType) !void",
        "pub fn ReLU_lean(comptime T: anytype, input_tensor: *Tensor(T), output_tensor: *Tensor(T)) !void",
        "pub fn leakyReLU_lean(comptime T: anytype, input_tensor: *Tensor(T), slope: T, output_tensor: *Tensor(T)) !void",
        "pub fn softmax_lean(comptime T: anytype, input: *Tensor(T), output: *Tensor(T)) !void",
        "pub fn sum_tensors_lean(comptime inputType: anytype, comptime outputType: anytype, t1: *Tensor(inputType), t2: *Tensor(inputType), outputTensor: *Tensor(outputType)) !void",
        "pub fn reshape_lean(comptime T: anytype, input: *Tensor(T), newShape: []const usize, allowZero: ?bool, output: *Tensor(T)) !void",
        "pub fn sigmoid_lean(comptime T: anytype, input_tensor: *Tensor(T), output_tensor: *Tensor(T)) !void",
        "pub fn reduce_mean_lean(comptime T: anytype, input_tensor: *Tensor(T), output_tensor: *Tensor(T), axes: ?[]const i64, _: bool, noop_with_empty_axes: bool) !void",
        "pub fn lean_concatenate(comptime T: type, allocator: *const std.mem.Allocator, tensors: []const Tensor(T), axis: isize, output: *Tensor(T)) !void",
        # the quantised family (not in the reference): house style -- comptime element types, pre-shaped output, !void --
        # and the ONNX input order
        "pub fn quantize_linear_lean(comptime T_in: type, comptime T_out: type, x: *Tensor(T_in), y_scale: *Tensor(T_in), y_zero_point: ?*Tensor(T_out), axis: i64, y: *Tensor(T_out)) !void",
        "pub fn dequantize_linear_lean(comptime T_in: type, comptime T_out: type, x: *Tensor(T_in), x_scale: *Tensor(T_out), x_zero_point: ?*Tensor(T_in), axis: i64, y: *Tensor(T_out)) !void",
        "pub fn qlinearconv_lean(x: *Tensor(u8), x_scale: f32, x_zero_point: u8, w: *Tensor(i8), w_scale: *Tensor(f32), w_zero_point: ?*Tensor(i8), y_scale: f32, y_zero_point: u8, bias: ?*const Tensor(i32), y: *Tensor(u8), stride: []const usize, pads: ?[]const usize, dilations: ?[]const usize, group: ?usize) !void",
    ]
    # the façade calls the u8 pooling entry and every quantised entry it wraps
    for used in ("zant_hip_maxpool2d_u8(ctx", "zant_hip_quantize_linear_f32_u8(ctx", "zant_hip_quantize_linear_f32_i8(ctx",
                 "zant_hip_dequantize_linear_u8_f32(ctx", "zant_hip_dequantize_linear_i8_f32(ctx",
                 "zant_hip_dequantize_linear_i32_f32(ctx", "zant_hip_qlinearconv_u8i8(ctx", "zant_hip_qlinearconv_prepack(ctx",
                 "zant_hip_qlinearconv_u8i8_packed(ctx", "zant_hip_conv2d_f32_prepack(ctx", "zant_hip_conv2d_f32_packed(ctx"):
        assert used in zig, used
    for sig in lean:
        assert sig in zig, sig
    # every status the header names maps to an error (or to the catch-all for HIP / memory failures)
    header = open(HEADER).read()
    for code in re.findall(r"ZANT_\w+ = (-\d+),", header):
        if int(code) > -100 and int(code) != -13:
            assert f"        {code} => " in zig, code
