"""A minimal ONNX reader for the operator set of the hot path: decodes the protobuf wire format directly (no onnx
package), folds Reshape on initialisers, and builds a ``Model`` (the executor behind the generated ``predict()``).

The reference parses ONNX in Zig (src/onnx/protobuf.zig:31-203, src/onnx/onnx.zig) and turns each node into one
``tensMath.*_lean`` call (src/codeGen/math_handler.zig:31-108); this does the same for Conv, Add, Relu, LeakyRelu,
MaxPool, AveragePool, BatchNormalization, Reshape, MatMul, Gemm and Softmax, which covers the bundled mnist-8 network, and for quantised graphs in
operator form: QuantizeLinear, DequantizeLinear, QLinearConv, MaxPool on u8, QLinearAdd and
QLinearGlobalAveragePool (com.microsoft), and the activation idiom DequantizeLinear -> Relu | LeakyRelu | Clip(0, 6)
-> QuantizeLinear, which becomes one quantised activation node (the executor then folds it into the convolution).
"""
import struct

import numpy as np

# ------------------------------------------------------------------------------------------------ protobuf wire format


def _varint(buf, pos):
    result = shift = 0
    while True:
        b = buf[pos]
        pos += 1
        result |= (b & 0x7F) << shift
        if not b & 0x80:
            return result, pos
        shift += 7


def _fields(buf):
    """Yields (field number, wire type, value) of one message; length-delimited values are memoryviews."""
    pos, end = 0, len(buf)
    while pos < end:
        key, pos = _varint(buf, pos)
        num, wt = key >> 3, key & 7
        if wt == 0:
            val, pos = _varint(buf, pos)
        elif wt == 1:
            val, pos = bytes(buf[pos:pos + 8]), pos + 8
        elif wt == 2:
            n, pos = _varint(buf, pos)
            val, pos = buf[pos:pos + n], pos + n
        elif wt == 5:
            val, pos = bytes(buf[pos:pos + 4]), pos + 4
        else:
            raise ValueError(f"unsupported protobuf wire type {wt}")
        yield num, wt, val


def _signed(v):
    return v - (1 << 64) if v >= 1 << 63 else v


def _packed_ints(wt, val):
    if wt == 0:
        return [_signed(val)]
    out, pos = [], 0
    while pos < len(val):
        v, pos = _varint(val, pos)
        out.append(_signed(v))
    return out


_DTYPES = {1: np.float32, 2: np.uint8, 3: np.int8, 6: np.int32, 7: np.int64, 11: np.float64}


def _tensor(buf):
    dims, dtype, name, raw, floats, ints = [], 1, "", None, [], []
    for num, wt, val in _fields(buf):
        if num == 1:
            dims += _packed_ints(wt, val)
        elif num == 2:
            dtype = val
        elif num == 8:
            name = bytes(val).decode()
        elif num == 9:
            raw = bytes(val)
        elif num == 4:
            floats += [struct.unpack("<f", val)[0]] if wt == 5 else list(np.frombuffer(bytes(val), "<f4"))
        elif num in (5, 7):
            ints += _packed_ints(wt, val)
    np_dtype = _DTYPES[dtype]
    if raw is not None:
        arr = np.frombuffer(raw, dtype=np.dtype(np_dtype).newbyteorder("<")).astype(np_dtype)
    elif floats:
        arr = np.array(floats, np_dtype)
    else:
        arr = np.array(ints, np_dtype)
    return name, arr.reshape(dims)


def _attribute(buf):
    name, out, ints, floats = "", None, [], []
    for num, wt, val in _fields(buf):
        if num == 1:
            name = bytes(val).decode()
        elif num == 2:
            out = struct.unpack("<f", val)[0]
        elif num == 3:
            out = _signed(val)
        elif num == 4:
            out = bytes(val).decode()
        elif num == 5:
            out = _tensor(val)[1]
        elif num == 7:
            floats += [struct.unpack("<f", val)[0]] if wt == 5 else list(np.frombuffer(bytes(val), "<f4"))
        elif num == 8:
            ints += _packed_ints(wt, val)
    if ints:
        out = ints
    elif floats:
        out = floats
    return name, out


def _node(buf):
    node = {"inputs": [], "outputs": [], "op": "", "attrs": {}}
    for num, _, val in _fields(buf):
        if num == 1:
            node["inputs"].append(bytes(val).decode())
        elif num == 2:
            node["outputs"].append(bytes(val).decode())
        elif num == 4:
            node["op"] = bytes(val).decode()
        elif num == 5:
            k, v = _attribute(val)
            node["attrs"][k] = v
    return node


def _value_info(buf):
    name, dims, elem = "", [], 1
    for num, _, val in _fields(buf):
        if num == 1:
            name = bytes(val).decode()
        elif num == 2:  # TypeProto
            for n2, _, v2 in _fields(val):
                if n2 == 1:  # tensor_type
                    for n3, _, v3 in _fields(v2):
                        if n3 == 1:
                            elem = int(v3)
                        elif n3 == 2:  # shape
                            for n4, _, v4 in _fields(v3):
                                if n4 == 1:  # dim
                                    d = 1
                                    for n5, _, v5 in _fields(v4):
                                        if n5 == 1:
                                            d = v5
                                    dims.append(int(d))
    return name, dims, elem


def read_graph(path):
    """-> {"nodes": [...], "initializers": {name: ndarray}, "inputs": [(name, dims)], "outputs": [(name, dims)],
    "elem_types": {name: ONNX element type of a graph input / output}}"""
    buf = memoryview(open(path, "rb").read())
    graph = None
    for num, _, val in _fields(buf):
        if num == 7:
            graph = val
    if graph is None:
        raise ValueError("no graph in the ONNX file")
    g = {"nodes": [], "initializers": {}, "inputs": [], "outputs": [], "elem_types": {}}
    for num, _, val in _fields(graph):
        if num == 1:
            g["nodes"].append(_node(val))
        elif num == 5:
            name, arr = _tensor(val)
            g["initializers"][name] = arr
        elif num in (11, 12):
            name, dims, elem = _value_info(val)
            g["inputs" if num == 11 else "outputs"].append((name, dims))
            g["elem_types"][name] = elem
    g["inputs"] = [(n, d) for n, d in g["inputs"] if n not in g["initializers"]]
    return g


# ------------------------------------------------------------------------------------------------ graph -> executor

def _pool_or_conv_attrs(a, rank2_default):
    strides = a.get("strides", rank2_default)
    pads = a.get("pads")
    dil = a.get("dilations", [1, 1])
    auto_pad = a.get("auto_pad", "NOTSET")
    return strides, pads, dil, auto_pad


def _lift4(arr):
    """An ONNX Gemm operand in the reference's rank-4 form: leading ones."""
    return arr.reshape((1,) * (4 - arr.ndim) + arr.shape)


def run_graph(graph, ops, x):
    """Executes the graph with ``ops`` (an object with the reference-named operators: the CPU oracle module, or any
    other implementation with the same signatures) on the numpy input ``x``.  Used by tests as the checker's driver."""
    vals = dict(graph["initializers"])
    vals[graph["inputs"][0][0]] = x
    for nd in graph["nodes"]:
        i = [vals[n] for n in nd["inputs"] if n]
        a = nd["attrs"]
        if nd["op"] == "Conv":
            s, p, d, ap = _pool_or_conv_attrs(a, [1, 1])
            y = ops.Conv(i[0], i[1], i[2] if len(i) > 2 else None, s, p if p is not None else ([0, 0, 0, 0] if ap == "NOTSET" else None), d,
                         a.get("group", 1), ap)
        elif nd["op"] == "Add":
            y = ops.sum_tensors_lean(i[0], i[1])
        elif nd["op"] == "Relu":
            y = ops.ReLU(i[0])
        elif nd["op"] == "MaxPool":
            s, p, d, ap = _pool_or_conv_attrs(a, [1, 1])
            y = ops.onnx_maxpool(i[0], a["kernel_shape"], s, d, p if p is not None else [0, 0, 0, 0], ap)
        elif nd["op"] == "AveragePool":
            s, p, _, ap = _pool_or_conv_attrs(a, [1, 1])
            y = ops.avgpool(i[0], a["kernel_shape"], s, p if p is not None else [0, 0, 0, 0], bool(a.get("ceil_mode", 0)),
                            bool(a.get("count_include_pad", 0)))
        elif nd["op"] == "BatchNormalization":
            y = ops.batchnorm(i[0], i[1], i[2], i[3], i[4], a.get("epsilon", 1e-5))
        elif nd["op"] == "Reshape":
            y = ops.reshape_lean(i[0], [int(v) for v in i[1]])
        elif nd["op"] == "MatMul":
            y = ops.mat_mul(i[0], i[1])
        elif nd["op"] == "Gemm":
            # the reference's gemm takes {1, 1, rows, cols} tensors (op_gemm.zig:22-27): ONNX's 2-D operands are lifted
            a4, b4 = _lift4(i[0]), _lift4(i[1])
            c4 = _lift4(i[2]) if len(i) > 2 else None
            y = ops.gemm(a4, b4, c4, a.get("alpha", 1.0), a.get("beta", 1.0), bool(a.get("transA", 0)), bool(a.get("transB", 0)))
            if i[0].ndim == 2:
                y = y.reshape(y.shape[2], y.shape[3])
        elif nd["op"] == "Softmax":
            y = ops.softmax(i[0])
        elif nd["op"] == "Sigmoid":
            y = ops.sigmoid(i[0])
        elif nd["op"] == "LeakyRelu":
            y = ops.leakyReLU(i[0], a.get("alpha", 0.01))
        elif nd["op"] == "GlobalAveragePool":
            y = ops.reduce_mean(i[0], [2, 3], True, False)
        elif nd["op"] == "ReduceMean":
            axes = a.get("axes")
            if axes is None and len(i) > 1:
                axes = [int(v) for v in i[1].reshape(-1)]
            y = ops.reduce_mean(i[0], axes, bool(a.get("keepdims", 1)), False)
        elif nd["op"] == "Concat":
            y = ops.concatenate(i, a["axis"])
        elif nd["op"] == "Resize":
            names = nd["inputs"] + ["", "", ""]
            scales = vals[names[2]].reshape(-1) if names[2] and vals[names[2]].size else None
            sizes = vals[names[3]].reshape(-1) if names[3] and vals[names[3]].size else None
            coord = a.get("coordinate_transformation_mode", "half_pixel")
            coord = coord.decode() if isinstance(coord, bytes) else coord
            y = ops.resize(i[0], "nearest", None if scales is None else [float(v) for v in scales],
                           None if sizes is None else [int(v) for v in sizes], coord)
        else:
            raise NotImplementedError(nd["op"])
        vals[nd["outputs"][0]] = y
    return vals[graph["outputs"][0][0]]


def _resize_has_ties(in_dims, out_dims, coord):
    """Whether any output coordinate of a nearest-neighbour Resize lands exactly between two input elements, computed in
    f32 like the reference (lib_shape_math.zig:128-139): only then does the rounding convention matter."""
    for n_in, n_out in zip(in_dims, out_dims):
        o = np.arange(n_out, dtype=np.float32)
        scale = np.float32(n_out) / np.float32(n_in)
        if coord == "half_pixel":
            pos = (o + np.float32(0.5)) / scale - np.float32(0.5)
        elif coord == "align_corners":
            pos = o * np.float32(n_in - 1) / np.float32(max(n_out - 1, 1))
        else:
            pos = o / scale
        pos = pos[(pos > 0) & (pos < n_in - 1)]  # outside that range the clamp decides
        if np.any(pos - np.floor(pos) == np.float32(0.5)):
            return True
    return False


def build_model(ctx, graph, model=None):
    """Turns the graph into a finalized ``Model``: one executor node per ONNX node, initialisers as parameters, Reshape
    of an initialiser folded on the host (as the reference's code generator does for constant inputs).  ``model``: an
    object with Model's builder methods to drive instead of a new Model (the code generator passes its recorder)."""
    from .model import Model, U8
    m = model if model is not None else Model(ctx)
    consts = dict(graph["initializers"])
    name, dims = graph["inputs"][0]
    nodes = graph["nodes"]
    readers = {}  # tensor name -> indices of the nodes that read it
    for k, nd in enumerate(nodes):
        for n in nd["inputs"]:
            readers.setdefault(n, []).append(k)
    qparams = {}  # name of a u8 tensor -> (scale, zero point)
    if graph["elem_types"].get(name, 1) == 2:
        # a u8 graph input carries no quantisation parameters of its own: they are those its first reader names
        first = nodes[readers[name][0]]
        if first["op"] not in ("QLinearConv", "DequantizeLinear", "QLinearAdd", "QLinearGlobalAveragePool"):
            raise NotImplementedError("a uint8 graph input must feed a quantised operator")
        sc = float(consts[first["inputs"][1]].reshape(-1)[0])
        zp = int(consts[first["inputs"][2]].reshape(-1)[0]) if len(first["inputs"]) > 2 and first["inputs"][2] else 0
        tens = {name: m.input(tuple(dims), U8, sc, zp)}
        qparams[name] = (sc, zp)
    else:
        tens = {name: m.input(tuple(dims))}

    def reshape_const(arr, shape):
        shape = [arr.shape[k] if v == 0 else int(v) for k, v in enumerate(shape)]
        return arr.reshape(shape)

    def scalar(n, default=0):
        return default if not n else consts[n].reshape(-1)[0]

    def check_q(n, scale_name, zp_name):
        sc, zp = qparams[n]
        if np.float32(scalar(scale_name)) != np.float32(sc) or int(scalar(zp_name)) != zp:
            raise ValueError(f"{n}: quantisation parameters differ from those of its producer")

    skip = set()
    for k, nd in enumerate(nodes):
        if k in skip:
            continue
        ins, a, out = nd["inputs"], nd["attrs"], nd["outputs"][0]
        op = nd["op"]
        if op == "Reshape" and ins[0] in consts:
            consts[out] = reshape_const(consts[ins[0]], consts[ins[1]])
            continue
        if op == "Conv":
            s, p, d, ap = _pool_or_conv_attrs(a, [1, 1])
            bias = consts[ins[2]] if len(ins) > 2 and ins[2] else None
            if p is None and ap == "NOTSET":
                p = [0, 0, 0, 0]
            t = m.conv(tens[ins[0]], consts[ins[1]].astype(np.float32), bias, s, p, d, a.get("group", 1), ap)
        elif op == "Add":
            if ins[1] in consts:
                t = m.add_const(tens[ins[0]], consts[ins[1]].astype(np.float32))
            elif ins[0] in consts:
                t = m.add_const(tens[ins[1]], consts[ins[0]].astype(np.float32))
            else:
                t = m.add(tens[ins[0]], tens[ins[1]])
        elif op == "Relu":
            t = m.relu(tens[ins[0]])
        elif op == "LeakyRelu":
            t = m.leaky_relu(tens[ins[0]], a.get("alpha", 0.01))
        elif op == "MaxPool":
            s, p, d, ap = _pool_or_conv_attrs(a, [1, 1])
            t = m.maxpool(tens[ins[0]], a["kernel_shape"], s, d, p if p is not None else [0, 0, 0, 0], ap,
                          bool(a.get("ceil_mode", 0)))
            if ins[0] in qparams:
                qparams[out] = qparams[ins[0]]
        elif op == "AveragePool":
            s, p, d, ap = _pool_or_conv_attrs(a, [1, 1])
            if ap != "NOTSET" or any(v != 1 for v in d):
                raise NotImplementedError("AveragePool with auto_pad or dilations")
            t = m.avgpool(tens[ins[0]], a["kernel_shape"], s, p, bool(a.get("ceil_mode", 0)), bool(a.get("count_include_pad", 0)))
        elif op == "BatchNormalization":
            if a.get("training_mode", 0) or len(nd["outputs"]) > 1:
                raise NotImplementedError("BatchNormalization in training mode")
            t = m.batchnorm(tens[ins[0]], consts[ins[1]], consts[ins[2]], consts[ins[3]], consts[ins[4]], a.get("epsilon", 1e-5))
        elif op == "Reshape":
            t = m.reshape(tens[ins[0]], [int(v) for v in consts[ins[1]]])
        elif op == "MatMul":
            t = m.matmul(tens[ins[0]], consts[ins[1]].astype(np.float32))
        elif op == "Gemm":
            # gemm_lean works on {1, 1, rows, cols} tensors (op_gemm.zig:22-27, 52-60): a 2-D A is viewed as such, B and
            # C get leading ones, and the result is viewed back as ONNX's (M, N)
            c = consts[ins[2]].astype(np.float32) if len(ins) > 2 and ins[2] else None
            a_id, a_shape = tens[ins[0]], m.tensor_shape(tens[ins[0]])
            if len(a_shape) > 4 or len(a_shape) < 2:
                raise NotImplementedError(f"Gemm with a rank-{len(a_shape)} input")
            if len(a_shape) < 4:
                a_id = m.reshape(a_id, [1] * (4 - len(a_shape)) + list(a_shape))
            t = m.gemm(a_id, consts[ins[1]].astype(np.float32), c, a.get("alpha", 1.0), a.get("beta", 1.0),
                       bool(a.get("transA", 0)), bool(a.get("transB", 0)))
            if len(a_shape) < 4:
                t = m.reshape(t, list(m.tensor_shape(t))[4 - len(a_shape):])
        elif op == "Softmax":
            t = m.softmax(tens[ins[0]])
        elif op == "Sigmoid":
            t = m.sigmoid(tens[ins[0]])
        elif op == "GlobalAveragePool":
            t = m.global_average_pool(tens[ins[0]])
        elif op == "ReduceMean":
            if a.get("noop_with_empty_axes", 0):
                raise NotImplementedError("ReduceMean with noop_with_empty_axes")
            axes = a.get("axes")
            if axes is None and len(ins) > 1 and ins[1]:
                axes = [int(v) for v in consts[ins[1]].reshape(-1)]
            t = m.reduce_mean(tens[ins[0]], axes, bool(a.get("keepdims", 1)))
        elif op == "Concat":
            t = m.concat([tens[n] for n in ins], a["axis"])
            if ins[0] in qparams:
                qparams[out] = qparams[ins[0]]
        elif op == "Resize":
            mode = a.get("mode", b"nearest")
            mode = mode.decode() if isinstance(mode, bytes) else mode
            if mode != "nearest":
                raise NotImplementedError(f"Resize mode {mode}")
            coord = a.get("coordinate_transformation_mode", b"half_pixel")
            coord = coord.decode() if isinstance(coord, bytes) else coord
            if coord not in ("half_pixel", "align_corners", "asymmetric"):
                raise NotImplementedError(f"Resize coordinate_transformation_mode {coord}")
            scales = consts[ins[2]].reshape(-1) if len(ins) > 2 and ins[2] and consts[ins[2]].size else None
            sizes = consts[ins[3]].reshape(-1) if len(ins) > 3 and ins[3] and consts[ins[3]].size else None
            nearest = a.get("nearest_mode", b"round_prefer_floor")
            nearest = nearest.decode() if isinstance(nearest, bytes) else nearest
            in_dims = m.tensor_shape(tens[ins[0]])
            out_dims = [int(np.floor(np.float32(d) * np.float32(f))) for d, f in zip(in_dims, scales)] if scales is not None \
                else [int(v) for v in sizes]
            if nearest != "round_prefer_ceil" and _resize_has_ties(in_dims, out_dims, coord):
                # the reference rounds half away from zero (lib_shape_math.zig:141), which is round_prefer_ceil here
                raise NotImplementedError(f"Resize nearest_mode {nearest} differs from the reference's rounding on this shape")
            t = m.resize_nearest(tens[ins[0]], None if scales is None else [float(v) for v in scales],
                                 None if sizes is None else out_dims, coord)
            if ins[0] in qparams:
                qparams[out] = qparams[ins[0]]
        elif op == "QuantizeLinear":
            sc, zp = float(scalar(ins[1])), int(scalar(ins[2] if len(ins) > 2 else ""))
            t = m.quantize(tens[ins[0]], sc, zp)
            qparams[out] = (sc, zp)
        elif op == "DequantizeLinear":
            check_q(ins[0], ins[1], ins[2] if len(ins) > 2 else "")
            # DequantizeLinear -> activation -> QuantizeLinear with single readers in between: one quantised activation
            fused = False
            r1 = readers.get(out, [])
            if len(r1) == 1 and nodes[r1[0]]["op"] in ("Relu", "LeakyRelu", "Clip"):
                an = nodes[r1[0]]
                r2 = readers.get(an["outputs"][0], [])
                if len(r2) == 1 and nodes[r2[0]]["op"] == "QuantizeLinear":
                    qn = nodes[r2[0]]
                    act, alpha = None, 0.0
                    if an["op"] == "Relu":
                        act = "relu"
                    elif an["op"] == "LeakyRelu":
                        act, alpha = "leaky", float(an["attrs"].get("alpha", 0.01))
                    else:
                        lo = float(scalar(an["inputs"][1])) if len(an["inputs"]) > 1 else float(an["attrs"].get("min", -np.inf))
                        hi = float(scalar(an["inputs"][2])) if len(an["inputs"]) > 2 else float(an["attrs"].get("max", np.inf))
                        if lo == 0.0 and hi == 6.0:
                            act = "relu6"
                    if act is not None:
                        sc, zp = float(scalar(qn["inputs"][1])), int(scalar(qn["inputs"][2] if len(qn["inputs"]) > 2 else ""))
                        t = m.qlinear_act(tens[ins[0]], act, alpha, sc, zp)
                        out = qn["outputs"][0]
                        qparams[out] = (sc, zp)
                        skip.update((r1[0], r2[0]))
                        fused = True
            if not fused:
                t = m.dequantize(tens[ins[0]])
        elif op == "QLinearConv":
            check_q(ins[0], ins[1], ins[2])
            if ins[5] and np.any(consts[ins[5]] != 0):
                raise NotImplementedError("QLinearConv with a non-zero weight zero point")
            s, p, d, ap = _pool_or_conv_attrs(a, [1, 1])
            if ap != "NOTSET":
                raise NotImplementedError("QLinearConv with auto_pad")
            sc, zp = float(scalar(ins[6])), int(scalar(ins[7]))
            bias = consts[ins[8]] if len(ins) > 8 and ins[8] else None
            t = m.qlinearconv(tens[ins[0]], consts[ins[3]], consts[ins[4]], bias, sc, zp, s, p if p is not None else [0, 0, 0, 0],
                              d, a.get("group", 1))
            qparams[out] = (sc, zp)
        elif op == "QLinearAdd":
            check_q(ins[0], ins[1], ins[2])
            check_q(ins[3], ins[4], ins[5])
            sc, zp = float(scalar(ins[6])), int(scalar(ins[7]))
            t = m.qlinear_add(tens[ins[0]], tens[ins[3]], sc, zp)
            qparams[out] = (sc, zp)
        elif op == "QLinearGlobalAveragePool":
            check_q(ins[0], ins[1], ins[2])
            if a.get("channels_last", 0):
                raise NotImplementedError("QLinearGlobalAveragePool with channels_last")
            sc, zp = float(scalar(ins[3])), int(scalar(ins[4]))
            t = m.qlinear_global_avgpool(tens[ins[0]], sc, zp)
            qparams[out] = (sc, zp)
        else:
            raise NotImplementedError(f"ONNX operator {op} is outside the hot path")
        tens[out] = t
    return m.finalize()
