"""Test infrastructure: writes the int8 benchmark networks as ONNX files (protobuf wire format by hand, no onnx package)
in QOperator form -- QLinearConv, MaxPool, QLinearAdd / QLinearGlobalAveragePool (com.microsoft) and the
DequantizeLinear -> activation -> QuantizeLinear idiom -- so that the ONNX front end can be exercised on them."""
import struct

import numpy as np


def _varint(n):
    n &= (1 << 64) - 1
    out = bytearray()
    while True:
        b = n & 0x7F
        n >>= 7
        out.append(b | (0x80 if n else 0))
        if not n:
            return bytes(out)


def _key(field, wt):
    return _varint((field << 3) | wt)


def _ld(field, payload):
    return _key(field, 2) + _varint(len(payload)) + payload


def _int(field, v):
    return _key(field, 0) + _varint(int(v))


_ONNX_TYPE = {np.dtype(np.float32): 1, np.dtype(np.uint8): 2, np.dtype(np.int8): 3, np.dtype(np.int32): 6, np.dtype(np.int64): 7}


def tensor(name, arr):
    arr = np.ascontiguousarray(arr)
    out = b"".join(_int(1, d) for d in arr.shape)
    out += _int(2, _ONNX_TYPE[arr.dtype]) + _ld(8, name.encode()) + _ld(9, arr.astype(arr.dtype.newbyteorder("<")).tobytes())
    return out


def attr(name, v):
    out = _ld(1, name.encode())
    if isinstance(v, float):
        return out + _key(2, 5) + struct.pack("<f", v) + _int(20, 1)
    if isinstance(v, int):
        return out + _int(3, v) + _int(20, 2)
    if isinstance(v, str):
        return out + _ld(4, v.encode()) + _int(20, 3)
    return out + b"".join(_int(8, i) for i in v) + _int(20, 7)


def node(op, inputs, outputs, domain="", **attrs):
    out = b"".join(_ld(1, i.encode()) for i in inputs) + b"".join(_ld(2, o.encode()) for o in outputs)
    out += _ld(3, (op + "_" + outputs[0]).encode()) + _ld(4, op.encode())
    out += b"".join(_ld(5, attr(k, v)) for k, v in attrs.items())
    if domain:
        out += _ld(7, domain.encode())
    return out


def value_info(name, shape, dtype):
    dims = b"".join(_ld(1, _int(1, d)) for d in shape)
    ttype = _int(1, _ONNX_TYPE[np.dtype(dtype)]) + _ld(2, dims)
    return _ld(1, name.encode()) + _ld(2, _ld(1, ttype))


def model(nodes, initializers, inputs, outputs):
    graph = b"".join(_ld(1, n) for n in nodes) + _ld(2, b"zant_test_graph")
    graph += b"".join(_ld(5, t) for t in initializers) + b"".join(_ld(11, v) for v in inputs) + b"".join(_ld(12, v) for v in outputs)
    opsets = _ld(8, _ld(1, b"") + _int(2, 13)) + _ld(8, _ld(1, b"com.microsoft") + _int(2, 1))
    return _int(1, 8) + opsets + _ld(7, graph)


def int8_network(arch, params, quant, batch):
    """The layer list of zant_amd.networks as ONNX bytes; returns (bytes, output shape)."""
    nodes, inits = [], []
    cnt = [0]

    def const(arr):
        cnt[0] += 1
        name = f"c{cnt[0]}"
        inits.append(tensor(name, np.asarray(arr)))
        return name

    def qp(scale, zp):
        return const(np.float32(scale)), const(np.uint8(zp))

    c, h, w = arch["input"]
    t, shape = "input", (batch, c, h, w)
    s, z = quant["input"]
    outs, meta = [], []
    for i, (L, P, Q) in enumerate(zip(arch["layers"], params, quant["layers"])):
        o = f"t{i}"
        if L["op"] == "conv":
            xs, xz = qp(s, z)
            ys, yz = qp(Q[0], Q[1])
            K = L["cout"]
            ins = [t, xs, xz, const(P["w"]), const(P["w_scale"]), const(np.zeros(K, np.int8)), ys, yz, const(P["bias"])]
            co = o + "_conv" if L["act"] else o
            nodes.append(node("QLinearConv", ins, [co], strides=[L["stride"]] * 2, pads=[L["pad"]] * 4, dilations=[1, 1],
                              group=L["group"], kernel_shape=[L["k"], L["k"]]))
            s, z = Q[0], Q[1]
            oh = (shape[2] + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            ow = (shape[3] + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            shape = (batch, K, oh, ow)
            if L["act"]:
                ds, dz = qp(s, z)
                nodes.append(node("DequantizeLinear", [co, ds, dz], [o + "_f"]))
                if L["act"] == "leaky":
                    nodes.append(node("LeakyRelu", [o + "_f"], [o + "_a"], alpha=float(L["alpha"])))
                elif L["act"] == "relu6":
                    nodes.append(node("Clip", [o + "_f", const(np.float32(0.0)), const(np.float32(6.0))], [o + "_a"]))
                else:
                    nodes.append(node("Relu", [o + "_f"], [o + "_a"]))
                as_, az = qp(Q[2], Q[3])
                nodes.append(node("QuantizeLinear", [o + "_a", as_, az], [o]))
                s, z = Q[2], Q[3]
        elif L["op"] == "pool":
            nodes.append(node("MaxPool", [t], [o], kernel_shape=[2, 2], strides=[2, 2]))
            shape = (batch, shape[1], shape[2] // 2, shape[3] // 2)
        elif L["op"] == "add":
            r, (rs, rz) = outs[L["res"]], meta[L["res"]]
            a_s, a_z = qp(s, z)
            b_s, b_z = qp(rs, rz)
            c_s, c_z = qp(Q[0], Q[1])
            nodes.append(node("QLinearAdd", [t, a_s, a_z, r, b_s, b_z, c_s, c_z], [o], domain="com.microsoft"))
            s, z = Q[0], Q[1]
        elif L["op"] == "gap":
            xs, xz = qp(s, z)
            ys, yz = qp(Q[0], Q[1])
            nodes.append(node("QLinearGlobalAveragePool", [t, xs, xz, ys, yz], [o], domain="com.microsoft", channels_last=0))
            s, z = Q[0], Q[1]
            shape = (batch, shape[1], 1, 1)
        t = o
        outs.append(t)
        meta.append((s, z))
    data = model(nodes, inits, [value_info("input", (batch, c, h, w), np.uint8)], [value_info(t, shape, np.uint8)])
    return data, shape
