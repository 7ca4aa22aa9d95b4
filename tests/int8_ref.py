"""Oracle forward pass (and calibration) of the int8 benchmark networks; test infrastructure only."""
import numpy as np

from oracle import oracle as zo


def forward(arch, params, quant, x, keep=False):
    """Runs the layer list with the CPU oracle; returns the final u8 tensor (and all layer outputs with keep=True)."""
    t = x
    s, z = quant["input"]
    outs, meta = [], []
    for L, P, Q in zip(arch["layers"], params, quant["layers"]):
        if L["op"] == "conv":
            t = zo.qlinearconv(t, s, int(z), P["w"], P["w_scale"], None, Q[0], int(Q[1]), P["bias"], [L["stride"]] * 2,
                               [L["pad"]] * 4, [1, 1], L["group"])
            s, z = Q[0], Q[1]
            if L["act"]:
                t = zo.qlinear_act(t, s, int(z), L["act"], L.get("alpha", 0.0), Q[2], int(Q[3]))
                s, z = Q[2], Q[3]
        elif L["op"] == "pool":
            t = zo.onnx_maxpool(t, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
        elif L["op"] == "add":
            r, (rs, rz) = outs[L["res"]], meta[L["res"]]
            t = zo.qlinear_add(t, s, int(z), r, rs, int(rz), Q[0], int(Q[1]))
            s, z = Q[0], Q[1]
        elif L["op"] == "gap":
            t = zo.qlinear_global_avgpool(t, s, int(z), Q[0], int(Q[1]))
            s, z = Q[0], Q[1]
        outs.append(t)
        meta.append((s, z))
    return (t, outs) if keep else t


def calibrate(arch, params, x, in_scale=0.02, in_zp=128):
    """Chooses per-tensor activation scales from the real-valued range each layer produces on the batch `x`:
    conv outputs are centred on 128 with scale max|v|/120; activation outputs use the range of act(v)."""
    quant = {"input": [in_scale, in_zp], "layers": []}
    t, s, z = x, np.float32(in_scale), in_zp
    outs, meta = [], []
    for L, P in zip(arch["layers"], params):
        if L["op"] == "conv":
            acc = zo.qconv_acc(t, int(z), P["w"], None, P["bias"], [L["stride"]] * 2, [L["pad"]] * 4, [1, 1], L["group"])
            real = acc.astype(np.float64) * float(s) * P["w_scale"].astype(np.float64)[None, :, None, None]
            cs = np.float32(max(np.abs(real).max(), 1e-6) / 120.0)
            q = [float(cs), 128]
            t = zo.qlinearconv(t, s, int(z), P["w"], P["w_scale"], None, cs, 128, P["bias"], [L["stride"]] * 2,
                               [L["pad"]] * 4, [1, 1], L["group"])
            s, z = cs, 128
            if L["act"]:
                v = zo.dequantize_linear(t, s, z).astype(np.float64)
                if L["act"] == "leaky":
                    v = np.where(v <= 0, L["alpha"] * v, v)
                else:
                    v = np.clip(v, 0, 6)
                lo, hi = min(v.min(), 0.0), max(v.max(), 1e-6)
                a_s = np.float32((hi - lo) / 250.0)
                a_z = int(np.clip(round(-lo / float(a_s)), 0, 255))
                q += [float(a_s), a_z]
                t = zo.qlinear_act(t, s, int(z), L["act"], L.get("alpha", 0.0), a_s, a_z)
                s, z = a_s, a_z
            quant["layers"].append(q)
        elif L["op"] == "pool":
            t = zo.onnx_maxpool(t, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
            quant["layers"].append(None)
        elif L["op"] == "add":
            r, (rs, rz) = outs[L["res"]], meta[L["res"]]
            v = zo.dequantize_linear(t, s, z).astype(np.float64) + zo.dequantize_linear(r, rs, rz).astype(np.float64)
            a_s = np.float32(max(np.abs(v).max(), 1e-6) / 120.0)
            quant["layers"].append([float(a_s), 128])
            t = zo.qlinear_add(t, s, int(z), r, rs, int(rz), a_s, 128)
            s, z = a_s, 128
        elif L["op"] == "gap":
            quant["layers"].append([float(s), int(z)])
            t = zo.qlinear_global_avgpool(t, s, int(z), s, int(z))
        outs.append(t)
        meta.append((s, z))
    return quant
