"""Seeded synthetic networks of the benchmark configurations, built on the operator mirror.

``ReadmeCNN`` is the reference's README / src/main.zig:41-272 model (Conv32-ReLU-MaxPool-Conv64-ReLU-MaxPool-
Flatten-Dense512-ReLU-Dense10-Softmax) with He-normal weights and zero biases from one numpy seed.  Each layer
is one call into libzant_hip.so on preallocated device buffers (ReLU rides in the producing kernel's epilogue).
"""
import numpy as np
import torch

from . import tensor_math as tm


def readme_cnn_params(seed=0):
    g = np.random.default_rng(seed)

    def he(shape, fan_in):
        return (g.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)

    return {
        "w1": he((32, 1, 3, 3), 9), "b1": np.zeros(32, np.float32),
        "w2": he((64, 32, 3, 3), 288), "b2": np.zeros(64, np.float32),
        "g1": he((1, 1, 1600, 512), 1600), "c1": np.zeros((1, 1, 1, 512), np.float32),
        "g2": he((1, 1, 512, 10), 512), "c2": np.zeros((1, 1, 1, 10), np.float32),
    }


def readme_cnn_flops_per_inference():
    """Multiply-adds x 2 of one inference.  "total" counts the graph as written (conv2 at its 11 x 11 outputs);
    "executed" counts what the fused pass computes: the 2x2/2 pool behind conv2 drops row and column 10, and the
    fused kernel does not compute them (10 x 10 outputs)."""
    conv1 = 2 * 32 * 26 * 26 * 9
    conv2 = 2 * 64 * 11 * 11 * 32 * 9
    conv2_executed = 2 * 64 * 10 * 10 * 32 * 9
    gemm1 = 2 * 1600 * 512
    gemm2 = 2 * 512 * 10
    return {"conv1": conv1, "conv2": conv2, "conv2_executed": conv2_executed, "gemm1": gemm1, "gemm2": gemm2,
            "total": conv1 + conv2 + gemm1 + gemm2, "executed": conv1 + conv2_executed + gemm1 + gemm2}


def build_readme_cnn_model(ctx, batch, params):
    """The README CNN as a zant_model: the node list a generated predict() would call, fused and arena-planned."""
    from .model import Model
    m = Model(ctx)
    t = m.input((batch, 1, 28, 28))
    t = m.conv(t, params["w1"], params["b1"], [1, 1], None, None, 1, None)
    t = m.relu(t)
    t = m.maxpool(t, [2, 2], [2, 2])
    t = m.conv(t, params["w2"], params["b2"], [1, 1], None, None, 1, None)
    t = m.relu(t)
    t = m.maxpool(t, [2, 2], [2, 2])
    t = m.reshape(t, [1, 1, batch, 1600])
    t = m.gemm(t, params["g1"], params["c1"])
    t = m.relu(t)
    t = m.gemm(t, params["g2"], params["c2"])
    t = m.reshape(t, [batch, 10])
    t = m.softmax(t)
    return m.finalize()


class ReadmeCNN:
    def __init__(self, batch, params, device="cuda:0"):
        self.n = batch
        dev = torch.device(device)
        self.p = {k: torch.from_numpy(v).to(dev) for k, v in params.items()}
        f = dict(dtype=torch.float32, device=dev)
        # every activation is allocated once; a forward pass allocates nothing
        self.a1 = torch.zeros((batch, 32, 26, 26), **f)
        self.p1 = torch.zeros((batch, 32, 13, 13), **f)
        self.a2 = torch.zeros((batch, 64, 11, 11), **f)
        self.p2 = torch.zeros((batch, 64, 5, 5), **f)
        self.h1 = torch.zeros((1, 1, batch, 512), **f)
        self.h2 = torch.zeros((1, 1, batch, 10), **f)
        self.out = torch.zeros((batch, 10), **f)

        self.plans = None
        self.fused = False

    def prepare(self, fuse_pool=False):
        """Prepared-weights handles for the two convolutions: forward() then calls conv2d_f32_packed (the weights are
        packed at the first call, later calls launch the convolution kernels only).  fuse_pool: each handle is the chain
        Conv -> ReLU -> MaxPool 2x2/2 in one kernel, as a code generator that peephole-fuses the chain would emit it."""
        p = self.p
        if fuse_pool:
            self.plans = (tm.ConvPlan((self.n, 1, 28, 28), p["w1"], p["b1"], self.p1.shape, [1, 1], None, None, 1, None, "relu", True),
                          tm.ConvPlan(self.p1.shape, p["w2"], p["b2"], self.p2.shape, [1, 1], None, None, 1, None, "relu", True))
        else:
            self.plans = (tm.ConvPlan((self.n, 1, 28, 28), p["w1"], p["b1"], self.a1.shape, [1, 1], None, None, 1, None, "relu"),
                          tm.ConvPlan(self.p1.shape, p["w2"], p["b2"], self.a2.shape, [1, 1], None, None, 1, None, "relu"))
        self.fused = bool(fuse_pool)
        return self

    def forward(self, x):
        p = self.p
        if self.plans and self.fused:
            self.plans[0](x, self.p1)
            self.plans[1](self.p1, self.p2)
        else:
            if self.plans:
                self.plans[0](x, self.a1)
            else:
                tm.conv_lean(x, p["w1"], self.a1, p["b1"], [1, 1], None, None, 1, None, "relu")
            tm.onnx_maxpool_lean(self.a1, self.p1, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
            if self.plans:
                self.plans[1](self.p1, self.a2)
            else:
                tm.conv_lean(self.p1, p["w2"], self.a2, p["b2"], [1, 1], None, None, 1, None, "relu")
            tm.onnx_maxpool_lean(self.a2, self.p2, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
        flat = self.p2.view(1, 1, self.n, 1600)  # reshape_lean as a view
        tm.gemm_lean(flat, p["g1"], p["c1"], 1.0, 1.0, False, False, self.h1, "relu")
        tm.gemm_lean(self.h1, p["g2"], p["c2"], 1.0, 1.0, False, False, self.h2)
        tm.softmax_lean(self.h2.view(self.n, 10), self.out)
        return self.out


# ------------------------------------------------------------------------------------------------
# int8 networks of the benchmark configurations (tiny-YOLO style detector, MobileNetV2-0.35 @ 96)
# ------------------------------------------------------------------------------------------------
# An architecture is a list of layer dicts executed in order; "src"/"res" name earlier layer outputs.
#   conv : QLinearConv  (k, stride, pad, cin, cout, group)   [+ act: None | "leaky" | "relu6"]
#   pool : MaxPool 2x2/2 on the quantised values
#   add  : quantised residual add with the output of layer `res`
#   gap  : quantised global average pool
# Activation scales / zero points are NOT chosen here: they come from a calibration pass recorded as a
# fixture (tests/golden/int8_networks.json) and are passed in as `quant`.

def _make_divisible(v, d=8):
    return max(d, int(v + d / 2) // d * d)


def tiny_yolo_arch():
    """Six 3x3 pad-1 convolutions 3->16->32->64->128->256->256 with LeakyReLU(0.1), a 2x2/2 MaxPool after each of
    the first five, and a 1x1 head to 3*(5+4) = 27 channels; 3x96x96 input -> 27x3x3 output."""
    arch, cin = [], 3
    for i, cout in enumerate([16, 32, 64, 128, 256, 256]):
        arch.append(dict(op="conv", k=3, stride=1, pad=1, cin=cin, cout=cout, group=1, act="leaky", alpha=0.1))
        if i < 5:
            arch.append(dict(op="pool"))
        cin = cout
    arch.append(dict(op="conv", k=1, stride=1, pad=0, cin=256, cout=27, group=1, act=None))
    return dict(name="tiny_yolo_int8", input=(3, 96, 96), layers=arch)


def mobilenet_v2_035_arch():
    """MobileNetV2, width 0.35, 96x96 input: 3x3/2 stem, 17 inverted-residual blocks (1x1 expand x6 + ReLU6,
    3x3 depthwise + ReLU6, 1x1 linear projection, residual add where shapes match), 1x1 to 1280 + ReLU6, global
    average pool, 1280->1000 classifier (a 1x1 QLinearConv on the pooled [N,1280,1,1] tensor)."""
    w = 0.35
    layers = [dict(op="conv", k=3, stride=2, pad=1, cin=3, cout=_make_divisible(32 * w), group=1, act="relu6")]
    cin = layers[0]["cout"]
    for t, c, n, s in [(6, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]:
        cout = _make_divisible(c * w)
        for i in range(n):
            stride = s if i == 0 else 1
            block_in = len(layers) - 1  # index of the layer whose output feeds this block
            hidden = cin * t
            layers.append(dict(op="conv", k=1, stride=1, pad=0, cin=cin, cout=hidden, group=1, act="relu6"))
            layers.append(dict(op="conv", k=3, stride=stride, pad=1, cin=hidden, cout=hidden, group=hidden, act="relu6"))
            layers.append(dict(op="conv", k=1, stride=1, pad=0, cin=hidden, cout=cout, group=1, act=None))
            if stride == 1 and cin == cout:
                layers.append(dict(op="add", res=block_in))
            cin = cout
    layers.append(dict(op="conv", k=1, stride=1, pad=0, cin=cin, cout=1280, group=1, act="relu6"))
    layers.append(dict(op="gap"))
    layers.append(dict(op="conv", k=1, stride=1, pad=0, cin=1280, cout=1000, group=1, act=None))
    return dict(name="mobilenet_v2_035_int8", input=(3, 96, 96), layers=layers)


def int8_params(arch, seed=0):
    """Per-channel int8 weights ~U{-127..127}, per-channel scales sized like He initialisation, int32 biases."""
    g = np.random.default_rng(seed)
    params = []
    for L in arch["layers"]:
        if L["op"] != "conv":
            params.append(None)
            continue
        cg = L["cin"] // L["group"]
        fan_in = cg * L["k"] * L["k"]
        w = g.integers(-127, 128, (L["cout"], cg, L["k"], L["k"]), dtype=np.int8)
        ws = (np.sqrt(2.0 / fan_in) / 73.0 * g.uniform(0.5, 1.5, L["cout"])).astype(np.float32)
        b = g.integers(-64, 65, L["cout"], dtype=np.int32)
        params.append(dict(w=w, w_scale=ws, bias=b))
    return params


def int8_macs_per_inference(arch):
    c, h, w = arch["input"]
    macs = 0
    for L in arch["layers"]:
        if L["op"] == "conv":
            oh = (h + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            ow = (w + 2 * L["pad"] - L["k"]) // L["stride"] + 1
            macs += L["cout"] * oh * ow * (L["cin"] // L["group"]) * L["k"] * L["k"]
            c, h, w = L["cout"], oh, ow
        elif L["op"] == "pool":
            h, w = h // 2, w // 2
        elif L["op"] == "gap":
            h, w = 1, 1
    return macs


def build_int8_model(ctx, arch, params, quant, batch):
    """quant: {"input": [scale, zp], "layers": [[conv_scale, conv_zp, out_scale, out_zp] | [scale, zp] | None ...]}"""
    from .model import Model, U8
    m = Model(ctx)
    c, h, w = arch["input"]
    t = m.input((batch, c, h, w), U8, quant["input"][0], int(quant["input"][1]))
    outs = []
    for L, P, Q in zip(arch["layers"], params, quant["layers"]):
        if L["op"] == "conv":
            t = m.qlinearconv(t, P["w"], P["w_scale"], P["bias"], Q[0], int(Q[1]), [L["stride"]] * 2, [L["pad"]] * 4,
                              [1, 1], L["group"])
            if L["act"]:
                t = m.qlinear_act(t, L["act"], L.get("alpha", 0.0), Q[2], int(Q[3]))
        elif L["op"] == "pool":
            t = m.maxpool(t, [2, 2], [2, 2])
        elif L["op"] == "add":
            t = m.qlinear_add(t, outs[L["res"]], Q[0], int(Q[1]))
        elif L["op"] == "gap":
            t = m.qlinear_global_avgpool(t, Q[0], int(Q[1]))
        outs.append(t)
    return m.finalize()
