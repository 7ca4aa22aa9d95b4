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
    conv1 = 2 * 32 * 26 * 26 * 9
    conv2 = 2 * 64 * 11 * 11 * 32 * 9
    gemm1 = 2 * 1600 * 512
    gemm2 = 2 * 512 * 10
    return {"conv1": conv1, "conv2": conv2, "gemm1": gemm1, "gemm2": gemm2, "total": conv1 + conv2 + gemm1 + gemm2}


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

    def forward(self, x):
        p = self.p
        tm.conv_lean(x, p["w1"], self.a1, p["b1"], [1, 1], None, None, 1, None, "relu")
        tm.onnx_maxpool_lean(self.a1, self.p1, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
        tm.conv_lean(self.p1, p["w2"], self.a2, p["b2"], [1, 1], None, None, 1, None, "relu")
        tm.onnx_maxpool_lean(self.a2, self.p2, [2, 2], [2, 2], [1, 1], [0, 0, 0, 0])
        flat = self.p2.view(1, 1, self.n, 1600)  # reshape_lean as a view
        tm.gemm_lean(flat, p["g1"], p["c1"], 1.0, 1.0, False, False, self.h1, "relu")
        tm.gemm_lean(self.h1, p["g2"], p["c2"], 1.0, 1.0, False, False, self.h2)
        tm.softmax_lean(self.h2.view(self.n, 10), self.out)
        return self.out
