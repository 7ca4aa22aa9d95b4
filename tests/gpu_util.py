"""Helpers of the GPU parity tests: load the package, move numpy arrays to the card and back."""
import numpy as np
import torch

import __graft_entry__ as ge

za = ge.load_package()
tm = za.tensor_math
ZantError = za.ZantError

RTOL, ATOL = 1e-4, 1e-5  # the f32 tolerance of the hot path (bit-exact is required for int8)


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def T(d, dtype=np.float32):
    return None if d is None else np.array(d["data"], dtype=dtype).reshape(d["shape"])
