"""The five benchmark / parity workloads and their seeded synthetic inputs.

Shapes, distributions and seed follow the workload list this library is
measured on: x ~ U[-1,1] (ReLU'd N(0,1) for the ResNet-stage case), upstream
gradient dy ~ N(0,1), factors ~ N(0, sigma) with sigma = 1/sqrt(R*C) read as a
standard deviation (1/sqrt(R*K) for the backward-data case), numpy
``default_rng(seed)`` drawing x, dy, FK, FC, FH, FW in that order.
"""
from collections import namedtuple

import numpy as np

Workload = namedtuple("Workload", "name pass_ N C H W pad T Y X R x_dist")

WORKLOADS = {
    "C1": Workload("C1", "forward", 1, 16, 32, 32, 1, 16, 3, 3, 8, "uniform"),
    "C2": Workload("C2", "forward", 16, 64, 32, 32, 1, 64, 3, 3, 16, "uniform"),
    "C3": Workload("C3", "forward", 32, 256, 56, 56, 1, 256, 3, 3, 32, "relu_normal"),
    "C4": Workload("C4", "backward_data", 32, 128, 28, 28, 2, 128, 5, 5, 16, "uniform"),
    "C5": Workload("C5", "backward_filter", 64, 256, 14, 14, 1, 256, 3, 3, 64, "uniform"),
}


def algorithmic_bytes(w, pass_=None):
    """4*(N*C*H*W + N*T*H*W + R*(T+C+Y+X)) for forward / backward-data -- the
    reference's own formula (Cuda_kernels/cp4Conv2d.cu:176-178) -- and the same
    with the factor term doubled for backward-filter (factors read, four
    gradients written)."""
    pass_ = pass_ or w.pass_
    act = w.N * w.C * w.H * w.W + w.N * w.T * w.H * w.W
    fac = w.R * (w.T + w.C + w.Y + w.X)
    return 4 * (act + (2 * fac if pass_ == "backward_filter" else fac))


def minimal_flops(w, pass_=None):
    pass_ = pass_ or w.pass_
    px = w.N * w.H * w.W
    if pass_ == "backward_filter":
        return 2 * w.R * (2 * w.C + 2 * w.T + 3 * w.Y + 3 * w.X) * px
    return 2 * w.R * (w.C + w.T + w.Y + w.X) * px


def make_inputs(w, seed=0):
    """dict of float32 numpy arrays: x, dy, FK, FC, FH, FW."""
    rng = np.random.default_rng(seed)
    if w.x_dist == "relu_normal":
        x = np.maximum(rng.standard_normal((w.N, w.C, w.H, w.W), np.float32), 0)
    else:
        x = rng.random((w.N, w.C, w.H, w.W), np.float32) * 2 - 1
    dy = rng.standard_normal((w.N, w.T, w.H, w.W), np.float32)
    sigma = 1.0 / np.sqrt(w.R * (w.T if w.pass_ == "backward_data" else w.C))
    fac = {k: (rng.standard_normal((d, w.R), np.float32) * np.float32(sigma))
           for k, d in (("FK", w.T), ("FC", w.C), ("FH", w.Y), ("FW", w.X))}
    return dict(x=x, dy=dy, **fac)
