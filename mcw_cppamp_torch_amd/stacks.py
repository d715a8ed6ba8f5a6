"""The convolution stacks of the benchmark configurations, built from the nn
modules exactly as a Torch user would write them (nn.Sequential of
SpatialConvolutionMM / ReLU / SpatialMaxPooling), plus the bookkeeping of
their algorithmic work.

Layer tuples: ("conv", C, M, kW, kH, dW, dH, padW, padH), ("relu",),
("pool", kW, kH, dW, dH).
"""
import math

import numpy as np

from . import nn


def _c(cin, cout, k, s=1, p=0):
    return ("conv", cin, cout, k, k, s, s, p, p)


def _p(k, s):
    return ("pool", k, k, s, s)


R = ("relu",)

STACKS = {
    # single layer of the first configuration
    "conv1_b16": {"batch": 16, "input": (3, 224, 224), "init": "uniform",
                  "layers": [_c(3, 64, 11, 4, 2)]},
    "alexnet": {"batch": 128, "input": (3, 224, 224), "init": "uniform",
                "layers": [_c(3, 64, 11, 4, 2), R, _p(3, 2),
                           _c(64, 192, 5, 1, 2), R, _p(3, 2),
                           _c(192, 384, 3, 1, 1), R,
                           _c(384, 256, 3, 1, 1), R,
                           _c(256, 256, 3, 1, 1), R, _p(3, 2)]},
    "overfeat": {"batch": 128, "input": (3, 231, 231), "init": "uniform",
                 "layers": [_c(3, 96, 11, 4, 0), R, _p(2, 2),
                            _c(96, 256, 5, 1, 0), R, _p(2, 2),
                            _c(256, 512, 3, 1, 1), R,
                            _c(512, 1024, 3, 1, 1), R,
                            _c(1024, 1024, 3, 1, 1), R, _p(2, 2)]},
    "vgg_a": {"batch": 64, "input": (3, 224, 224), "init": "normal",
              "layers": [_c(3, 64, 3, 1, 1), R, _p(2, 2),
                         _c(64, 128, 3, 1, 1), R, _p(2, 2),
                         _c(128, 256, 3, 1, 1), R,
                         _c(256, 256, 3, 1, 1), R, _p(2, 2),
                         _c(256, 512, 3, 1, 1), R,
                         _c(512, 512, 3, 1, 1), R, _p(2, 2),
                         _c(512, 512, 3, 1, 1), R,
                         _c(512, 512, 3, 1, 1), R, _p(2, 2)]},
}


def trace_shapes(layers, in_shape):
    """Per-layer (kind, in_shape, out_shape) for a (C,H,W) input."""
    C, H, W = in_shape
    out = []
    for l in layers:
        if l[0] == "conv":
            _, cin, cout, kW, kH, dW, dH, pW, pH = l
            assert cin == C, (cin, C)
            Ho, Wo = (H + 2 * pH - kH) // dH + 1, (W + 2 * pW - kW) // dW + 1
            out.append((l, (C, H, W), (cout, Ho, Wo)))
            C, H, W = cout, Ho, Wo
        elif l[0] == "pool":
            _, kW, kH, dW, dH = l
            Ho, Wo = (H - kH) // dH + 1, (W - kW) // dW + 1
            out.append((l, (C, H, W), (C, Ho, Wo)))
            H, W = Ho, Wo
        else:
            out.append((l, (C, H, W), (C, H, W)))
    return out


def work(name, batch=None):
    """Algorithmic work of one forward+backward pass of a stack: GEMM flops
    (2*M*N*K per image, three GEMMs per conv layer) and the bytes of the
    HBM-bound kernels (im2col once, col2im once, pool fwd+bwd, ReLU fwd+bwd)."""
    cfg = STACKS[name]
    B = batch or cfg["batch"]
    flops = 0.0
    by = {"im2col": 0.0, "col2im": 0.0, "maxpool_fwd": 0.0, "maxpool_bwd": 0.0, "threshold_fwd": 0.0,
          "threshold_bwd": 0.0}
    for l, (C, H, W), (Co, Ho, Wo) in trace_shapes(cfg["layers"], cfg["input"]):
        if l[0] == "conv":
            K, N = C * l[3] * l[4], Ho * Wo
            flops += 3 * 2.0 * Co * N * K * B
            by["im2col"] += 4.0 * (C * H * W + K * N) * B
            by["col2im"] += 4.0 * (C * H * W + K * N) * B
        elif l[0] == "pool":
            by["maxpool_fwd"] += 4.0 * (C * H * W + 3 * C * Ho * Wo) * B
            by["maxpool_bwd"] += 4.0 * (C * H * W + 3 * C * Ho * Wo) * B
        else:
            n = C * H * W * B
            by["threshold_fwd"] += 8.0 * n
            by["threshold_bwd"] += 12.0 * n
    return {"gemm_flops": flops, "bytes": by}


def build(name, seed_base=0):
    """nn.Sequential for a stack with seeded weights (host tensors; call .gpu()).
    Seeds: seed_base + 10*layer_index + {1: weight, 2: bias}."""
    cfg = STACKS[name]
    net = nn.Sequential()
    for li, l in enumerate(cfg["layers"]):
        if l[0] == "conv":
            _, cin, cout, kW, kH, dW, dH, pW, pH = l
            m = nn.SpatialConvolutionMM(cin, cout, kW, kH, dW, dH, 0, padW=pW, padH=pH)
            fan_in = cin * kH * kW
            rw = np.random.Generator(np.random.PCG64(seed_base + 10 * li + 1))
            rb = np.random.Generator(np.random.PCG64(seed_base + 10 * li + 2))
            if cfg["init"] == "normal":
                w = rw.normal(0.0, math.sqrt(2.0 / fan_in), size=(cout, fan_in))
                b = np.zeros(cout)
            else:
                s = 1.0 / math.sqrt(fan_in)
                w = rw.uniform(-s, s, size=(cout, fan_in))
                b = rb.uniform(-s, s, size=(cout,))
            m._assign("weight", w)
            m._assign("bias", b)
            m.gradWeight[...] = 0
            m.gradBias[...] = 0
            net.add(m)
        elif l[0] == "pool":
            net.add(nn.SpatialMaxPooling(l[1], l[2], l[3], l[4]))
        else:
            net.add(nn.ReLU())
    return net


def make_input(name, batch=None, seed=0):
    cfg = STACKS[name]
    B = batch or cfg["batch"]
    rng = np.random.Generator(np.random.PCG64(seed))
    return rng.uniform(-1.0, 1.0, size=(B,) + cfg["input"]).astype(np.float32)


def output_shape(name, batch=None):
    cfg = STACKS[name]
    B = batch or cfg["batch"]
    return (B,) + trace_shapes(cfg["layers"], cfg["input"])[-1][2]
