"""Shared test helpers: golden-fixture inputs, brute-force restatements written
independently of the oracle (pure numpy / Python loops from the closed-form
index maps), seeded generators and the parity metrics."""
import json
import math
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_kat.json")


def load_kat():
    with open(GOLDEN) as f:
        return json.load(f)


def wsum(a):
    v = np.asarray(a, dtype=np.float64).ravel()
    return float(np.sum(v * ((np.arange(v.size) % 97) + 1)))


def check_digest(arr, dig):
    """Compare an array with a fixture digest (shape, sum, wsum, first8, last)."""
    arr = np.asarray(arr)
    assert list(arr.shape) == dig["shape"], (arr.shape, dig["shape"])
    flat = arr.ravel()
    assert float(flat.astype(np.float64).sum()) == dig["sum"]
    assert wsum(flat) == dig["wsum"]
    n8 = len(dig["first8"])
    assert flat[:n8].tolist() == [float(v) for v in dig["first8"]]
    assert float(flat[-1]) == dig["last"]


# ---- formula-defined inputs of the fixture --------------------------------
def kat_conv_inputs(cfg):
    B, C, H, W, M = cfg["B"], cfg["C"], cfg["H"], cfg["W"], cfg["M"]
    kH, kW = cfg["kH"], cfg["kW"]
    Ho = (H + 2 * cfg["pH"] - kH) // cfg["sH"] + 1
    Wo = (W + 2 * cfg["pW"] - kW) // cfg["sW"] + 1
    b, c, h, w = np.ogrid[:B, :C, :H, :W]
    inp = (((37 * b + 11 * c + 5 * h + 3 * w) % 7) - 3).astype(np.float32)
    m, k = np.ogrid[:M, :C * kH * kW]
    weight = (((13 * m + 7 * k) % 5) - 2).astype(np.float32)
    bias = (np.arange(M) - 1).astype(np.float32)
    b, m, h, w = np.ogrid[:B, :M, :Ho, :Wo]
    go = (((5 * b + 4 * m + h * h + 3 * w) % 7) - 2).astype(np.float32)
    return inp, weight, bias, go


def kat_pool_inputs(cfg):
    C, H, W = cfg["C"], cfg["H"], cfg["W"]
    Ho = (H - cfg["kH"]) // cfg["dH"] + 1
    Wo = (W - cfg["kW"]) // cfg["dW"] + 1
    c, h, w = np.ogrid[:C, :H, :W]
    inp = ((3 * c + 2 * h + 5 * w) % 4).astype(np.float32)[None]
    c, i, j = np.ogrid[:C, :Ho, :Wo]
    go = (9 * c + 3 * i + j + 1).astype(np.float32)[None]
    return inp, go


# ---- brute force from the closed-form index maps --------------------------
def brute_im2col(im, kH, kW, pH, pW, sH, sW):
    B, C, H, W = im.shape
    Ho, Wo = (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1
    col = np.zeros((B, C * kH * kW, Ho * Wo), np.float32)
    for b in range(B):
        for c in range(C):
            for kh in range(kH):
                for kw in range(kW):
                    k = (c * kH + kh) * kW + kw
                    for ho in range(Ho):
                        for wo in range(Wo):
                            y, x = ho * sH - pH + kh, wo * sW - pW + kw
                            if 0 <= y < H and 0 <= x < W:
                                col[b, k, ho * Wo + wo] = im[b, c, y, x]
    return col


def brute_col2im(col, C, H, W, kH, kW, pH, pW, sH, sW):
    """Per-pixel gather in kh-ascending, kw-ascending order with float32 adds
    starting from 0 -- the order the reference's accumulate loop produces."""
    B = col.shape[0]
    Ho, Wo = (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1
    im = np.zeros((B, C, H, W), np.float32)
    for b in range(B):
        for c in range(C):
            for y in range(H):
                for x in range(W):
                    acc = np.float32(0)
                    for kh in range(kH):
                        for kw in range(kW):
                            hy, wx = y + pH - kh, x + pW - kw
                            if hy % sH or wx % sW:
                                continue
                            ho, wo = hy // sH, wx // sW
                            if 0 <= ho < Ho and 0 <= wo < Wo:
                                acc = np.float32(acc + col[b, (c * kH + kh) * kW + kw, ho * Wo + wo])
                    im[b, c, y, x] = acc
    return im


def brute_maxpool(inp, kH, kW, dH, dW):
    B, C, H, W = inp.shape
    Ho, Wo = (H - kH) // dH + 1, (W - kW) // dW + 1
    out = np.empty((B, C, Ho, Wo), np.float32)
    ind = np.empty((2, B, C, Ho, Wo), np.float32)
    for b in range(B):
        for c in range(C):
            for i in range(Ho):
                for j in range(Wo):
                    best, by, bx = -math.inf, 0, 0
                    for y in range(kH):
                        for x in range(kW):
                            v = float(inp[b, c, i * dH + y, j * dW + x])
                            if v > best:
                                best, by, bx = v, y, x
                    out[b, c, i, j] = best
                    ind[0, b, c, i, j] = by + 1
                    ind[1, b, c, i, j] = bx + 1
    return out, ind


def brute_maxpool_bwd(go, ind, in_shape, dH, dW):
    B, C, H, W = in_shape
    Ho, Wo = go.shape[2:]
    gi = np.zeros(in_shape, np.float32)
    for b in range(B):
        for c in range(C):
            for i in range(Ho):
                for j in range(Wo):
                    y = int(ind[0, b, c, i, j]) - 1 + i * dH
                    x = int(ind[1, b, c, i, j]) - 1 + j * dW
                    gi[b, c, y, x] = np.float32(gi[b, c, y, x] + go[b, c, i, j])
    return gi


# ---- seeded inputs and parity metrics --------------------------------------
def rng_for(seed):
    return np.random.Generator(np.random.PCG64(seed))


def uniform(rng, shape, lo=-1.0, hi=1.0):
    return rng.uniform(lo, hi, size=shape).astype(np.float32)


def rel_err(got, ref):
    """Norm-wise max relative error: max|got-ref| / max|ref|."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    denom = max(float(np.max(np.abs(ref))), 1e-30)
    return float(np.max(np.abs(got - ref))) / denom


def elem_rel_err(got, ref):
    """Element-wise max relative error over the elements with |ref| > 1e-3 * max|ref| (smaller ones are
    dominated by cancellation and carry no relative meaning)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    top = float(np.max(np.abs(ref)))
    mask = np.abs(ref) > 1e-3 * top
    if not mask.any():
        return 0.0
    return float(np.max(np.abs(got - ref)[mask] / np.abs(ref)[mask]))


def both_rel_err(got, ref):
    """The larger of the norm-wise and the element-wise maximum relative error: what a test compares with the parity
    bound 1e-4*sqrt(reduction length), so that both readings of "maximum relative error" are held to it."""
    return max(rel_err(got, ref), elem_rel_err(got, ref))


MARGIN_LOG = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpurun_out",
                          "parity_margins.jsonl")


def check_close(tag, got, ref, k_red):
    """Asserts the bound 1e-4*sqrt(k_red) on the norm-wise error and on the element-wise maximum relative error (over
    the elements that carry a relative meaning, see elem_rel_err), and puts both observed errors on
    record (printed, and appended to the file MARGIN_LOG names) so the margin under the bound is known."""
    norm, elem, bound = rel_err(got, ref), elem_rel_err(got, ref), gemm_tol(k_red)
    rec = {"case": tag, "k_red": int(k_red), "bound": bound, "norm_rel_err": norm, "elem_rel_err": elem,
           "bound_used": norm / bound}
    print("parity %s: norm-wise %.3e, element-wise %.3e, bound %.3e (%.1f %% used)"
          % (tag, norm, elem, bound, 100.0 * norm / bound), flush=True)
    try:
        os.makedirs(os.path.dirname(MARGIN_LOG), exist_ok=True)
        with open(MARGIN_LOG, "a") as f:
            f.write(json.dumps(rec) + "\n")
    except OSError:
        pass
    assert norm < bound, rec
    assert elem < bound, rec
    return rec


def gemm_tol(k_red):
    """Parity bound for fp32 GEMM results: 1e-4 * sqrt(reduction length)."""
    return 1e-4 * math.sqrt(max(int(k_red), 1))


# ---- CPU-oracle evaluation of a whole stack --------------------------------
def oracle_stack(layers, params, x, grad_out, scale=1.0):
    """Runs forward+backward of a layer list through the CPU oracle with the
    sequencing of nn.Sequential / nn.Module:backward.  `params` is a list with
    (weight, bias) for conv layers and None otherwise.  Returns the forward
    outputs per layer, gradInput per layer and (gradWeight, gradBias) per conv."""
    import oracle
    outs, saved = [], []
    cur = x
    for l, p in zip(layers, params):
        if l[0] == "conv":
            _, cin, cout, kW, kH, dW, dH, pW, pH = l
            out, finput = oracle.conv_updateOutput(cur, p[0], p[1], kH, kW, pH, pW, dH, dW)
            saved.append((cur, finput))
        elif l[0] == "pool":
            _, kW, kH, dW, dH = l
            out, ind = oracle.maxpool_updateOutput(cur, kH, kW, dH, dW)
            saved.append((cur, ind))
        else:
            out = oracle.threshold_updateOutput(cur, 0.0, 0.0)
            saved.append((cur, None))
        outs.append(out)
        cur = out
    gins = [None] * len(layers)
    grads = [None] * len(layers)
    g = grad_out
    for i in range(len(layers) - 1, -1, -1):
        l, p = layers[i], params[i]
        inp, aux = saved[i]
        if l[0] == "conv":
            _, cin, cout, kW, kH, dW, dH, pW, pH = l
            gi, _ = oracle.conv_updateGradInput(g, p[0], inp.shape, kH, kW, pH, pW, dH, dW)
            gw = np.zeros_like(p[0])
            gb = np.zeros_like(p[1])
            oracle.conv_accGradParameters(g, aux, gw, gb, scale)
            grads[i] = (gw, gb)
        elif l[0] == "pool":
            _, kW, kH, dW, dH = l
            gi = oracle.maxpool_updateGradInput(g, aux, inp.shape, dH, dW)
        else:
            gi = oracle.threshold_updateGradInput(inp, g, 0.0)
        gins[i] = gi
        g = gi
    return outs, gins, grads
