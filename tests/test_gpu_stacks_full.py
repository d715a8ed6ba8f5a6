"""GPU parity at the full benchmark sizes, layer by layer.

Each stack (AlexNet-style b128, OverFeat-fast-style b128, VGG-A-style b64) runs
once through the CPU oracle; then every GPU module is fed the ORACLE's input and
gradOutput of its layer, so a layer's result is compared at the strict bar and
does not inherit the rounding of the layers before it:
  * conv output / gradInput / gradWeight / gradBias within 1e-4*sqrt(reduction
    length) (max error relative to the largest reference magnitude);
  * the im2col buffer (on the gathered route: the zero-padded input), max-pool
    output, argmax-driven gradient and ReLU bit-exact.
Every stack runs on the column route (mode 0) and with the library choosing the
route per layer (mode 1, its initial mode).
The oracle's sgemm runs on the host BLAS here (tests/test_oracle_math.py pins
that path against the reference's plain loops).
"""
import numpy as np
import pytest

from helpers import check_close, oracle_stack, rng_for, uniform

pytestmark = pytest.mark.gpu

import oracle  # noqa: E402


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


_oracle_runs = {}


def oracle_run(stacks, name):
    """Forward + backward of a stack through the oracle, once per stack for the module."""
    if name not in _oracle_runs:
        cfg = stacks.STACKS[name]
        B, layers = cfg["batch"], cfg["layers"]
        net = stacks.build(name, seed_base=4000)
        params = [(np.array(m.weight), np.array(m.bias)) if hasattr(m, "weight") else None for m in net.modules]
        x = stacks.make_input(name, B, seed=4000)
        go = uniform(rng_for(4003), stacks.output_shape(name, B))
        oracle.use_blas(True)
        try:
            outs, gins, grads = oracle_stack(layers, params, x, go)
        finally:
            oracle.use_blas(False)
        _oracle_runs[name] = (x, go, outs, gins, grads)
    return _oracle_runs[name]


@pytest.mark.parametrize("mode", [0, 1], ids=["columns", "auto"])
@pytest.mark.parametrize("name", ["alexnet", "overfeat", "vgg_a"])
def test_full_size_stack_layerwise(gt, name, mode):
    stacks = gt.stacks
    cfg = stacks.STACKS[name]
    B, layers = cfg["batch"], cfg["layers"]
    x, go, outs, gins, grads = oracle_run(stacks, name)
    net = stacks.build(name, seed_base=4000)
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(mode) == 0
    try:
        check_layers(gt, name, net, layers, B, x, go, outs, gins, grads, mode)
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0


def check_layers(gt, name, net, layers, B, x, go, outs, gins, grads, mode):
    net.gpu()
    ins = [x] + outs[:-1]
    gouts = gins[1:] + [go]
    for i, (l, m) in enumerate(zip(layers, net.modules)):
        print("%s layer %d %s in %s" % (name, i, l, ins[i].shape), flush=True)
        dx, dgo = dev(gt, ins[i]), dev(gt, gouts[i])
        m.zeroGradParameters()
        out = m.forward(dx).float()
        gi = m.backward(dx, dgo).float()
        if l[0] == "conv":
            _, cin, cout, kW, kH, dW, dH, pW, pH = l
            K = cin * kH * kW
            N = outs[i].shape[2] * outs[i].shape[3]
            tag = "%s b%d mode%d layer%d " % (name, B, mode, i)
            check_close(tag + "output", out, outs[i], K)
            gathered = m.finput.dim() == 4   # [B, C, H+2pH, W+2pW] instead of [B, K, N]
            # the gathered gradInput product sums over (plane, tap) at once, the column route over planes
            check_close(tag + "gradInput", gi, gins[i], cout if mode == 0 else cout * kH * kW)
            check_close(tag + "gradWeight", m.gradWeight.float(), grads[i][0], B * N)
            check_close(tag + "gradBias", m.gradBias.float(), grads[i][1], B * N)
            if m.finput.nElement() == 0:
                assert (pH, pW) == (0, 0) and mode != 0, (name, i)   # a dense unpadded input is gathered in place: no copy
            elif gathered:
                ref_pad = np.pad(ins[i], [(0, 0), (0, 0), (pH, pH), (pW, pW)])
                assert np.array_equal(bits(m.finput.float()), bits(ref_pad)), (name, i)
            elif B * K * N * 4 <= (1 << 30):  # the column buffer, where the copy back stays modest
                ref_cols = oracle.im2col(ins[i], kH, kW, pH, pW, dH, dW)
                assert np.array_equal(bits(m.finput.float()), bits(ref_cols)), (name, i)
        else:
            assert np.array_equal(bits(out), bits(outs[i])), (name, i)
            assert np.array_equal(bits(gi), bits(gins[i])), (name, i)
            if l[0] == "pool":
                _, ind_ref = oracle.maxpool_updateOutput(ins[i], l[2], l[1], l[4], l[3])
                assert np.array_equal(bits(m.indices.float()), bits(ind_ref)), (name, i)
        del dx, dgo, out, gi


def test_full_size_alexnet_fused_layerwise(gt):
    """The benchmark's configuration -- the AlexNet-style stack at batch 128 after Sequential.fuse(), route chosen per
    layer -- against the oracle, layer by layer on the oracle's inputs: a convolution's output is compared after the
    ReLU it applies itself, a layer behind a ReLU returns the gradient already masked with it.  (Modules called one by
    one take dense tensors; the padded buffers and delivered gradients that the container adds when it runs the whole
    stack are held to bit-identity with the unfused stack at the same size in tests/test_gpu_fusion.py.)"""
    stacks = gt.stacks
    name = "alexnet"
    cfg = stacks.STACKS[name]
    B, layers = cfg["batch"], cfg["layers"]
    x, go, outs, gins, grads = oracle_run(stacks, name)
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(1) == 0
    try:
        net = stacks.build(name, seed_base=4000).gpu().fuse()
        ins = [x] + outs[:-1]
        gouts = gins[1:] + [go]
        n = len(layers)
        for i, (l, m) in enumerate(zip(layers, net.modules)):
            if l[0] == "relu":
                assert m.fusedForward and (m.fusedBackward or i == n - 1 or layers[i + 1][0] == "relu"), i
                continue
            print("alexnet fused layer %d %s" % (i, l), flush=True)
            relu_behind = i + 1 < n and layers[i + 1][0] == "relu" and l[0] == "conv"
            relu_front = i > 0 and layers[i - 1][0] == "relu"
            dx = dev(gt, ins[i])
            # the gradient that reaches this module is the same as in the unfused stack: where a ReLU follows, its
            # backward has been applied by the module behind it
            dgo = dev(gt, gouts[i])
            want_out = outs[i + 1] if relu_behind else outs[i]
            want_gi = gins[i - 1] if relu_front else gins[i]   # masked with the ReLU in front
            m.zeroGradParameters()
            out = m.forward(dx).float()
            gi = m.backward(dx, dgo).float()
            if l[0] == "conv":
                assert (m.fusedThreshold is not None) == relu_behind and (m.inputThreshold is not None) == relu_front, i
                _, cin, cout, kW, kH, dW, dH, pW, pH = l
                K, N = cin * kH * kW, outs[i].shape[2] * outs[i].shape[3]
                tag = "alexnet b%d fused layer%d " % (B, i)
                check_close(tag + "output", out, want_out, K)
                assert np.array_equal(out == 0, want_out == 0) or not relu_behind or \
                    np.mean((out == 0) != (want_out == 0)) < 1e-4          # the threshold bites in the same places
                check_close(tag + "gradInput", gi, want_gi, cout * kH * kW)
                check_close(tag + "gradWeight", m.gradWeight.float(), grads[i][0], B * N)
                check_close(tag + "gradBias", m.gradBias.float(), grads[i][1], B * N)
            else:
                assert (m.inputThreshold is not None) == relu_front, i
                assert np.array_equal(bits(out), bits(want_out)), i
                assert np.array_equal(bits(gi), bits(want_gi)), i
            del dx, dgo, out, gi
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0
