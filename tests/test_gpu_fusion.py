"""nn.Threshold / nn.ReLU fused into the neighbouring modules (Sequential.fuse()): the convolution in front applies
the threshold as it stores its output, the convolution or max-pooling layer behind zeroes its gradInput where the
Threshold's output is not above the threshold.  The bar is bit-identity with the unfused modules (a threshold is a
select, not arithmetic), on both convolution routes and with every kernel that carries the fused store forced."""
import numpy as np
import pytest

from helpers import rng_for, uniform

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def build(gt, spec, seed):
    nn = gt.nn
    rng = rng_for(seed)
    net = nn.Sequential()
    for l in spec:
        if l[0] == "conv":
            _, cin, cout, k, s, p = l
            net.add(nn.SpatialConvolutionMM(cin, cout, k, k, s, s, p, rng=rng))
        elif l[0] == "pool":
            net.add(nn.SpatialMaxPooling(l[1], l[1], l[2], l[2]))
        elif l[0] == "relu":
            net.add(nn.ReLU())
        else:
            net.add(nn.Threshold(l[1], l[2]))
    return net


def run(gt, spec, x, seed, fused, go=None):
    net = build(gt, spec, seed).gpu()
    if fused:
        net.fuse()
    net.zeroGradParameters()
    dx = dev(gt, x)
    out = net.forward(dx).float()
    if go is None:
        go = uniform(rng_for(seed + 1), out.shape)
    gi = net.backward(dx, dev(gt, go)).float()
    outs = [m.output.float() for m in net.modules]
    grads = [(m.gradWeight.float(), m.gradBias.float()) for m in net.modules if hasattr(m, "gradWeight")]
    return net, out, gi, outs, grads, go


SPEC = [("conv", 3, 64, 5, 2, 2), ("relu",), ("pool", 3, 2), ("conv", 64, 96, 3, 1, 1), ("relu",),
        ("conv", 96, 64, 3, 1, 1), ("thr", 0.25, -3.0), ("pool", 2, 2), ("conv", 64, 70, 5, 1, 2), ("relu",)]


@pytest.mark.parametrize("mode", [0, 2], ids=["columns", "gathered"])
def test_fused_stack_is_bit_identical_to_unfused(gt, mode):
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(mode) == 0
    try:
        x = uniform(rng_for(90), (3, 3, 45, 41))
        net_u, out_u, gi_u, outs_u, grads_u, go = run(gt, SPEC, x, 91, False)
        net_f, out_f, gi_f, outs_f, grads_f, _ = run(gt, SPEC, x, 91, True, go)
        thr = [m for m in net_f.modules if isinstance(m, gt.nn.Threshold)]
        assert [t.fusedForward for t in thr] == [True] * 4
        assert [t.fusedBackward for t in thr] == [True, True, True, False]      # the last one has nothing behind it
        assert np.array_equal(bits(out_u), bits(out_f))
        assert np.array_equal(bits(gi_u), bits(gi_f))
        for i, l in enumerate(SPEC):
            if l[0] in ("relu", "thr", "pool"):
                assert np.array_equal(bits(outs_u[i]), bits(outs_f[i])), i
            if l[0] in ("relu", "thr"):         # the fused convolution's output is the thresholded one
                assert np.array_equal(bits(outs_f[i - 1]), bits(outs_u[i])), i
        for (gw_u, gb_u), (gw_f, gb_f) in zip(grads_u, grads_f):
            assert np.array_equal(bits(gw_u), bits(gw_f)) and np.array_equal(bits(gb_u), bits(gb_f))
        assert (out_u == 0).mean() > 0.2                # the threshold did bite
        # in gathered mode the layers in front of a padded convolution wrote that convolution's padded image themselves
        marks = [getattr(m.output, "_zero_border", None) for m in net_f.modules]
        if mode == 2:
            assert marks[2] == (1, 1) and marks[3] == (1, 1) and marks[7] == (2, 2), marks   # pool1, conv2 (+ReLU), pool2
            assert marks[4] is marks[3] or marks[4] == (1, 1)                                 # the fused ReLU passes it on
            buf = net_f.modules[2].output._padded_buffer.float()
            assert not buf[:, :, 0, :].any() and not buf[:, :, -1, :].any() and not buf[:, :, :, 0].any() \
                and not buf[:, :, :, -1].any()                                                # the border is still zero
            assert np.array_equal(bits(buf[:, :, 1:-1, 1:-1]), bits(outs_u[2]))
        else:
            assert marks == [None] * len(marks)
        # unfuse() restores the separate passes
        net_f.unfuse()
        assert not any(t.fusedForward or t.fusedBackward for t in thr)
        dx = dev(gt, x)
        net_f.forward(dx)
        assert np.array_equal(bits(net_f.modules[0].output.float()), bits(outs_u[0]))
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0


def test_threshold_with_value_above_threshold_is_not_fused(gt):
    nn = gt.nn
    net = nn.Sequential().add(nn.SpatialConvolutionMM(3, 4, 3, 3)).add(nn.Threshold(0.1, 0.5)) \
        .add(nn.SpatialMaxPooling(2, 2)).fuse()
    t = net.get(1)
    assert not t.fusedForward and not t.fusedBackward
    assert net.get(0).fusedThreshold is None and net.get(2).inputThreshold is None


CASES = [
    # what is forced                    conv spec behind the ReLU                 mode
    ({"col2im_generic": "1"}, ("conv", 8, 16, 3, 1, 1), 0),
    ({}, ("conv", 8, 16, 3, 1, 1), 0),                       # col2im_unit_kernel<3,3>
    ({}, ("conv", 8, 16, 5, 1, 2), 0),                       # col2im_unit_kernel<5,5>
    ({}, ("conv", 8, 16, 7, 3, 2), 0),                       # col2im_strided_kernel (W >= 64 below)
    ({}, ("conv", 8, 16, 4, 2, 1), 0),
    ({}, ("conv", 64, 64, 3, 1, 1), 2),                      # gathered gradInput: tiled GEMM epilogue
    ({"gemm_split": "3"}, ("conv", 64, 64, 3, 1, 1), 2),     # ... through the split reduction's final pass
    ({"gemm_tile": "64x64"}, ("conv", 64, 128, 3, 1, 1), 2),
    ({"gemm_tile": "128x128", "gemm_split": "2"}, ("conv", 128, 128, 3, 1, 1), 2),
    ({}, ("conv", 16, 64, 7, 3, 2), 2),                      # strided gathered gradInput: the scattered store
    ({"gemm_tile": "64x64"}, ("conv", 8, 64, 4, 2, 1), 2),   # ... with its rows padded to a tile
    ({"gemm_tile": "96x128"}, ("conv", 96, 100, 3, 1, 1), 2),  # the 96-row tile: thresholded output, masked gradInput
    ({"gemm_tile": "48x128"}, ("conv", 12, 64, 4, 2, 1), 2),   # the short-row kernel's masked scattered store
]


@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_every_kernel_that_stores_a_masked_gradient_or_a_thresholded_output(gt, case, switches):
    forced, conv, mode = case
    for k, v in forced.items():
        switches(k, v)
    cin = conv[1]
    spec = [("conv", 3, cin, 3, 1, 1), ("relu",), conv, ("relu",)]
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(mode) == 0
    try:
        x = uniform(rng_for(92), (2, 3, 20, 70))
        _, out_u, gi_u, outs_u, grads_u, go = run(gt, spec, x, 93, False)
        _, out_f, gi_f, outs_f, grads_f, _ = run(gt, spec, x, 93, True, go)
        assert np.array_equal(bits(out_u), bits(out_f)) and np.array_equal(bits(gi_u), bits(gi_f))
        for (gw_u, gb_u), (gw_f, gb_f) in zip(grads_u, grads_f):
            assert np.array_equal(bits(gw_u), bits(gw_f)) and np.array_equal(bits(gb_u), bits(gb_f))
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0


@pytest.mark.parametrize("kernel", ["auto", "tile", "direct", "cell", "staged", "staged_small_share"])
@pytest.mark.parametrize("pool", [(3, 2), (2, 2), (3, 1)])
def test_masked_pooling_backward(gt, pool, kernel, switches):
    switches("pool_bwd_direct", "1" if kernel == "direct" else None)
    switches("pool_bwd_tile", "1" if kernel == "tile" else None)
    switches("pool_bwd_cell", "1" if kernel == "cell" else None)
    switches("pool_bwd_pixels", {"staged": "4096", "staged_small_share": "300"}.get(kernel))
    spec = [("conv", 3, 8, 3, 1, 1), ("relu",), ("pool",) + pool]
    x = uniform(rng_for(94), (3, 3, 29, 31))
    _, out_u, gi_u, _, grads_u, go = run(gt, spec, x, 95, False)
    _, out_f, gi_f, _, grads_f, _ = run(gt, spec, x, 95, True, go)
    assert np.array_equal(bits(out_u), bits(out_f)) and np.array_equal(bits(gi_u), bits(gi_f))
    assert np.array_equal(bits(grads_u[0][0]), bits(grads_f[0][0]))


def test_full_size_alexnet_fused_equals_unfused(gt):
    """The benchmark runs the fused stack: at its full size (batch 128) every result must equal the unfused stack's,
    which tests/test_gpu_stacks_full.py holds to the oracle layer by layer."""
    stacks = gt.stacks
    name, B = "alexnet", 128
    x = stacks.make_input(name, B, seed=4000)
    go = uniform(rng_for(4003), stacks.output_shape(name, B))
    res = []
    for fused in (False, True):
        net = stacks.build(name, seed_base=4000).gpu()
        if fused:
            net.fuse()
        net.zeroGradParameters()
        dx = dev(gt, x)
        out = net.forward(dx).float()
        gi = net.backward(dx, dev(gt, go)).float()
        res.append((out, gi, [(m.gradWeight.float(), m.gradBias.float()) for m in net.modules if hasattr(m, "gradWeight")]))
        del net, dx
    (out_u, gi_u, gr_u), (out_f, gi_f, gr_f) = res
    assert np.array_equal(bits(out_u), bits(out_f)) and np.array_equal(bits(gi_u), bits(gi_f))
    for (gw_u, gb_u), (gw_f, gb_f) in zip(gr_u, gr_f):
        assert np.array_equal(bits(gw_u), bits(gw_f)) and np.array_equal(bits(gb_u), bits(gb_f))


def test_padded_buffer_claims_are_checked_and_a_column_route_producer_can_feed_a_gathering_consumer(gt):
    lib, L = gt._lib.lib, gt._lib
    nn = gt.nn
    # the flag is refused for a tensor that does not lie in a buffer of the claimed geometry
    conv = nn.SpatialConvolutionMM(64, 64, 3, 3, 1, 1, 1).gpu()
    x = dev(gt, uniform(rng_for(96), (2, 64, 9, 9)))
    rc = lib.thgpu_SpatialConvolutionMM_updateOutputFused(x._p, conv.weight._p, conv.bias._p, conv.finput._p,
                                                          conv.fgradInput._p, conv.output._p, 3, 3, 1, 1, 1, 1, 2, 0.0, 0.0)
    assert rc != 0 and b"not the interior" in lib.thgpu_last_error()
    assert lib.thgpu_SpatialConvolutionMM_updateOutputFused(x._p, conv.weight._p, conv.bias._p, conv.finput._p,
                                                            conv.fgradInput._p, conv.output._p, 3, 3, 1, 1, 1, 1, 8, 0.0, 0.0) != 0
    assert lib.thgpu_conv_gathers(2, 64, 9, 9, 64, 3, 3, 1, 1, 1, 1) == (1 if lib.thgpu_conv_get_mode() != 0 else 0)
    assert lib.thgpu_conv_gathers(2, 1, 9, 9, 64, 3, 3, 1, 1, 1, 1) == 0      # K = 9: below the shortest reduction
    # mode 1: a producer whose products no tiled kernel takes (K = 9) stays on columns, its 64-plane consumer gathers
    # from the producer's padded output
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(1) == 0
    try:
        spec = [("conv", 1, 64, 3, 1, 1), ("relu",), ("conv", 64, 64, 3, 1, 1), ("relu",), ("pool", 2, 2)]
        xx = uniform(rng_for(97), (2, 1, 12, 14))
        net_u, out_u, gi_u, outs_u, grads_u, go = run(gt, spec, xx, 98, False)
        net_f, out_f, gi_f, outs_f, grads_f, _ = run(gt, spec, xx, 98, True, go)
        assert net_f.modules[0].finput.dim() == 3 and net_f.modules[0].output._zero_border == (1, 1)
        assert net_f.modules[2].finput.nElement() == 0               # nothing copied
        assert np.array_equal(bits(out_u), bits(out_f)) and np.array_equal(bits(gi_u), bits(gi_f))
        for (gw_u, gb_u), (gw_f, gb_f) in zip(grads_u, grads_f):
            assert np.array_equal(bits(gw_u), bits(gw_f)) and np.array_equal(bits(gb_u), bits(gb_f))
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0


# ---- gradients delivered in the padded layout of the next gathered gradInput product ("twin") ----------------------
def kernel_labels(gt, fn):
    """Runs fn with per-kernel timing on; returns {label: launches}."""
    gp = gt.gputorch
    gp.synchronize()
    gp.prof_reset()
    gp.prof_enable(True)
    try:
        fn()
        gp.synchronize()
        return {k: v["calls"] for k, v in gp.prof_report().items()}
    finally:
        gp.prof_enable(False)
        gp.prof_reset()


TWIN_SPEC = [("conv", 3, 64, 5, 2, 2), ("relu",), ("pool", 3, 2), ("conv", 64, 128, 3, 1, 1), ("relu",),
             ("conv", 128, 64, 3, 1, 1), ("relu",), ("pool", 2, 2), ("conv", 64, 64, 5, 1, 2), ("relu",), ("pool", 3, 2)]


@pytest.mark.parametrize("forced", [{}, {"gemm_split": "3"}, {"gemm_split": "1"}, {"pool_bwd_tile": "1"},
                                    {"pool_bwd_cell": "1"}, {"pool_bwd_pixels": "4096"}, {"pool_bwd_pixels": "500"}],
                         ids=["auto", "split", "unsplit", "pool_tile", "pool_cell", "pool_staged", "pool_staged_strips"])
def test_gradients_written_into_the_next_products_padded_buffer(gt, forced, switches):
    """In a fused Sequential on the gathered route every producer of a convolution's gradOutput (max-pooling backward,
    a unit-stride convolution's gradInput product through its epilogue or its split reduction) also stores it in that
    convolution's zero-bordered buffer: results stay bit-identical to the unfused stack, and the padding launches of
    those layers disappear from the backward pass.  A producer whose kernel keeps no second copy (the LDS tile pooling
    kernel) leaves the padded copy to be made as before."""
    for k, v in forced.items():
        switches(k, v)
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(2) == 0
    try:
        x = uniform(rng_for(190), (4, 3, 61, 57))
        net_u, out_u, gi_u, outs_u, grads_u, go = run(gt, TWIN_SPEC, x, 191, False)
        net_f = build(gt, TWIN_SPEC, 191).gpu().fuse()
        dx, dgo = dev(gt, x), dev(gt, go)
        for step in range(3):                         # the buffers and their zero borders are reused step after step
            net_f.zeroGradParameters()
            out_f = net_f.forward(dx).float()
            labels = kernel_labels(gt, lambda: net_f.backward(dx, dgo))
            gi_f = net_f.gradInput.float()
            assert np.array_equal(bits(out_u), bits(out_f)) and np.array_equal(bits(gi_u), bits(gi_f)), step
            grads_f = [(m.gradWeight.float(), m.gradBias.float()) for m in net_f.modules if hasattr(m, "gradWeight")]
            for (gw_u, gb_u), (gw_f, gb_f) in zip(grads_u, grads_f):
                assert np.array_equal(bits(gw_u), bits(gw_f)) and np.array_equal(bits(gb_u), bits(gb_f)), step
            pads = sum(n for k, n in labels.items() if k.startswith("pad_planes"))
            reorders = labels.get("kernel_bank_reorder", 0)
            # backward of four convolutions: their gradOutput arrives from the last pooling layer (conv4), the second
            # (conv3), conv3's gradInput product (conv2: through its epilogue or split reduction) and the first
            # pooling layer (conv1: the strided layer's own layout)
            # The kernel bank of the receiving layer is re-ordered by workgroups that ride in the delivering launch
            # (pooling kernel, split reduction); only an unsplit product, which delivers from its own epilogue, leaves
            # that to a small launch of the receiver's.
            split3 = any("gemm_conv_gradinput M=128" in k and "split=1" not in k for k in labels)
            if "pool_bwd_tile" in forced:
                assert pads == 3 + 1 and reorders == (0 if split3 else 1), labels   # only conv3's product delivers
            else:
                assert pads == 1 and reorders == (0 if split3 else 1), labels   # left: conv1's accGradParameters input
            if "gemm_split" in forced:
                assert split3 == (forced["gemm_split"] != "1"), labels
        # a module called on its own takes the ordinary route and gives the same result
        conv3 = net_f.get(5)
        labels = kernel_labels(gt, lambda: conv3.updateGradInput(net_f.get(4).output, net_f.get(7).gradInput))
        assert any(k.startswith("pad_planes") for k in labels), labels
        ref3 = net_u.get(4).gradInput.float()          # (the fused layer's gradInput carries the ReLU's mask)
        assert np.array_equal(bits(conv3.gradInput.float()), bits(ref3))
        # and the fused pass still works afterwards (the padded copy just made keeps the borders zero)
        net_f.zeroGradParameters()
        net_f.forward(dx)
        assert np.array_equal(bits(net_f.backward(dx, dgo).float()), bits(gi_u))
        # another batch size: new buffers, new borders
        x2 = uniform(rng_for(192), (2, 3, 61, 57))
        net_u2, out_u2, gi_u2, _, grads_u2, go2 = run(gt, TWIN_SPEC, x2, 191, False)
        net_f.zeroGradParameters()
        assert np.array_equal(bits(net_f.forward(dev(gt, x2)).float()), bits(out_u2))
        assert np.array_equal(bits(net_f.backward(dev(gt, x2), dev(gt, go2)).float()), bits(gi_u2))
        # unfuse(): no deliveries any more
        net_f.unfuse()
        net_f.zeroGradParameters()
        net_f.forward(dx)
        labels = kernel_labels(gt, lambda: net_f.backward(dx, dgo))
        assert labels.get("kernel_bank_reorder", 0) == 0 and np.array_equal(bits(net_f.gradInput.float()), bits(gi_u))
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0


def test_twin_view_is_refused_when_the_buffer_is_not_the_prepared_one(gt):
    """THGPU_GRADOUTPUT_IN_TWIN is only honoured for the buffer thgpu_SpatialConvolutionMM_gradOutputTwin prepared:
    handed a layer whose fgradInput was never prepared (or has been resized since), the entry point makes the padded copy
    itself and the result is right."""
    import ctypes
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(2) == 0
    try:
        rng = rng_for(195)
        conv = gt.nn.SpatialConvolutionMM(64, 64, 3, 3, 1, 1, 1, rng=rng).gpu()
        x, go = uniform(rng, (2, 64, 12, 10)), uniform(rng, (2, 64, 12, 10))
        dx, dgo = dev(gt, x), dev(gt, go)
        conv.forward(dx)
        ref = conv.updateGradInput(dx, dgo).float().copy()
        fresh = gt.nn.SpatialConvolutionMM(64, 64, 3, 3, 1, 1, 1, rng=rng).gpu()
        fresh.weight.copy(conv.weight)
        fresh.forward(dx)
        wrote = ctypes.c_int(7)
        labels = kernel_labels(gt, lambda: gt._lib.check_status(lib.thgpu_SpatialConvolutionMM_updateGradInputTwin(
            dx._p, dgo._p, fresh.weight._p, fresh.finput._p, fresh.fgradInput._p, fresh.gradInput._p,
            3, 3, 1, 1, 1, 1, 8, 0.0, None, ctypes.byref(wrote))))
        assert wrote.value == 0 and any(k.startswith("pad_planes") for k in labels), labels
        assert np.array_equal(bits(fresh.gradInput.float()), bits(ref))
        # the view: sizes of gradOutput, rows inside planes of (H + 2) x (W + 2), borders zero after preparation
        twin = fresh._gradOutputTwin(dx)
        assert twin is not None and tuple(twin.size()) == (2, 64, 12, 10) and tuple(twin.stride()) == (64 * 14 * 12, 14 * 12, 12, 1)
        # on the column route no view is handed out
        assert lib.thgpu_conv_set_mode(0) == 0
        assert fresh._gradOutputTwin(dx) is None
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0
