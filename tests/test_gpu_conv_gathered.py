"""GPU parity tests of nn.SpatialConvolutionMM in mode 1 (no column buffer: the GEMMs gather their second
operand from a zero-padded copy of the image), through the C ABI, against the CPU oracle's
im2col + sgemm + col2im on identical seeded inputs.

Bars: fp32 outputs and gradients within a norm-wise relative error of 1e-4*sqrt(reduction length); the
padded input kept in finput bit-exact; repeated runs bit-identical.
"""
import numpy as np
import pytest

from helpers import check_close, gemm_tol, oracle_stack, rel_err, both_rel_err, rng_for, uniform

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


def run_conv(gt, x, w, b, go, geo, scale=1.0, gw0=None, gb0=None, forward_first=True):
    kH, kW, pH, pW, sH, sW = geo
    M = w.shape[0]
    C = x.shape[-3]
    m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m._assign("bias", b)
    m.gradWeight[...] = 0 if gw0 is None else gw0
    m.gradBias[...] = 0 if gb0 is None else gb0
    m.gpu()
    dx, dgo = dev(gt, x), dev(gt, go)
    out = m.forward(dx).float() if forward_first else None
    finput = m.finput.float()
    gi = m.updateGradInput(dx, dgo).float()
    m.accGradParameters(dx, dgo, scale)
    return dict(output=out, finput=finput, finput_after=m.finput.float(), gradInput=gi,
                gradWeight=m.gradWeight.float(), gradBias=m.gradBias.float())


def padded(x, pH, pW):
    return np.pad(x, [(0, 0)] * (x.ndim - 2) + [(pH, pH), (pW, pW)])


def reference(x, w, b, go_shape_rng, geo, scale, gw0, gb0):
    out_ref, finput_ref = oracle.conv_updateOutput(x, w, b, *geo)
    go = uniform(go_shape_rng, out_ref.shape)
    gi_ref, _ = oracle.conv_updateGradInput(go, w, x.shape, *geo)
    gw_ref, gb_ref = gw0.copy(), gb0.copy()
    oracle.conv_accGradParameters(go, finput_ref, gw_ref, gb_ref, scale)
    return out_ref, go, gi_ref, gw_ref, gb_ref


GATHERED = [
    # B, C, H, W, M, kH, kW, pH, pW, sH, sW            forward/gradWeight gathered, gradInput gathered
    (2, 64, 9, 9, 64, 3, 3, 1, 1, 1, 1),               # yes, yes
    (3, 70, 12, 10, 80, 3, 3, 1, 1, 2, 2),             # yes, no (stride 2)
    (2, 64, 8, 8, 64, 5, 5, 2, 2, 1, 1),               # yes, yes
    (1, 64, 16, 16, 96, 3, 3, 0, 0, 1, 1),             # no padding
    (4, 64, 27, 27, 192, 5, 5, 2, 2, 1, 1),            # AlexNet conv2 shape
    (1, 384, 13, 13, 256, 3, 3, 1, 1, 1, 1),           # batch 1
    (2, 64, 20, 17, 128, 7, 3, 3, 1, 1, 1),            # anisotropic kernel and padding
    (3, 66, 11, 13, 72, 3, 5, 2, 0, 1, 1),             # padding kH-1 in one direction, none in the other
    (2, 64, 10, 10, 64, 3, 3, 3, 3, 1, 1),             # padding above kH-1: gradInput takes the column route
    (2, 130, 9, 9, 70, 3, 3, 1, 1, 1, 1),              # nothing a multiple of the tile
    (5, 67, 23, 19, 65, 4, 2, 1, 0, 3, 2),             # even kernels, strides 3 x 2
    (16, 3, 224, 224, 64, 11, 11, 2, 2, 4, 4),         # first benchmark configuration, full size
    (2, 48, 12, 12, 64, 3, 3, 1, 1, 1, 1),             # C < 64: forward gathered, gradInput by columns
    (2, 64, 12, 12, 48, 3, 3, 1, 1, 1, 1),             # M < 64: forward by columns, gradInput gathered
    # fewer than 64 taps: the gradWeight product runs 64 columns wide and stores K of them
    (4, 3, 40, 36, 64, 3, 3, 1, 1, 1, 1),              # VGG-style first layer, K = 27
    (3, 1, 33, 35, 128, 5, 5, 2, 2, 1, 1),             # one input plane, K = 25, two row tiles
    (5, 3, 31, 29, 70, 4, 4, 1, 1, 2, 2),              # K = 48, stride 2, rows ragged against the tile
    (2, 3, 64, 48, 128, 7, 3, 3, 1, 2, 1),             # K = 63: the non-square edge case with three input planes
    (2, 2, 30, 30, 64, 3, 3, 0, 0, 1, 1),              # K = 18, unpadded: gathered from the dense input in place
]


@pytest.mark.parametrize("cfg", GATHERED)
def test_gathered_conv_fwd_bwd_parity(gt, gathered_route, cfg):
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = cfg
    geo = (kH, kW, pH, pW, sH, sW)
    K = C * kH * kW
    rng = rng_for(41)
    s = 1.0 / np.sqrt(K)
    x = uniform(rng, (B, C, H, W))
    w, b = uniform(rng, (M, K), -s, s), uniform(rng, (M,), -s, s)
    gw0, gb0 = uniform(rng, (M, K)), uniform(rng, (M,))
    scale = 0.5
    out_ref, go, gi_ref, gw_ref, gb_ref = reference(x, w, b, rng, geo, scale, gw0, gb0)
    got = run_conv(gt, x, w, b, go, geo, scale, gw0, gb0)
    N = out_ref.shape[2] * out_ref.shape[3]
    if M >= 64 and K >= 16 and (pH, pW) == (0, 0):
        assert got["finput"].size <= 1            # an unpadded dense input is gathered from where it lies: no copy
    elif M >= 64 and K >= 16:
        assert np.array_equal(bits(got["finput"]), bits(padded(x, pH, pW)))   # the padded input, not columns
    else:
        assert got["finput"].shape == (B, K, N)
    tag = "conv b%d %d->%d %dx%d k%dx%d p%dx%d s%dx%d gathered " % (B, C, M, H, W, kH, kW, pH, pW, sH, sW)
    check_close(tag + "output", got["output"], out_ref, K)
    # the gathered gradInput product sums over (output plane, tap) at once: that is its reduction length
    check_close(tag + "gradInput", got["gradInput"], gi_ref, M * kH * kW)
    check_close(tag + "gradWeight", got["gradWeight"], gw_ref, B * N)
    check_close(tag + "gradBias", got["gradBias"], gb_ref, B * N)


def test_gathered_matches_column_route_and_reruns_identically(gt, gathered_route):
    B, C, H, W, M, kH, kW = 3, 64, 14, 15, 96, 3, 5
    geo = (kH, kW, 1, 2, 1, 1)
    rng = rng_for(42)
    x, w, b = uniform(rng, (B, C, H, W)), uniform(rng, (M, C * kH * kW), -0.05, 0.05), uniform(rng, (M,))
    ref, _ = oracle.conv_updateOutput(x, w, b, *geo)
    go = uniform(rng, ref.shape)
    a = run_conv(gt, x, w, b, go, geo)
    a2 = run_conv(gt, x, w, b, go, geo)
    for k in a:
        assert np.array_equal(bits(a[k]), bits(a2[k])), k   # deterministic: no atomics anywhere
    lib = gt._lib.lib
    assert lib.thgpu_conv_set_mode(0) == 0
    try:
        c = run_conv(gt, x, w, b, go, geo)
    finally:
        assert lib.thgpu_conv_set_mode(2) == 0
    assert c["finput"].shape == (B, C * kH * kW, ref.shape[2] * ref.shape[3])
    for k in ("output", "gradInput", "gradWeight", "gradBias"):
        assert rel_err(a[k], c[k]) < 1e-5, k


def test_gathered_non_batch_input(gt, gathered_route):
    C, H, W, M, kH, kW = 64, 12, 11, 64, 3, 3
    geo = (kH, kW, 1, 1, 1, 1)
    rng = rng_for(43)
    x, w, b = uniform(rng, (C, H, W)), uniform(rng, (M, C * kH * kW), -0.05, 0.05), uniform(rng, (M,))
    gw0, gb0 = np.zeros((M, C * kH * kW), np.float32), np.zeros((M,), np.float32)
    out_ref, go, gi_ref, gw_ref, gb_ref = reference(x[None], w, b, rng, geo, 1.0, gw0, gb0)
    got = run_conv(gt, x, w, b, go[0], geo)
    assert got["output"].shape == out_ref.shape[1:] and got["gradInput"].shape == x.shape
    assert got["finput"].shape == (C, H + 2, W + 2)
    assert both_rel_err(got["output"], out_ref[0]) < gemm_tol(C * kH * kW)
    assert both_rel_err(got["gradInput"], gi_ref[0]) < gemm_tol(M * kH * kW)
    assert both_rel_err(got["gradWeight"], gw_ref) < gemm_tol(H * W)


def test_gathered_gradweight_without_forward_rebuilds_the_padded_input(gt, gathered_route):
    B, C, H, W, M, kH, kW = 2, 64, 10, 9, 64, 3, 3
    geo = (kH, kW, 1, 1, 1, 1)
    rng = rng_for(44)
    x, w, b = uniform(rng, (B, C, H, W)), uniform(rng, (M, C * kH * kW), -0.05, 0.05), uniform(rng, (M,))
    gw0, gb0 = uniform(rng, (M, C * kH * kW)), uniform(rng, (M,))
    out_ref, go, gi_ref, gw_ref, gb_ref = reference(x, w, b, rng, geo, 2.0, gw0, gb0)
    got = run_conv(gt, x, w, b, go, geo, 2.0, gw0, gb0, forward_first=False)
    assert got["finput"].shape != (B, C, H + 2, W + 2)   # no forward pass has filled it
    assert np.array_equal(bits(got["finput_after"]), bits(padded(x, 1, 1)))
    assert both_rel_err(got["gradWeight"], gw_ref) < gemm_tol(B * H * W)
    assert both_rel_err(got["gradBias"], gb_ref) < gemm_tol(B * H * W)
    assert both_rel_err(got["gradInput"], gi_ref) < gemm_tol(M * kH * kW)


def random_gathered_geometries(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        kH, kW = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        sH, sW = (1, 1) if rng.random() < 0.6 else (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
        pH, pW = int(rng.integers(0, kH + 1)), int(rng.integers(0, kW + 1))
        C, M = int(rng.integers(64, 150)), int(rng.integers(64, 150))
        H, W = int(rng.integers(6, 20)), int(rng.integers(6, 20))
        B = int(rng.integers(1, 4))
        if H + 2 * pH < kH or W + 2 * pW < kW:
            continue
        Ho, Wo = (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1
        if Ho * Wo < 16 or B * Ho * Wo < 64:
            continue
        out.append((B, C, H, W, M, kH, kW, pH, pW, sH, sW))
    return out


@pytest.mark.parametrize("cfg", random_gathered_geometries(24, 2101))
def test_gathered_conv_random_geometry(gt, gathered_route, cfg):
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = cfg
    geo = (kH, kW, pH, pW, sH, sW)
    K = C * kH * kW
    rng = rng_for(45)
    s = 1.0 / np.sqrt(K)
    x = uniform(rng, (B, C, H, W))
    w, b = uniform(rng, (M, K), -s, s), uniform(rng, (M,), -s, s)
    gw0, gb0 = uniform(rng, (M, K)), uniform(rng, (M,))
    out_ref, go, gi_ref, gw_ref, gb_ref = reference(x, w, b, rng, geo, 1.5, gw0, gb0)
    got = run_conv(gt, x, w, b, go, geo, 1.5, gw0, gb0)
    N = out_ref.shape[2] * out_ref.shape[3]
    if (pH, pW) == (0, 0):
        assert got["finput"].size <= 1            # an unpadded dense input is gathered from where it lies: no copy
    else:
        assert np.array_equal(bits(got["finput"]), bits(padded(x, pH, pW)))
    assert both_rel_err(got["output"], out_ref) < gemm_tol(K)
    assert both_rel_err(got["gradInput"], gi_ref) < gemm_tol(M * kH * kW)
    assert both_rel_err(got["gradWeight"], gw_ref) < gemm_tol(B * N)
    assert both_rel_err(got["gradBias"], gb_ref) < gemm_tol(B * N)


@pytest.mark.parametrize("split", [1, 3])
@pytest.mark.parametrize("tile", ["128x128", "192x128", "64x256", "128x256", "256x128", "64x64", "64x128", "96x128"])
def test_gathered_conv_every_tile_configuration(gt, gathered_route, tile, split, switches):
    """Every tile of the GEMM has its own gathering kernels (plain and reduction-batched); the library's choice
    would leave most of them to the large benchmark shapes, so each is forced here on a shape all of them fit."""
    switches("gemm_tile", tile)
    switches("gemm_split", split)
    B, C, H, W, M, kH, kW = 2, 256, 12, 12, 256, 3, 3
    geo = (kH, kW, 1, 1, 1, 1)
    K = C * kH * kW
    rng = rng_for(48)
    s = 1.0 / np.sqrt(K)
    x = uniform(rng, (B, C, H, W))
    w, b = uniform(rng, (M, K), -s, s), uniform(rng, (M,), -s, s)
    gw0, gb0 = uniform(rng, (M, K)), uniform(rng, (M,))
    out_ref, go, gi_ref, gw_ref, gb_ref = reference(x, w, b, rng, geo, 1.0, gw0, gb0)
    got = run_conv(gt, x, w, b, go, geo, 1.0, gw0, gb0)
    assert got["finput"].shape == (B, C, H + 2, W + 2)
    assert both_rel_err(got["output"], out_ref) < gemm_tol(K)
    assert both_rel_err(got["gradInput"], gi_ref) < gemm_tol(M * kH * kW)
    assert both_rel_err(got["gradWeight"], gw_ref) < gemm_tol(B * H * W)


def test_mode_1_gathers_where_a_tiled_kernel_takes_the_product(gt):
    """The library's own choice: narrow and wide layers alike compute without columns; a layer too small for the
    tiled kernels (fewer than 64 output planes) stays on the column route."""
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(1) == 0
    try:
        rng = rng_for(46)
        for M, gathers in ((128, True), (512, True), (24, False)):
            B, C, H, W, kH, kW = 2, 64, 8, 8, 3, 3
            geo = (kH, kW, 1, 1, 1, 1)
            x, w, b = uniform(rng, (B, C, H, W)), uniform(rng, (M, C * kH * kW), -0.05, 0.05), uniform(rng, (M,))
            gw0, gb0 = np.zeros((M, C * kH * kW), np.float32), np.zeros((M,), np.float32)
            out_ref, go, gi_ref, gw_ref, gb_ref = reference(x, w, b, rng, geo, 1.0, gw0, gb0)
            got = run_conv(gt, x, w, b, go, geo)
            assert got["finput"].shape == ((B, C, H + 2, W + 2) if gathers else (B, C * kH * kW, H * W))
            assert both_rel_err(got["output"], out_ref) < gemm_tol(C * kH * kW)
            assert both_rel_err(got["gradInput"], gi_ref) < gemm_tol(M * kH * kW)
            assert both_rel_err(got["gradWeight"], gw_ref) < gemm_tol(B * H * W)
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0


def test_route_switched_between_forward_and_accgradparameters(gt):
    """2x2 kernels at stride 2 on an even image: the columns have as many elements as the (unpadded) image, so only
    the buffer's shape tells accGradParameters which of the two finput holds."""
    B, C, H, W, M, k = 2, 64, 12, 12, 64, 2
    geo = (k, k, 0, 0, 2, 2)
    rng = rng_for(47)
    x, w, b = uniform(rng, (B, C, H, W)), uniform(rng, (M, C * k * k), -0.05, 0.05), uniform(rng, (M,))
    gw0, gb0 = np.zeros((M, C * k * k), np.float32), np.zeros((M,), np.float32)
    out_ref, go, gi_ref, gw_ref, gb_ref = reference(x, w, b, rng, geo, 1.0, gw0, gb0)
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    try:
        for fwd_mode, acc_mode in ((2, 0), (0, 2)):
            m = gt.nn.SpatialConvolutionMM(C, M, k, k, 2, 2, 0)
            m._assign("weight", w)
            m._assign("bias", b)
            m.gradWeight[...] = 0
            m.gradBias[...] = 0
            m.gpu()
            dx, dgo = dev(gt, x), dev(gt, go)
            assert lib.thgpu_conv_set_mode(fwd_mode) == 0
            out = m.forward(dx).float()
            if fwd_mode == 0:
                assert m.finput.float().size == B * C * H * W
            else:
                assert m.finput.nElement() == 0       # the unpadded dense input is gathered in place
            assert lib.thgpu_conv_set_mode(acc_mode) == 0
            m.accGradParameters(dx, dgo, 1.0)
            assert both_rel_err(out, out_ref) < gemm_tol(C * k * k)
            assert both_rel_err(m.gradWeight.float(), gw_ref) < gemm_tol(B * out_ref.shape[2] * out_ref.shape[3])
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0


def test_offset_table_cache_starts_over_after_many_geometries(gt, gathered_route):
    """The per-geometry offset tables are cached (two per pass); past 512 entries the cache is emptied.  Results
    before, across and after that point must agree with the column route."""
    lib = gt._lib.lib
    B, C, H, M, k = 1, 64, 8, 64, 3
    rng = rng_for(49)
    w, b = uniform(rng, (M, C * k * k), -0.05, 0.05), uniform(rng, (M,))
    m = gt.nn.SpatialConvolutionMM(C, M, k, k, 1, 1, 1)
    m._assign("weight", w)
    m._assign("bias", b)
    m.gpu()
    for W in range(8, 8 + 280):                     # 280 geometries x 2 tables
        x = uniform(rng, (B, C, H, W))
        dx = dev(gt, x)
        out = m.forward(dx).float()
        if W % 40 == 0 or W >= 8 + 254:            # the cache is emptied near the 256th geometry
            assert lib.thgpu_conv_set_mode(0) == 0
            try:
                ref = m.forward(dx).float()
            finally:
                assert lib.thgpu_conv_set_mode(2) == 0
            assert rel_err(out, ref) < 1e-5, W


def test_conv_mode_api(gt):
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert before in (0, 1, 2)
    for bad in (-1, 3):
        assert lib.thgpu_conv_set_mode(bad) != 0 and b"mode" in lib.thgpu_last_error()
        assert lib.thgpu_conv_get_mode() == before
    for mode in (2, 1, 0):
        assert lib.thgpu_conv_set_mode(mode) == 0 and lib.thgpu_conv_get_mode() == mode
    assert lib.thgpu_conv_set_mode(before) == 0


def test_gathered_alexnet_stack_matches_oracle(gt, gathered_route):
    stacks = gt.stacks
    name, B = "alexnet", 2
    layers = stacks.STACKS[name]["layers"]
    net = stacks.build(name, seed_base=2100)
    params = [(np.array(m.weight), np.array(m.bias)) if hasattr(m, "weight") else None for m in net.modules]
    x = stacks.make_input(name, B, seed=2100)
    go = uniform(rng_for(2103), stacks.output_shape(name, B))
    outs, gins, grads = oracle_stack(layers, params, x, go)
    net.gpu()
    dx = dev(gt, x)
    out = net.forward(dx).float()
    gi = net.backward(dx, dev(gt, go)).float()
    assert rel_err(out, outs[-1]) < 1e-3
    assert rel_err(gi, gins[0]) < 5e-3
    for m, g in zip(net.modules, grads):
        if g is not None:
            assert rel_err(m.gradWeight.float(), g[0]) < 5e-3
            assert rel_err(m.gradBias.float(), g[1]) < 5e-3


@pytest.mark.parametrize("mode", [0, 2], ids=["columns", "gathered"])
def test_accgradparameters_depends_on_its_arguments_alone(gt, mode):
    """forward(x1) then accGradParameters(x2): the reference GPU code re-extracts the columns from its `input`
    argument on every call (gpunn-impl/SpatialConvolutionMM.cpp:388-396), so the result is the oracle's for x2, not
    a product with the stale buffer of x1; likewise when two same-shaped modules share finput / fgradInput.  With
    thgpu_conv_set_finput_reuse(1) the buffer is taken on trust, as the CPU module does."""
    lib = gt._lib.lib
    B, C, H, W, M, kH, kW = 3, 64, 11, 12, 80, 3, 3
    geo = (kH, kW, 1, 1, 1, 1)
    rng = rng_for(49)
    x1, x2 = uniform(rng, (B, C, H, W)), uniform(rng, (B, C, H, W))
    w, b = uniform(rng, (M, C * kH * kW), -0.05, 0.05), uniform(rng, (M,))
    out2, cols2 = oracle.conv_updateOutput(x2, w, b, *geo)
    go = uniform(rng, out2.shape)
    gw_ref, gb_ref = np.zeros_like(w), np.zeros_like(b)
    oracle.conv_accGradParameters(go, cols2, gw_ref, gb_ref, 1.0)
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(mode) == 0 and lib.thgpu_conv_get_finput_reuse() == 0
    try:
        def module():
            m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, 1, 1, 1)
            m._assign("weight", w)
            m._assign("bias", b)
            m.gradWeight[...] = 0
            m.gradBias[...] = 0
            return m.gpu()
        m = module()
        d1, d2, dgo = dev(gt, x1), dev(gt, x2), dev(gt, go)
        m.forward(d1)
        m.accGradParameters(d2, dgo, 1.0)
        check_close("accGradParameters on another input than the forward's, mode %d" % mode, m.gradWeight.float(),
                    gw_ref, B * H * W)
        # two modules sharing their buffers, as memory-saving Torch scripts do
        a, c = module(), module()
        c.finput, c.fgradInput = a.finput, a.fgradInput
        a.forward(d2)
        c.forward(d1)                       # overwrites the shared finput with x1's
        a.updateGradInput(d2, dgo)
        a.accGradParameters(d2, dgo, 1.0)
        check_close("accGradParameters with a shared finput, mode %d" % mode, a.gradWeight.float(), gw_ref, B * H * W)
        # opt-in reuse: right after its own forward pass the buffer is the forward's and the result is the same
        assert lib.thgpu_conv_set_finput_reuse(1) == 0
        r = module()
        r.forward(d2)
        r.accGradParameters(d2, dgo, 1.0)
        assert np.array_equal(bits(r.gradWeight.float()), bits(a.gradWeight.float()))
    finally:
        assert lib.thgpu_conv_set_finput_reuse(0) == 0
        assert lib.thgpu_conv_set_mode(before) == 0


STRIDED = [
    # B, C, H, W, M, kH, kW, pH, pW, sH, sW
    (2, 3, 40, 37, 64, 11, 11, 2, 2, 4, 4),     # the first-layer geometry: 48 rows padded to a 64-row tile
    (3, 5, 23, 19, 16, 2, 2, 0, 0, 3, 3),       # kernel smaller than the stride: some pixels receive nothing
    (2, 8, 17, 30, 24, 5, 3, 4, 2, 2, 3),       # padding above the stride, anisotropic everything
    (1, 20, 64, 64, 32, 3, 3, 1, 1, 2, 2),      # 80 rows: an edge tile shifted back
    (2, 70, 12, 10, 80, 3, 3, 1, 1, 2, 1),      # strided along one axis only
    (4, 3, 101, 77, 37, 5, 5, 0, 0, 3, 3),      # odd sizes of the edge sweep
    (32, 64, 128, 96, 128, 7, 3, 3, 1, 2, 1),   # the non-square case of the edge sweep at its stated size
]


@pytest.mark.parametrize("cfg", STRIDED)
def test_strided_gradinput_by_residue_class(gt, gathered_route, cfg):
    """gradInput of a strided layer as one product over the residue classes of the pixel coordinates (scattered
    store, no column buffer), against the oracle's GEMM + col2im; the timing label shows that this product ran:
    its reduction is M*ceil(kH/sH)*ceil(kW/sW) long and it has one column per cell of the strided grid."""
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = cfg
    geo = (kH, kW, pH, pW, sH, sW)
    K = C * kH * kW
    rng = rng_for(51)
    s = 1.0 / np.sqrt(K)
    x = uniform(rng, (B, C, H, W))
    w, b = uniform(rng, (M, K), -s, s), uniform(rng, (M,), -s, s)
    Ho, Wo = (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1
    go = uniform(rng, (B, M, Ho, Wo))
    gi_ref, _ = oracle.conv_updateGradInput(go, w, x.shape, *geo)
    m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m._assign("bias", b)
    m.gpu()
    dx, dgo = dev(gt, x), dev(gt, go)
    gt.gputorch.synchronize()
    gt.gputorch.prof_reset()
    gt.gputorch.prof_enable(True)
    try:
        gi = m.updateGradInput(dx, dgo).float()
        gi2 = m.updateGradInput(dx, dgo).float()
        gt.gputorch.synchronize()
        labels = [k for k in gt.gputorch.prof_report() if k.startswith("gemm_conv_gradinput")]
    finally:
        gt.gputorch.prof_enable(False)
        gt.gputorch.prof_reset()
    A, Bk = -(-kH // sH), -(-kW // sW)
    Yn, Xn = (H - 1 + pH) // sH + 1, (W - 1 + pW) // sW + 1
    assert len(labels) == 1 and " J=%d R=%d " % (B * Yn * Xn, M * A * Bk) in labels[0], labels
    assert np.array_equal(bits(gi), bits(gi2))
    check_close("conv b%d %d->%d %dx%d k%dx%d p%dx%d s%dx%d gradInput by residue class" %
                (B, C, M, H, W, kH, kW, pH, pW, sH, sW), gi, gi_ref, M * kH * kW)


def test_strided_gradinput_integer_exact_and_untouched_neighbours(gt, gathered_route):
    """Small integers make every sum exact: the scattered store must then reproduce the oracle bit for bit, and it
    must write nothing outside gradInput (checked with a guard band around a view of a larger buffer)."""
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = 3, 6, 21, 26, 40, 5, 4, 2, 1, 3, 2
    geo = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(52)
    ints = lambda lo, hi, shape: rng.integers(lo, hi + 1, size=shape).astype(np.float32)
    x, w = ints(-2, 2, (B, C, H, W)), ints(-2, 2, (M, C * kH * kW))
    Ho, Wo = (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1
    go = ints(-2, 2, (B, M, Ho, Wo))
    gi_ref, _ = oracle.conv_updateGradInput(go, w, x.shape, *geo)
    m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m.gpu()
    n = B * C * H * W
    guard = 4096
    big = dev(gt, np.full(n + 2 * guard, 7.5, np.float32))
    m.gradInput = big.narrow(0, guard, n).view(B, C, H, W)
    gi = m.updateGradInput(dev(gt, x), dev(gt, go)).float()
    assert np.array_equal(gi, gi_ref)
    host = big.float()
    assert np.all(host[:guard] == 7.5) and np.all(host[guard + n:] == 7.5)
    assert np.array_equal(host[guard:guard + n].reshape(B, C, H, W), gi_ref)


SHORT_ROWS = [
    # B, C, H, W, kH, kW, pH, pW, sH, sW: C*sH*sW <= 48 rows in use of the product's single 64-row tile
    (3, 3, 45, 38, 11, 11, 2, 2, 4, 4),    # 48 rows: the first-layer geometry
    (3, 12, 21, 30, 3, 5, 1, 2, 2, 2),     # 48 rows from twelve planes
    (3, 2, 50, 41, 7, 6, 3, 0, 5, 4),      # 40 rows, strides that differ
    (2, 11, 33, 35, 4, 4, 1, 1, 3, 1),     # 33 rows: one row of the third block of sixteen
    (4, 1, 64, 49, 9, 9, 4, 4, 4, 4),      # 16 rows
]


@pytest.mark.parametrize("tile", ["48x128", "48x256"])
@pytest.mark.parametrize("masked", [False, True])
@pytest.mark.parametrize("cfg", SHORT_ROWS)
def test_strided_gradinput_short_row_kernel_integer_exact(gt, gathered_route, switches, cfg, masked, tile):
    """The scattered product whose rows fit 48 of its 64-row tile runs on the kernel that multiplies 48 rows in
    16x16 blocks.  Small integers make every sum exact, so the result must equal the oracle's bit for bit, with and
    without the fused nn.Threshold mask, and nothing outside gradInput may be written."""
    B, C, H, W, kH, kW, pH, pW, sH, sW = cfg
    M = 24
    geo = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(53)
    ints = lambda lo, hi, shape: rng.integers(lo, hi + 1, size=shape).astype(np.float32)
    x, w = ints(-2, 2, (B, C, H, W)), ints(-2, 2, (M, C * kH * kW))
    Ho, Wo = (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1
    go = ints(-2, 2, (B, M, Ho, Wo))
    gi_ref, _ = oracle.conv_updateGradInput(go, w, x.shape, *geo)
    if masked:
        gi_ref = np.where(x > 0.0, gi_ref, np.float32(0.0))
    m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m.gpu()
    n = B * C * H * W
    guard = 4096
    big = dev(gt, np.full(n + 2 * guard, 7.5, np.float32))
    m.gradInput = big.narrow(0, guard, n).view(B, C, H, W)
    switches("gemm_tile", tile)
    dx, dgo = dev(gt, x), dev(gt, go)
    gt.gputorch.synchronize()
    gt.gputorch.prof_reset()
    gt.gputorch.prof_enable(True)
    try:
        if masked:
            m.inputThreshold = 0.0  # what Sequential.fuse() sets on a convolution that follows an nn.Threshold
        gi = m.updateGradInput(dx, dgo).float()
        gt.gputorch.synchronize()
        labels = [k for k in gt.gputorch.prof_report() if k.startswith("gemm_conv_gradinput")]
    finally:
        gt.gputorch.prof_enable(False)
        gt.gputorch.prof_reset()
    assert len(labels) == 1 and "tile=%s " % tile in labels[0], labels
    assert np.array_equal(gi, gi_ref)
    host = big.float()
    assert np.all(host[:guard] == 7.5) and np.all(host[guard + n:] == 7.5)


@pytest.mark.parametrize("split", [None, 2, 7])
@pytest.mark.parametrize("cfg", [(4, 3, 40, 36, 64, 3, 3, 1, 1, 1, 1), (3, 1, 33, 35, 128, 5, 5, 2, 2, 1, 1),
                                 (5, 3, 31, 29, 70, 4, 4, 1, 1, 2, 2), (2, 3, 64, 48, 128, 7, 3, 3, 1, 2, 1),
                                 (1, 3, 40, 36, 64, 3, 3, 1, 1, 1, 1)])     # (the last: one image, no batched reduction)
def test_narrow_gradweight_runs_wide_and_stores_its_own_columns_integer_exact(gt, gathered_route, switches, cfg, split):
    """A layer with fewer than 64 taps (K = C*kH*kW: a first layer with 3x3 or 5x5 kernels) has a gradWeight product
    narrower than the narrowest GEMM tile.  It runs 64 columns wide on a padded tap table and the split reduction's
    final pass stores the first K columns only: on integer data every result equals the oracle's bit for bit, gradBias
    (summed on the side by the same product) included, and what lies around gradWeight in memory is untouched."""
    switches("conv_narrow_off", "1")      # (this test is about the tiled product; conv_narrow.hip has its own below)
    if split is not None:
        switches("gemm_split", split)
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = cfg
    geo = (kH, kW, pH, pW, sH, sW)
    K = C * kH * kW
    rng = rng_for(48)
    ints = lambda shape: rng.integers(-3, 4, shape).astype(np.float32)  # noqa: E731
    x, w, b = ints((B, C, H, W)), ints((M, K)), ints((M,))
    gw0, gb0 = ints((M, K)), ints((M,))
    out_ref, finput_ref = oracle.conv_updateOutput(x, w, b, *geo)
    go = ints(out_ref.shape)
    gi_ref, _ = oracle.conv_updateGradInput(go, w, x.shape, *geo)
    gw_ref, gb_ref = gw0.copy(), gb0.copy()
    oracle.conv_accGradParameters(go, finput_ref, gw_ref, gb_ref, 2.0)
    # gradWeight as a window of a larger buffer: guard rows before and behind it
    m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m._assign("bias", b)
    m.gpu()
    big = dev(gt, np.full((M + 2, K), 9.0, np.float32))
    m.gradWeight = big.narrow(0, 1, M)
    m.gradWeight.copy(gw0)
    m.gradBias.copy(gb0)
    dx, dgo = dev(gt, x), dev(gt, go)
    gt.gputorch.prof_reset()
    gt.gputorch.prof_enable(True)
    try:
        out = m.forward(dx).float()
        gi = m.updateGradInput(dx, dgo).float()
        m.accGradParameters(dx, dgo, 2.0)
        gt.gputorch.synchronize()
        labels = list(gt.gputorch.prof_report())
    finally:
        gt.gputorch.prof_enable(False)
        gt.gputorch.prof_reset()
    assert np.array_equal(out, out_ref) and np.array_equal(gi, gi_ref)
    got = big.float()
    assert np.array_equal(got[1:-1], gw_ref) and np.all(got[0] == 9.0) and np.all(got[-1] == 9.0)
    assert np.array_equal(m.gradBias.float(), gb_ref)
    gw_label = [k for k in labels if k.startswith("gemm_conv_gradweight")]
    assert len(gw_label) == 1 and "J=64 " in gw_label[0] and "tile=64x64" in gw_label[0] and "split=1 " not in gw_label[0] + " ", labels
    # no columns; no separate bias sum either where the reduction runs over a batch (one image: the two-stage sum)
    assert not any(k.startswith(("im2col",) + (("gradbias",) if B > 1 else ())) for k in labels), labels


NARROW_FORWARD = [  # B, C, H, W, kH, kW, pH, pW, sH, sW: 64 output planes, at most 32 taps, unit column stride,
    # Wo a multiple of 4, Ho*Wo a multiple of 128
    (3, 3, 16, 16, 3, 3, 1, 1, 1, 1),     # K = 27: the first layer of a VGG-style stack, small
    (2, 1, 19, 35, 4, 4, 0, 0, 1, 1),     # K = 16, unpadded: the input is read in place
    (2, 2, 31, 16, 3, 3, 1, 1, 2, 1),     # K = 18, strided along the rows
    (2, 2, 15, 17, 4, 4, 2, 1, 1, 1),     # K = 32: every step full
    (3, 1, 16, 16, 5, 5, 2, 2, 1, 1),     # K = 25: an odd count (the last step holds one tap)
    (1, 3, 32, 33, 3, 2, 1, 0, 1, 1),     # K = 18, a non-square kernel, one image
    (2, 3, 31, 24, 3, 3, 1, 1, 2, 1),     # K = 27, rows of 24 positions: a group of 128 spans rows
]


@pytest.mark.parametrize("relu", [False, True], ids=["plain", "relu"])
@pytest.mark.parametrize("cfg", NARROW_FORWARD)
def test_layers_with_a_handful_of_taps_run_the_narrow_forward_kernel_integer_exact(gt, gathered_route, switches, cfg, relu):
    """A layer with at most 32 taps and 64 output planes (the first layer of a VGG-style stack) computes its forward
    pass with weights held in registers and no tiled GEMM (conv_narrow.hip).  On integer data the result equals the
    oracle's bit for bit, with the bias added and, inside a fused stack, the ReLU applied on the way out; the timing
    label shows which kernel ran; with the conv_narrow_off switch the tiled kernel gives the same values; memory around
    the output is untouched."""
    B, C, H, W, kH, kW, pH, pW, sH, sW = cfg
    M, K = 64, C * kH * kW
    geo = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(77 + K + H)
    ints = lambda shape: rng.integers(-3, 4, shape).astype(np.float32)  # noqa: E731
    x, w, b = ints((B, C, H, W)), ints((M, K)), ints((M,))
    ref, _ = oracle.conv_updateOutput(x, w, b, *geo)
    assert (ref.shape[2] * ref.shape[3]) % 128 == 0 and ref.shape[3] % 4 == 0 and sW == 1
    if relu:
        ref = oracle.threshold_updateOutput(ref)

    def run():
        conv = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
        conv._assign("weight", w)
        conv._assign("bias", b)
        net = gt.nn.Sequential().add(conv)
        if relu:
            net.add(gt.nn.ReLU())
        net.gpu()
        if relu:
            net.fuse()
        # the output as a window of a larger buffer: guard planes before and behind it
        big = dev(gt, np.full((B + 2,) + ref.shape[1:], 9.0, np.float32))
        conv.output = big.narrow(0, 1, B)
        gt.gputorch.prof_reset()
        gt.gputorch.prof_enable(True)
        try:
            out = net.forward(dev(gt, x)).float()
            gt.gputorch.synchronize()
            labels = list(gt.gputorch.prof_report())
        finally:
            gt.gputorch.prof_enable(False)
            gt.gputorch.prof_reset()
        guard = big.float()
        assert np.all(guard[0] == 9.0) and np.all(guard[-1] == 9.0)
        return out, labels

    out, labels = run()
    assert np.array_equal(out, ref)
    assert any(k.startswith("conv_narrow_fwd") for k in labels) and not any(k.startswith("gemm_conv_fwd") for k in labels), labels
    switches("conv_narrow_off", "1")
    tiled, labels = run()
    assert np.array_equal(tiled, ref)
    assert any(k.startswith("gemm_conv_fwd") for k in labels) and not any(k.startswith("conv_narrow") for k in labels), labels


def test_narrow_forward_kernel_on_real_values_at_the_first_layer_of_the_vgg_stack(gt, gathered_route):
    """3 -> 64 planes, 3x3, padding 1, on 224x224 images (batch 4): within 1e-4*sqrt(27) of the oracle, norm-wise and
    element-wise."""
    B, C, H, W, M = 4, 3, 224, 224, 64
    rng = rng_for(781)
    x = uniform(rng, (B, C, H, W))
    w = uniform(rng, (M, 27)) / np.float32(np.sqrt(27))
    b = uniform(rng, (M,))
    ref, _ = oracle.conv_updateOutput(x, w, b, 3, 3, 1, 1, 1, 1)
    conv = gt.nn.SpatialConvolutionMM(C, M, 3, 3, 1, 1, 1)
    conv._assign("weight", w)
    conv._assign("bias", b)
    conv.gpu()
    gt.gputorch.prof_reset()
    gt.gputorch.prof_enable(True)
    try:
        out = conv.forward(dev(gt, x)).float()
        labels = list(gt.gputorch.prof_report())
    finally:
        gt.gputorch.prof_enable(False)
        gt.gputorch.prof_reset()
    assert any(k.startswith("conv_narrow_fwd") for k in labels), labels
    check_close("vgg first layer, narrow forward kernel", out, ref, 27)


NARROW_GRADWEIGHT = NARROW_FORWARD + [
    (4, 3, 40, 36, 3, 3, 1, 1, 1, 1),     # Ho*Wo = 1440: a multiple of 32 that is none of 128
    (130, 1, 5, 9, 4, 4, 1, 1, 1, 1),     # 32 positions per image, 130 images: one block per image
]


@pytest.mark.parametrize("cfg", NARROW_GRADWEIGHT)
def test_layers_with_a_handful_of_taps_run_the_narrow_gradweight_kernels_integer_exact(gt, gathered_route, switches, cfg):
    """gradWeight and gradBias of a layer with at most 32 taps and 64 output planes: partial sums per wavefront in
    registers, added up by a second launch (conv_narrow.hip).  On integer data both equal the oracle's bit for bit,
    accumulated onto what the tensors held, scaled; memory around gradWeight is untouched; two runs give identical
    bits; the timing labels show which kernels ran and that no tiled product, im2col or separate bias sum did."""
    B, C, H, W, kH, kW, pH, pW, sH, sW = cfg
    M, K = 64, C * kH * kW
    geo = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(177 + K + H)
    ints = lambda shape: rng.integers(-3, 4, shape).astype(np.float32)  # noqa: E731
    x, w, b = ints((B, C, H, W)), ints((M, K)), ints((M,))
    gw0, gb0 = ints((M, K)), ints((M,))
    out_ref, finput_ref = oracle.conv_updateOutput(x, w, b, *geo)
    go = ints(out_ref.shape)
    gw_ref, gb_ref = gw0.copy(), gb0.copy()
    oracle.conv_accGradParameters(go, finput_ref, gw_ref, gb_ref, 2.0)
    results = []
    for _ in range(2):
        m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
        m._assign("weight", w)
        m._assign("bias", b)
        m.gpu()
        big = dev(gt, np.full((M + 2, K), 9.0, np.float32))
        m.gradWeight = big.narrow(0, 1, M)
        m.gradWeight.copy(gw0)
        m.gradBias.copy(gb0)
        dx, dgo = dev(gt, x), dev(gt, go)
        gt.gputorch.prof_reset()
        gt.gputorch.prof_enable(True)
        try:
            m.accGradParameters(dx, dgo, 2.0)          # (without a forward pass: the padded input is rebuilt)
            gt.gputorch.synchronize()
            labels = list(gt.gputorch.prof_report())
        finally:
            gt.gputorch.prof_enable(False)
            gt.gputorch.prof_reset()
        got = big.float()
        assert np.array_equal(got[1:-1], gw_ref) and np.all(got[0] == 9.0) and np.all(got[-1] == 9.0)
        assert np.array_equal(m.gradBias.float(), gb_ref)
        assert any(k.startswith("conv_narrow_gradweight ") for k in labels) and "conv_narrow_gradweight_finish" in labels, labels
        assert not any(k.startswith(("gemm_", "im2col", "gradbias")) for k in labels), labels
        results.append((got.copy(), m.gradBias.float()))
    assert np.array_equal(results[0][0], results[1][0]) and np.array_equal(results[0][1], results[1][1])


def test_narrow_gradweight_kernels_on_real_values_at_the_first_layer_of_the_vgg_stack(gt, gathered_route):
    """3 -> 64 planes, 3x3, padding 1, on 224x224 images (batch 4): gradWeight and gradBias within 1e-4*sqrt(B*N) of the
    oracle, norm-wise and element-wise."""
    B, C, H, W, M = 4, 3, 224, 224, 64
    rng = rng_for(782)
    x = uniform(rng, (B, C, H, W))
    w = uniform(rng, (M, 27)) / np.float32(np.sqrt(27))
    b = uniform(rng, (M,))
    out_ref, finput_ref = oracle.conv_updateOutput(x, w, b, 3, 3, 1, 1, 1, 1)
    go = uniform(rng, out_ref.shape)
    gw_ref, gb_ref = np.zeros((M, 27), np.float32), np.zeros((M,), np.float32)
    oracle.use_blas(True)
    try:
        oracle.conv_accGradParameters(go, finput_ref, gw_ref, gb_ref, 1.0)
    finally:
        oracle.use_blas(False)
    conv = gt.nn.SpatialConvolutionMM(C, M, 3, 3, 1, 1, 1)
    conv._assign("weight", w)
    conv._assign("bias", b)
    conv.gpu()
    conv.zeroGradParameters()
    conv.accGradParameters(dev(gt, x), dev(gt, go), 1.0)
    check_close("vgg first layer gradWeight, narrow kernels", conv.gradWeight.float(), gw_ref, B * H * W)
    check_close("vgg first layer gradBias, narrow kernels", conv.gradBias.float(), gb_ref, B * H * W)


def narrow_draws(count):
    """Seeded random layers with 64 output planes and 16 .. 32 taps; about a third of them have the shape the kernels of
    conv_narrow.hip take (unit column stride, Wo a multiple of 4, Ho*Wo a multiple of 32 or 128), the rest run the tiled
    products for layers with fewer than 64 taps."""
    rng = rng_for(4242)
    out = []
    while len(out) < count:
        it = len(out)
        C, kH, kW = int(rng.integers(1, 5)), int(rng.integers(1, 6)), int(rng.integers(1, 6))
        if not 16 <= C * kH * kW <= 32:
            continue
        pH, pW = int(rng.integers(0, kH)), int(rng.integers(0, kW))
        sH, sW = int(rng.integers(1, 3)), int(rng.choice([1, 1, 1, 2]))
        Wo = int(rng.integers(1, 12)) * (4 if it % 5 else 3)
        Ho = int(rng.integers(1, 40))
        if it % 3 == 0:
            Ho = max(1, (128 // int(np.gcd(128, Wo))) * int(rng.integers(1, 3)))   # Ho*Wo a multiple of 128
        H, W = (Ho - 1) * sH + kH - 2 * pH, (Wo - 1) * sW + kW - 2 * pW
        if H < 1 or W < 1:
            continue
        B = 1 if it % 4 == 0 else int(rng.integers(2, 4))
        out.append((B, C, H, W, kH, kW, pH, pW, sH, sW))
    return out


@pytest.mark.parametrize("cfg", narrow_draws(48))
def test_random_layers_with_a_handful_of_taps_integer_exact(gt, gathered_route, cfg):
    """Forward and accGradParameters of 48 seeded random layers with 16 .. 32 taps and 64 output planes (a quarter of
    them single images) on integer data: output, gradWeight and gradBias bit for bit against the oracle, whichever
    kernels the library picks for the shape."""
    B, C, H, W, kH, kW, pH, pW, sH, sW = cfg
    K = C * kH * kW
    geo = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(9000 + 31 * H + W + K)
    ints = lambda shape: rng.integers(-3, 4, shape).astype(np.float32)  # noqa: E731
    x, w, b = ints((B, C, H, W)), ints((64, K)), ints((64,))
    ref, finput_ref = oracle.conv_updateOutput(x, w, b, *geo)
    go, gw, gb = ints(ref.shape), ints((64, K)), ints((64,))
    m = gt.nn.SpatialConvolutionMM(C, 64, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m._assign("bias", b)
    m.gpu()
    m.gradWeight.copy(gw)
    m.gradBias.copy(gb)
    dx = dev(gt, x)
    out = m.forward(dx).float()
    assert out.shape == ref.shape and np.array_equal(out, ref)
    oracle.conv_accGradParameters(go, finput_ref, gw, gb, 3.0)
    m.accGradParameters(dx, dev(gt, go), 3.0)
    assert np.array_equal(m.gradWeight.float(), gw) and np.array_equal(m.gradBias.float(), gb)
