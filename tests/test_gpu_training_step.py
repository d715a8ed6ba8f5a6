"""Two SGD steps of a small conv net + classifier + criterion through the Lua-mirror modules on the GPU, against the
same steps computed module by module with the CPU oracle:

  conv 3->8 k5 p2 -> ReLU -> maxpool 2 -> conv 8->12 k3 p1 -> ReLU -> sub-sampling 2x2 -> View -> Linear 192->32 -> ReLU
  -> Linear 32->10 -> LogSoftMax, ClassNLLCriterion; zeroGradParameters / forward / backward / updateParameters.

Every updated parameter must agree within 1e-4 relative after each step (the GEMMs sum in another order than the CPU
BLAS); the loss within 1e-5.  This is the call sequence of mcw_nn/StochasticGradient.lua:37-45.
"""
import numpy as np
import pytest

import oracle
from helpers import rel_err, rng_for, uniform

pytestmark = pytest.mark.gpu
f32 = np.float32


class CpuNet:
    """The same network on the oracle's functions, keeping what each backward needs."""

    def __init__(self, params):
        self.p = {k: v.copy() for k, v in params.items()}
        self.g = {k: np.zeros_like(v) for k, v in params.items()}

    def zero(self):
        for v in self.g.values():
            v[...] = 0

    def forward(self, x):
        p = self.p
        self.x = x
        self.c1, self.f1 = oracle.conv_updateOutput(x, p["w1"], p["b1"], 5, 5, 2, 2, 1, 1)
        self.r1 = oracle.threshold_updateOutput(self.c1)
        self.m1, self.ind = oracle.maxpool_updateOutput(self.r1, 2, 2, 2, 2)
        self.c2, self.f2 = oracle.conv_updateOutput(self.m1, p["w2"], p["b2"], 3, 3, 1, 1, 1, 1)
        self.r2 = oracle.threshold_updateOutput(self.c2)
        self.s2 = oracle.subsample_updateOutput(self.r2, p["ws"], p["bs"], 2, 2, 2, 2)
        self.v = self.s2.reshape(x.shape[0], -1)
        self.l1 = oracle.linear_updateOutput(self.v, p["w3"], p["b3"])
        self.r3 = oracle.threshold_updateOutput(self.l1)
        self.l2 = oracle.linear_updateOutput(self.r3, p["w4"], p["b4"])
        self.logp = oracle.logsoftmax_updateOutput(self.l2)
        return self.logp

    def backward(self, target):
        p, g = self.p, self.g
        d = oracle.classnll_updateGradInput(self.logp, target)
        d = oracle.logsoftmax_updateGradInput(d, self.logp)
        oracle.linear_accGradParameters(self.r3, d, g["w4"], g["b4"])
        d = oracle.linear_updateGradInput(d, p["w4"])
        d = oracle.threshold_updateGradInput(self.l1, d)
        oracle.linear_accGradParameters(self.v, d, g["w3"], g["b3"])
        d = oracle.linear_updateGradInput(d, p["w3"]).reshape(self.s2.shape)
        oracle.subsample_accGradParameters(self.r2, d, g["ws"], g["bs"], 2, 2, 2, 2)
        d = oracle.subsample_updateGradInput(d, p["ws"], self.r2.shape, 2, 2, 2, 2)
        d = oracle.threshold_updateGradInput(self.c2, d)
        oracle.conv_accGradParameters(d, self.f2, g["w2"], g["b2"])
        d, _ = oracle.conv_updateGradInput(d, p["w2"], self.m1.shape, 3, 3, 1, 1, 1, 1)
        d = oracle.maxpool_updateGradInput(d, self.ind, self.r1.shape, 2, 2)
        d = oracle.threshold_updateGradInput(self.c1, d)
        oracle.conv_accGradParameters(d, self.f1, g["w1"], g["b1"])
        d, _ = oracle.conv_updateGradInput(d, p["w1"], self.x.shape, 5, 5, 2, 2, 1, 1)
        return d

    def update(self, lr):
        for k in self.p:
            self.p[k] = (self.p[k] + f32(-lr) * self.g[k]).astype(f32)


def test_two_sgd_steps_match_the_cpu_modules():
    import mcw_cppamp_torch_amd as gt
    nn = gt.nn
    assert gt._lib.lib.thgpu_init() == 0
    rng = rng_for(101)
    B = 16
    net = nn.Sequential()
    conv1, conv2 = nn.SpatialConvolutionMM(3, 8, 5, 5, 1, 1, 2, rng=rng), nn.SpatialConvolutionMM(8, 12, 3, 3, 1, 1, 1, rng=rng)
    sub = nn.SpatialSubSampling(12, 2, 2, 2, 2, rng=rng)
    lin1, lin2 = nn.Linear(12 * 4 * 4, 32, rng=rng), nn.Linear(32, 10, rng=rng)
    for m in (conv1, nn.ReLU(), nn.SpatialMaxPooling(2, 2), conv2, nn.ReLU(), sub, nn.View(12 * 4 * 4), lin1, nn.ReLU(),
              lin2, nn.LogSoftMax()):
        net.add(m)
    crit = nn.ClassNLLCriterion()
    params = {"w1": np.array(conv1.weight), "b1": np.array(conv1.bias), "w2": np.array(conv2.weight),
              "b2": np.array(conv2.bias), "ws": np.array(sub.weight), "bs": np.array(sub.bias),
              "w3": np.array(lin1.weight), "b3": np.array(lin1.bias), "w4": np.array(lin2.weight),
              "b4": np.array(lin2.bias)}
    cpu = CpuNet(params)
    net.gpu()
    crit.gpu()
    gpu_params = {"w1": conv1.weight, "b1": conv1.bias, "w2": conv2.weight, "b2": conv2.bias, "ws": sub.weight,
                  "bs": sub.bias, "w3": lin1.weight, "b3": lin1.bias, "w4": lin2.weight, "b4": lin2.bias}
    lr = 0.05
    for step in range(2):
        x = uniform(rng, (B, 3, 16, 16))
        target = rng.integers(1, 11, size=B)
        dx, dt = gt.GPUTensor.from_numpy(x), gt.GPUTensor.from_numpy(target.astype(f32))
        # mcw_nn/StochasticGradient.lua:37-45
        loss = crit.forward(net.forward(dx), dt)
        net.zeroGradParameters()
        gin = net.backward(dx, crit.backward(net.output, dt))
        net.updateParameters(lr)

        ref_loss = oracle.classnll_updateOutput(cpu.forward(x), target)
        cpu.zero()
        ref_gin = cpu.backward(target)
        cpu.update(lr)
        assert abs(loss - ref_loss) < 1e-5 * max(1.0, abs(ref_loss)), (step, loss, ref_loss)
        assert rel_err(net.output.float(), cpu.logp) < 1e-5
        assert rel_err(gin.float(), ref_gin) < 1e-4
        errs = {k: rel_err(t.float(), cpu.p[k]) for k, t in gpu_params.items()}
        assert max(errs.values()) < 1e-4, (step, errs)
    assert net.get(6).output.size() == (B, 192) and net.get(6).gradInput.size() == (B, 12, 4, 4)


def test_view_reshape_and_update_helpers():
    import mcw_cppamp_torch_amd as gt
    nn = gt.nn
    rng = rng_for(102)
    a = uniform(rng, (4, 3, 2, 5))
    d = gt.GPUTensor.from_numpy(a)
    v = d.view(4, 30)
    assert v.size() == (4, 30) and v.data_ptr() == d.data_ptr() and np.array_equal(v.float(), a.reshape(4, 30))
    assert d.view(-1, 10).size() == (12, 10) and d.view(2, 2, -1).size() == (2, 2, 30)
    with pytest.raises(gt.THGPUError, match="Wrong size for view"):
        d.view(7, 7)
    with pytest.raises(gt.THGPUError, match="contiguous"):
        d.transpose(0, 1).view(120)
    # nn.View keeps the batch dimension when the per-sample element count matches
    m = nn.View(30).gpu()
    assert m.forward(d).size() == (4, 30)
    assert m.backward(d, m.output).size() == a.shape
    assert nn.View(6, 5).forward(gt.GPUTensor.from_numpy(a[0])).size() == (6, 5)
    assert nn.View(30).setNumInputDims(3).forward(d).size() == (4, 30)
    # nn.Reshape copies a non-contiguous input
    r = nn.Reshape(10, 3).gpu()
    dt = d.transpose(2, 3)
    out = r.forward(dt)
    assert out.size() == (4, 10, 3) and np.array_equal(out.float(), a.transpose(0, 1, 3, 2).reshape(4, 10, 3))
    assert r.backward(dt, out).size() == dt.size()
    assert nn.Reshape(120, False).gpu().forward(d).size() == (120,)
    # accUpdateGradParameters adds -lr * gradient straight into the parameters (mcw_nn/Module.lua:49-57)
    lin = nn.Linear(5, 3, rng=rng)
    w0, b0 = np.array(lin.weight), np.array(lin.bias)
    lin.gpu()
    x, go = uniform(rng, (7, 5)), uniform(rng, (7, 3))
    dx, dgo = gt.GPUTensor.from_numpy(x), gt.GPUTensor.from_numpy(go)
    lin.forward(dx)
    lin.backwardUpdate(dx, dgo, 0.5)
    gw, gb = np.zeros_like(w0), np.zeros_like(b0)
    oracle.linear_accGradParameters(x, go, gw, gb, 1.0)
    assert rel_err(lin.weight.float(), w0 - 0.5 * gw) < 1e-5 and rel_err(lin.bias.float(), b0 - 0.5 * gb) < 1e-5
