"""Host-side mirror of the `nn` modules on the convolution hot path, dispatching
to the C ABI the way the Lua modules dispatch to `input.nn.<Op>_<method>`:

  nn.Module                mcw_nn/Module.lua:1-164
  nn.Sequential            mcw_nn/Sequential.lua:1-129
  nn.SpatialConvolutionMM  mcw_nn/SpatialConvolutionMM.lua:1-60
  nn.SpatialMaxPooling     mcw_nn/SpatialMaxPooling.lua:1-34
  nn.Threshold / nn.ReLU   mcw_nn/Threshold.lua:1-21, mcw_nn/ReLU.lua:1-5
  nn.Linear                mcw_nn/Linear.lua:1-104 (the classifier after a conv stack)
  nn.SpatialAveragePooling mcw_nn/SpatialAveragePooling.lua:1-20
  nn.SpatialSubSampling    mcw_nn/SpatialSubSampling.lua:1-54
  nn.View, nn.Reshape      mcw_nn/View.lua:1-47, mcw_nn/Reshape.lua:1-70 (between a conv stack and its classifier)
  nn.LogSoftMax            mcw_nn/LogSoftMax.lua:1-9
  nn.Criterion, nn.ClassNLLCriterion   mcw_nn/Criterion.lua:1-44, mcw_nn/ClassNLLCriterion.lua:1-72

Same constructor arguments, field names and call order.  Modules are created
with host tensors (numpy float32, like torch.Tensor) and moved with :gpu();
only torch.GPUTensor inputs are computed -- there is no CPU implementation in
this package.
"""
import ctypes
import math

import numpy as np

from . import _lib
from ._lib import THGPUError, lib
from .gputorch import FloatTensor, GPUTensor


def _is_tensor(v):
    return isinstance(v, (GPUTensor, np.ndarray))


def _convert(v, type_name):
    if isinstance(v, (list, tuple)) and v and all(_is_tensor(x) for x in v):
        return [_convert(x, type_name) for x in v]
    if isinstance(v, GPUTensor):
        return v.type(type_name)
    if isinstance(v, np.ndarray):
        if type_name == "torch.GPUTensor":
            return GPUTensor.from_numpy(v.astype(np.float32, copy=False))
        if type_name == "torch.FloatTensor":
            return np.ascontiguousarray(v, np.float32).view(FloatTensor)
        if type_name == "torch.DoubleTensor":
            return np.ascontiguousarray(v, np.float64)
        raise THGPUError("unknown tensor type %s" % type_name)
    return v


def _require_gpu(*tensors):
    for t in tensors:
        if not isinstance(t, GPUTensor):
            raise THGPUError("torch.GPUTensor expected (this package implements only the GPU path; "
                             "move tensors and modules with :gpu())")


class Module(object):
    def __init__(self):
        self.gradInput = FloatTensor()
        self.output = FloatTensor()

    def parameters(self):
        w, b = getattr(self, "weight", None), getattr(self, "bias", None)
        if w is not None and b is not None:
            return [w, b], [self.gradWeight, self.gradBias]
        if w is not None:
            return [w], [self.gradWeight]
        if b is not None:
            return [b], [self.gradBias]
        return None, None

    def updateOutput(self, input):
        return self.output

    def forward(self, input):
        return self.updateOutput(input)

    def backward(self, input, gradOutput, scale=1):
        self.updateGradInput(input, gradOutput)
        self.accGradParameters(input, gradOutput, scale)
        return self.gradInput

    def updateGradInput(self, input, gradOutput):
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1):
        pass

    def zeroGradParameters(self):
        _, grads = self.parameters()
        for g in grads or []:
            if isinstance(g, GPUTensor):
                g.zero()
            else:
                g[...] = 0

    def updateParameters(self, learningRate):
        # mcw_nn/Module.lua:75-82
        params, grads = self.parameters()
        for p, g in zip(params or [], grads or []):
            if isinstance(p, GPUTensor):
                p.add(-learningRate, g)
            else:
                p += np.float32(-learningRate) * g

    def accUpdateGradParameters(self, input, gradOutput, lr):
        # mcw_nn/Module.lua:49-57: accumulate straight into the parameters with scale -lr
        gw, gb = getattr(self, "gradWeight", None), getattr(self, "gradBias", None)
        self.gradWeight, self.gradBias = getattr(self, "weight", None), getattr(self, "bias", None)
        try:
            self.accGradParameters(input, gradOutput, -lr)
        finally:
            self.gradWeight, self.gradBias = gw, gb

    def backwardUpdate(self, input, gradOutput, lr):
        # mcw_nn/Module.lua:35-39
        self.updateGradInput(input, gradOutput)
        self.accUpdateGradParameters(input, gradOutput, lr)
        return self.gradInput

    def type(self, type_name):
        for key, val in list(self.__dict__.items()):
            if key != "modules":
                self.__dict__[key] = _convert(val, type_name)
        for m in getattr(self, "modules", []):
            m.type(type_name)
        return self

    def gpu(self):
        return self.type("torch.GPUTensor")

    def float(self):
        return self.type("torch.FloatTensor")

    def double(self):
        return self.type("torch.DoubleTensor")

    def reset(self, stdv=None):
        pass


class Sequential(Module):
    def __init__(self):
        Module.__init__(self)
        self.modules = []

    def add(self, module):
        if not self.modules:
            self.gradInput = module.gradInput
        self.modules.append(module)
        self.output = module.output
        return self

    def size(self):
        return len(self.modules)

    def get(self, index):
        return self.modules[index]

    def updateOutput(self, input):
        cur = input
        for m in self.modules:
            cur = m.updateOutput(cur)
        self.output = cur
        return cur

    def updateGradInput(self, input, gradOutput):
        # mcw_nn/Sequential.lua:45-57.  After fuse(), a module whose gradInput is the gradOutput of a convolution in
        # front of it (_grad_consumer) also stores it in the padded layout that convolution's gradInput product
        # gathers from, and the convolution is told so -- only here, where nothing can touch either copy in between;
        # a module called on its own always takes the ordinary route.
        cur = gradOutput
        ready_for = None                 # the convolution whose fgradInput already holds `cur` in padded form
        for i in range(len(self.modules) - 1, -1, -1):
            m = self.modules[i]
            inp = self.modules[i - 1].output if i > 0 else input
            link = getattr(m, "_grad_consumer", None)
            twin = None
            if link is not None:
                consumer, ci = link
                twin = consumer._gradOutputTwin(self.modules[ci - 1].output if ci > 0 else input)
            if twin is not None or (ready_for is m and ready_for is not None):
                cur = m._updateGradInputTwin(inp, cur, twin, ready_for is m)
                ready_for = link[0] if (twin is not None and m._wrote_twin) else None
            else:
                cur = m.updateGradInput(inp, cur)
                if not (isinstance(m, Threshold) and m.fusedBackward):   # that one hands its gradOutput on untouched
                    ready_for = None
        self.gradInput = cur
        return cur

    def accGradParameters(self, input, gradOutput, scale=1):
        cur = gradOutput
        for i in range(len(self.modules) - 1, 0, -1):
            self.modules[i].accGradParameters(self.modules[i - 1].output, cur, scale)
            cur = self.modules[i].gradInput
        self.modules[0].accGradParameters(input, cur, scale)

    def accUpdateGradParameters(self, input, gradOutput, lr):
        # mcw_nn/Sequential.lua:72-83
        cur = gradOutput
        for i in range(len(self.modules) - 1, 0, -1):
            self.modules[i].accUpdateGradParameters(self.modules[i - 1].output, cur, lr)
            cur = self.modules[i].gradInput
        self.modules[0].accUpdateGradParameters(input, cur, lr)

    def zeroGradParameters(self):
        # mcw_nn/Sequential.lua:85-89 calls every module's zeroGradParameters.  Modules that keep Module's own
        # implementation are served together -- their dense GPU gradients go in one launch; a module (or nested
        # container) that overrides the method has its own called.
        plain, grads = [], []
        for m in self.modules:
            if type(m).zeroGradParameters is Module.zeroGradParameters and type(m).parameters in (
                    Module.parameters,):
                plain.append(m)
            else:
                m.zeroGradParameters()
        for m in plain:
            _, g = m.parameters()
            grads.extend(g or [])
        gpu = [g for g in grads if isinstance(g, GPUTensor) and g.isContiguous()]
        if len(gpu) > 1:
            arr = (_lib.TensorP * len(gpu))(*[g._p for g in gpu])
            _lib.check_status(lib.thgpu_fill_many(arr, len(gpu), 0.0))
        else:
            gpu = []
        for g in grads:
            if isinstance(g, GPUTensor):
                if not any(g is h for h in gpu):
                    g.zero()
            else:
                g[...] = 0

    def fuse(self):
        """Lets the neighbours of every nn.Threshold / nn.ReLU do its work while they store their own results: a
        SpatialConvolutionMM in front applies the threshold to its output, a SpatialConvolutionMM or
        SpatialMaxPooling behind zeroes its gradInput where its input (the Threshold's output) is not above the
        threshold.  The Threshold module stays in place and passes tensors through, so the module API and every
        result downstream are unchanged bit for bit; what changes is that the convolution's `output` holds the
        thresholded values and no separate elementwise pass runs.  Needs value <= threshold (true of ReLU), so that
        output > threshold exactly where input > threshold.  Returns self; unfuse() undoes it."""
        self.unfuse()
        mods = self.modules
        for i, m in enumerate(mods):
            if isinstance(m, Sequential):
                m.fuse()
            if not isinstance(m, Threshold) or not m.val <= m.threshold:
                continue
            if i > 0 and isinstance(mods[i - 1], SpatialConvolutionMM) and mods[i - 1].fusedThreshold is None:
                mods[i - 1].fusedThreshold = (m.threshold, m.val)
                m.fusedForward = True
            if i + 1 < len(mods) and isinstance(mods[i + 1], (SpatialConvolutionMM, SpatialMaxPooling)):
                mods[i + 1].inputThreshold = m.threshold
                m.fusedBackward = True
        # A convolution or pooling layer whose output reaches a convolution unchanged (directly, or through a
        # Threshold the convolution in front applies itself) writes it into that convolution's padded image.
        for i, m in enumerate(mods):
            if not isinstance(m, (SpatialConvolutionMM, SpatialMaxPooling)):
                continue
            j = i + 1
            if j < len(mods) and isinstance(mods[j], Threshold) and mods[j].fusedForward:
                j += 1
            if j < len(mods) and isinstance(mods[j], SpatialConvolutionMM):
                m._consumer = mods[j]
        # Backward: the module whose gradInput reaches a convolution's updateGradInput as gradOutput unchanged
        # (directly, or through a Threshold whose backward that module applies itself).
        for i, m in enumerate(mods):
            if not isinstance(m, SpatialConvolutionMM) or m.gradInput is None:
                continue
            j = i + 1
            if j < len(mods) and isinstance(mods[j], Threshold) and mods[j].fusedBackward:
                j += 1
            if j < len(mods) and j > i and isinstance(mods[j], (SpatialConvolutionMM, SpatialMaxPooling)) and (
                    j == i + 1 or mods[j].inputThreshold is not None):
                mods[j]._grad_consumer = (m, i)
        return self

    def unfuse(self):
        for m in self.modules:
            if isinstance(m, Sequential):
                m.unfuse()
            elif isinstance(m, Threshold):
                if m.fusedForward or m.fusedBackward:
                    m.output, m.gradInput = type(m.output)(), type(m.gradInput)()
                m.fusedForward = m.fusedBackward = False
            elif isinstance(m, SpatialConvolutionMM):
                m.fusedThreshold = m.inputThreshold = None
            elif isinstance(m, SpatialMaxPooling):
                m.inputThreshold = None
            if isinstance(m, (SpatialConvolutionMM, SpatialMaxPooling)):
                m._consumer = None
                m._grad_consumer = None
                if getattr(m.output, "_zero_border", None) is not None:
                    m.output = type(m.output)()
        return self

    def updateParameters(self, learningRate):
        # mcw_nn/Sequential.lua:91-95
        for m in self.modules:
            m.updateParameters(learningRate)

    def parameters(self):
        # mcw_nn/Sequential.lua:121-141: the modules' parameters and gradients, flattened in module order
        w, gw = [], []
        for m in self.modules:
            mw, mgw = m.parameters()
            if mw:
                w.extend(mw)
                gw.extend(mgw)
        return w, gw

    def insert(self, module, index=None):
        # mcw_nn/Sequential.lua:17-25 (index counts from 0 here)
        index = len(self.modules) if index is None else index
        if index > len(self.modules):
            raise THGPUError("index should be contiguous to existing modules")
        self.modules.insert(index, module)
        self.output = self.modules[-1].output
        self.gradInput = self.modules[0].gradInput
        return self

    def reset(self, stdv=None):
        for m in self.modules:
            m.reset(stdv)


def _padded_output(module, sizes):
    """Gives `module.output` the `sizes` it is about to be resized to, as the interior of a zero-bordered buffer,
    when the convolution that consumes it (module._consumer, set by Sequential.fuse) gathers from its padded input
    at this size: the producer then writes the consumer's padded image itself and no copy of it is ever made.  The
    view carries the border it sits in as `_zero_border`; consumers trust no tensor without that mark."""
    consumer = getattr(module, "_consumer", None)
    out = module.output
    if consumer is not None and isinstance(out, GPUTensor):
        B = sizes[0] if len(sizes) == 4 else 1
        C, H, W = sizes[-3:]
        pH, pW = consumer.padH, consumer.padW
        if (pH or pW) and C == consumer.nInputPlane and lib.thgpu_conv_gathers(
                B, C, H, W, consumer.nOutputPlane, consumer.kW, consumer.kH, consumer.dW, consumer.dH, pW, pH):
            if getattr(out, "_zero_border", None) == (pH, pW) and tuple(out.size()) == tuple(sizes):
                return
            buf = GPUTensor(*(tuple(sizes[:-2]) + (H + 2 * pH, W + 2 * pW)))
            buf.zero()
            nd = len(sizes)
            view = buf.narrow(nd - 2, pH, H).narrow(nd - 1, pW, W)
            view._zero_border = (pH, pW)
            view._padded_buffer = buf
            module.output = view
            return
    if getattr(out, "_zero_border", None) is not None:
        module.output = GPUTensor()      # back to a tensor of its own


def _in_padded_buffer(input, padH, padW):
    """Whether `input` may be handed to a convolution as lying in its own zero-bordered buffer."""
    if (padH, padW) == (0, 0):
        return isinstance(input, GPUTensor) and input.isContiguous()
    return getattr(input, "_zero_border", None) == (padH, padW)


class SpatialConvolutionMM(Module):
    """nn.SpatialConvolutionMM(nInputPlane, nOutputPlane, kW, kH, dW, dH, padding).

    `padW`/`padH` (keyword only) override the single symmetric `padding` of the
    reference for kernels that need different vertical and horizontal padding.
    Unlike the reference CPU module (mcw_nn/generic/SpatialConvolutionMM.c:
    148-149) any stride is accepted.
    """

    def __init__(self, nInputPlane, nOutputPlane, kW, kH, dW=1, dH=1, padding=0, padW=None, padH=None, rng=None):
        Module.__init__(self)
        self.nInputPlane, self.nOutputPlane = nInputPlane, nOutputPlane
        self.kW, self.kH, self.dW, self.dH = kW, kH, dW, dH
        self.padding = padding or 0
        self.padW = self.padding if padW is None else padW
        self.padH = self.padding if padH is None else padH
        K = nInputPlane * kH * kW
        self.weight = FloatTensor(nOutputPlane, K)
        self.bias = FloatTensor(nOutputPlane)
        self.gradWeight = FloatTensor(nOutputPlane, K)
        self.gradBias = FloatTensor(nOutputPlane)
        self.finput = FloatTensor()
        self.fgradInput = FloatTensor()
        # set by Sequential.fuse(): (threshold, value) of a following nn.Threshold applied as the output is stored,
        # and the threshold of a preceding one whose backward is applied as gradInput is stored
        self.fusedThreshold = None
        self.inputThreshold = None
        self._rng = rng if rng is not None else np.random.default_rng()
        self.reset()

    def reset(self, stdv=None):
        # mcw_nn/SpatialConvolutionMM.lua:29-46
        if stdv:
            stdv = stdv * math.sqrt(3)
        else:
            stdv = 1.0 / math.sqrt(self.kW * self.kH * self.nInputPlane)
        w = self._rng.uniform(-stdv, stdv, size=(self.nOutputPlane, self.nInputPlane * self.kH * self.kW))
        b = self._rng.uniform(-stdv, stdv, size=(self.nOutputPlane,))
        self._assign("weight", w)
        self._assign("bias", b)

    def _assign(self, name, host):
        cur = getattr(self, name)
        if isinstance(cur, GPUTensor):
            cur.copy(np.asarray(host, np.float32))
        else:
            setattr(self, name, np.asarray(host, np.float32).view(FloatTensor))

    def _geom(self):
        return (self.kW, self.kH, self.dW, self.dH, self.padW, self.padH)

    def updateOutput(self, input):
        _require_gpu(input, self.weight, self.bias, self.finput, self.fgradInput, self.output)
        if getattr(self, "_consumer", None) is not None or getattr(self.output, "_zero_border", None) is not None:
            sz = input.size()
            if len(sz) in (3, 4):
                Ho = (sz[-2] + 2 * self.padH - self.kH) // self.dH + 1
                Wo = (sz[-1] + 2 * self.padW - self.kW) // self.dW + 1
                if Ho > 0 and Wo > 0:
                    _padded_output(self, tuple(sz[:-3]) + (self.nOutputPlane, Ho, Wo))
        flags = (1 if self.fusedThreshold is not None else 0) | (2 if _in_padded_buffer(input, self.padH, self.padW) else 0)
        if flags:
            th, val = self.fusedThreshold if self.fusedThreshold is not None else (0.0, 0.0)
            _lib.check_status(lib.thgpu_SpatialConvolutionMM_updateOutputFused(
                input._p, self.weight._p, self.bias._p, self.finput._p, self.fgradInput._p, self.output._p,
                *(self._geom() + (flags, float(th), float(val)))))
            return self.output
        _lib.check_status(lib.thgpu_SpatialConvolutionMM_updateOutput(
            input._p, self.weight._p, self.bias._p, self.finput._p, self.fgradInput._p, self.output._p,
            *self._geom()))
        return self.output

    def updateGradInput(self, input, gradOutput):
        if self.gradInput is None:
            return None
        _require_gpu(input, gradOutput, self.weight, self.finput, self.fgradInput, self.gradInput)
        if self.inputThreshold is not None:
            _lib.check_status(lib.thgpu_SpatialConvolutionMM_updateGradInputFused(
                input._p, gradOutput._p, self.weight._p, self.finput._p, self.fgradInput._p, self.gradInput._p,
                *(self._geom() + (1, float(self.inputThreshold)))))
            return self.gradInput
        _lib.check_status(lib.thgpu_SpatialConvolutionMM_updateGradInput(
            input._p, gradOutput._p, self.weight._p, self.finput._p, self.fgradInput._p, self.gradInput._p,
            *self._geom()))
        return self.gradInput

    def _gradOutputTwin(self, input):
        """The view through which the producer of this layer's gradOutput can store it in the padded layout at the
        head of fgradInput (thgpu_SpatialConvolutionMM_gradOutputTwin), or None when this layer's gradInput does not
        take the gathered route."""
        if self.gradInput is None or not all(isinstance(t, GPUTensor) for t in (input, self.weight, self.fgradInput)):
            return None
        twin = getattr(self, "_twin_view", None)
        if twin is None:
            twin = self._twin_view = GPUTensor()
        available = ctypes.c_int(0)
        _lib.check_status(lib.thgpu_SpatialConvolutionMM_gradOutputTwin(
            input._p, self.weight._p, self.fgradInput._p, twin._p, *(self._geom() + (ctypes.byref(available),))))
        return twin if available.value else None

    def _updateGradInputTwin(self, input, gradOutput, twin, ready):
        """updateGradInput inside a fused Sequential: `twin` (or None) receives a second copy of gradInput, `ready`
        says that gradOutput already lies in this layer's fgradInput (see Sequential.updateGradInput)."""
        self._wrote_twin = False
        if self.gradInput is None:
            return None
        _require_gpu(input, gradOutput, self.weight, self.finput, self.fgradInput, self.gradInput)
        flags = (1 if self.inputThreshold is not None else 0) | (8 if ready else 0)
        wrote = ctypes.c_int(0)
        _lib.check_status(lib.thgpu_SpatialConvolutionMM_updateGradInputTwin(
            input._p, gradOutput._p, self.weight._p, self.finput._p, self.fgradInput._p, self.gradInput._p,
            *(self._geom() + (flags, float(self.inputThreshold or 0.0), twin._p if twin is not None else None,
                              ctypes.byref(wrote)))))
        self._wrote_twin = bool(wrote.value)
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1):
        _require_gpu(input, gradOutput, self.gradWeight, self.gradBias, self.finput, self.fgradInput)
        if _in_padded_buffer(input, self.padH, self.padW):
            _lib.check_status(lib.thgpu_SpatialConvolutionMM_accGradParametersFused(
                input._p, gradOutput._p, self.gradWeight._p, self.gradBias._p, self.finput._p, self.fgradInput._p,
                *(self._geom() + (float(scale), 2))))
            return
        _lib.check_status(lib.thgpu_SpatialConvolutionMM_accGradParameters(
            input._p, gradOutput._p, self.gradWeight._p, self.gradBias._p, self.finput._p, self.fgradInput._p,
            *(self._geom() + (float(scale),))))


class Linear(Module):
    """nn.Linear(inputSize, outputSize): the statement-for-statement mirror of mcw_nn/Linear.lua:3-101 on GPU tensors
    (addmv / addr / addmm of the tensor library; 1-D and 2-D inputs, the nunit == 1 special case included)."""

    _assign = SpatialConvolutionMM._assign

    def __init__(self, inputSize, outputSize, rng=None):
        Module.__init__(self)
        self.weight = FloatTensor(outputSize, inputSize)
        self.bias = FloatTensor(outputSize)
        self.gradWeight = FloatTensor(outputSize, inputSize)
        self.gradBias = FloatTensor(outputSize)
        self._rng = rng if rng is not None else np.random.default_rng()
        self.reset()

    def reset(self, stdv=None):
        # mcw_nn/Linear.lua:15-32
        shape = tuple(self.weight.size()) if isinstance(self.weight, GPUTensor) else self.weight.shape
        stdv = stdv * math.sqrt(3) if stdv else 1.0 / math.sqrt(shape[1])
        self._assign("weight", self._rng.uniform(-stdv, stdv, size=shape))
        self._assign("bias", self._rng.uniform(-stdv, stdv, size=(shape[0],)))

    def updateOutput(self, input):
        _require_gpu(input, self.weight, self.bias, self.output)
        if input.dim() == 1:
            self.output.resize(self.bias.size(0))
            self.output.copy(self.bias)
            self.output.addmv(1, self.weight, input)
        elif input.dim() == 2:
            nframe, nunit = input.size(0), self.bias.size(0)
            self.output.resize(nframe, nunit)
            if nunit == 1:
                self.output.zero().add(self.bias[0])
                self.output.select(1, 0).addmv(1, input, self.weight.select(0, 0))
            else:
                self.output.zero().addr(1, GPUTensor(nframe).fill(1), self.bias)
                self.output.addmm(1, input, self.weight.t())
        else:
            raise ValueError("input must be vector or matrix")
        return self.output

    def updateGradInput(self, input, gradOutput):
        if self.gradInput is None:
            return None
        _require_gpu(input, gradOutput, self.weight, self.gradInput)
        n = self.gradInput.nElement()
        self.gradInput.resizeAs(input)
        if self.gradInput.nElement() != n:
            self.gradInput.zero()
        if input.dim() == 1:
            self.gradInput.addmv(0, 1, self.weight.t(), gradOutput)
        elif input.dim() == 2:
            self.gradInput.addmm(0, 1, gradOutput, self.weight)
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1):
        _require_gpu(input, gradOutput, self.gradWeight, self.gradBias)
        if input.dim() == 1:
            self.gradWeight.addr(scale, gradOutput, input)
            self.gradBias.add(scale, gradOutput)
        elif input.dim() == 2:
            nframe, nunit = input.size(0), self.bias.size(0)
            ones = GPUTensor(nframe).fill(1)
            if nunit == 1:
                self.gradWeight.select(0, 0).addmv(scale, input.t(), gradOutput.select(1, 0))
            else:
                self.gradWeight.addmm(scale, gradOutput.t(), input)
            self.gradBias.addmv(scale, gradOutput.t(), ones)


class SpatialMaxPooling(Module):
    """nn.SpatialMaxPooling(kW, kH, dW, dH); dW, dH default to kW, kH."""

    def __init__(self, kW, kH, dW=None, dH=None):
        Module.__init__(self)
        self.kW, self.kH = kW, kH
        self.dW = dW or kW
        self.dH = dH or kH
        self.indices = FloatTensor()
        self.inputThreshold = None   # set by Sequential.fuse(): the threshold of a preceding nn.Threshold

    def updateOutput(self, input):
        _require_gpu(input, self.output, self.indices)
        if getattr(self, "_consumer", None) is not None or getattr(self.output, "_zero_border", None) is not None:
            sz = input.size()
            if len(sz) in (3, 4):
                Ho, Wo = (sz[-2] - self.kH) // self.dH + 1, (sz[-1] - self.kW) // self.dW + 1
                if Ho > 0 and Wo > 0:
                    _padded_output(self, tuple(sz[:-2]) + (Ho, Wo))
        _lib.check_status(lib.thgpu_SpatialMaxPooling_updateOutput(
            input._p, self.output._p, self.indices._p, self.kW, self.kH, self.dW, self.dH))
        return self.output

    def updateGradInput(self, input, gradOutput):
        _require_gpu(input, gradOutput, self.gradInput, self.indices)
        if self.inputThreshold is not None:
            _lib.check_status(lib.thgpu_SpatialMaxPooling_updateGradInputMasked(
                input._p, gradOutput._p, self.gradInput._p, self.indices._p, self.kW, self.kH, self.dW, self.dH,
                float(self.inputThreshold)))
            return self.gradInput
        _lib.check_status(lib.thgpu_SpatialMaxPooling_updateGradInput(
            input._p, gradOutput._p, self.gradInput._p, self.indices._p, self.kW, self.kH, self.dW, self.dH))
        return self.gradInput


    def _updateGradInputTwin(self, input, gradOutput, twin, ready):
        """updateGradInput that also stores gradInput through `twin` (see Sequential.updateGradInput)."""
        _require_gpu(input, gradOutput, self.gradInput, self.indices)
        wrote = ctypes.c_int(0)
        _lib.check_status(lib.thgpu_SpatialMaxPooling_updateGradInputTwin(
            input._p, gradOutput._p, self.gradInput._p, self.indices._p, self.kW, self.kH, self.dW, self.dH,
            1 if self.inputThreshold is not None else 0, float(self.inputThreshold or 0.0),
            twin._p if twin is not None else None, ctypes.byref(wrote)))
        self._wrote_twin = bool(wrote.value)
        return self.gradInput


class SpatialAveragePooling(Module):
    """nn.SpatialAveragePooling(kW, kH, dW, dH); dW, dH default to 1 (mcw_nn/SpatialAveragePooling.lua:3-20).
    The module returns the window sum, as the reference's does."""

    def __init__(self, kW, kH, dW=None, dH=None):
        Module.__init__(self)
        self.kW, self.kH = kW, kH
        self.dW = dW or 1
        self.dH = dH or 1

    def updateOutput(self, input):
        _require_gpu(input, self.output)
        _lib.check_status(lib.thgpu_SpatialAveragePooling_updateOutput(
            input._p, self.output._p, self.kW, self.kH, self.dW, self.dH))
        return self.output

    def updateGradInput(self, input, gradOutput):
        _require_gpu(input, gradOutput, self.gradInput)
        _lib.check_status(lib.thgpu_SpatialAveragePooling_updateGradInput(
            input._p, gradOutput._p, self.gradInput._p, self.kW, self.kH, self.dW, self.dH))
        return self.gradInput


class SpatialSubSampling(Module):
    """nn.SpatialSubSampling(nInputPlane, kW, kH, dW, dH); dW, dH default to 1; weight and bias drawn from
    U(-1/sqrt(kW*kH), 1/sqrt(kW*kH)) (mcw_nn/SpatialSubSampling.lua:3-54)."""

    _assign = SpatialConvolutionMM._assign

    def __init__(self, nInputPlane, kW, kH, dW=None, dH=None, rng=None):
        Module.__init__(self)
        self.nInputPlane = nInputPlane
        self.kW, self.kH = kW, kH
        self.dW = dW or 1
        self.dH = dH or 1
        self.weight = FloatTensor(nInputPlane)
        self.bias = FloatTensor(nInputPlane)
        self.gradWeight = FloatTensor(nInputPlane)
        self.gradBias = FloatTensor(nInputPlane)
        self._rng = rng if rng is not None else np.random.default_rng()
        self.reset()

    def reset(self, stdv=None):
        stdv = stdv * math.sqrt(3) if stdv else 1.0 / math.sqrt(self.kW * self.kH)
        self._assign("weight", self._rng.uniform(-stdv, stdv, size=(self.nInputPlane,)))
        self._assign("bias", self._rng.uniform(-stdv, stdv, size=(self.nInputPlane,)))

    def updateOutput(self, input):
        _require_gpu(input, self.weight, self.bias, self.output)
        _lib.check_status(lib.thgpu_SpatialSubSampling_updateOutput(
            input._p, self.weight._p, self.bias._p, self.output._p, self.kW, self.kH, self.dW, self.dH))
        return self.output

    def updateGradInput(self, input, gradOutput):
        _require_gpu(input, gradOutput, self.weight, self.gradInput)
        _lib.check_status(lib.thgpu_SpatialSubSampling_updateGradInput(
            input._p, gradOutput._p, self.weight._p, self.gradInput._p, self.kW, self.kH, self.dW, self.dH))
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1.0):
        _require_gpu(input, gradOutput, self.gradWeight, self.gradBias)
        _lib.check_status(lib.thgpu_SpatialSubSampling_accGradParameters(
            input._p, gradOutput._p, self.gradWeight._p, self.gradBias._p, self.kW, self.kH, self.dW, self.dH,
            float(scale)))


class Threshold(Module):
    """nn.Threshold(threshold, value)."""

    def __init__(self, th=None, v=None):
        Module.__init__(self)
        for a in (th, v):
            if a is not None and not isinstance(a, (int, float)):
                raise THGPUError("nn.Threshold(threshold, value)")
        self.threshold = 1e-6 if th is None else th
        self.val = 0 if v is None else v
        # set by Sequential.fuse(): the neighbouring modules do this module's work as they store their results
        self.fusedForward = False
        self.fusedBackward = False

    def updateOutput(self, input):
        if self.fusedForward:
            self.output = input          # the convolution in front has already applied the threshold
            return input
        _require_gpu(input, self.output)
        _lib.check_status(lib.thgpu_Threshold_updateOutput(input._p, self.output._p, self.threshold, self.val))
        return self.output

    def updateGradInput(self, input, gradOutput):
        if self.fusedBackward:
            self.gradInput = gradOutput  # the module behind has already zeroed it where the output is not above the threshold
            return gradOutput
        _require_gpu(input, gradOutput, self.gradInput)
        _lib.check_status(lib.thgpu_Threshold_updateGradInput(input._p, gradOutput._p, self.gradInput._p,
                                                              self.threshold))
        return self.gradInput


class ReLU(Threshold):
    def __init__(self):
        Threshold.__init__(self, 0, 0)


class View(Module):
    """nn.View(sizes...) (mcw_nn/View.lua:1-47): a view of the input with the given sizes, keeping a leading batch
    dimension when the input has one more dimension than setNumInputDims says, or when its per-sample element count
    matches."""

    def __init__(self, *sizes):
        Module.__init__(self)
        if len(sizes) == 1 and not np.isscalar(sizes[0]):
            sizes = tuple(sizes[0])
        self.size = tuple(int(v) for v in sizes)
        self.numElements = int(np.prod(self.size, dtype=np.int64))
        self.output = None
        self.gradInput = None
        self.numInputDims = None

    def setNumInputDims(self, n):
        self.numInputDims = n
        return self

    def _is_minibatch(self, input):
        if self.numInputDims:
            return input.dim() == self.numInputDims + 1
        return input.dim() > 1 and input.nElement() // input.size(0) == self.numElements and \
            input.nElement() % input.size(0) == 0

    def updateOutput(self, input):
        _require_gpu(input)
        if self._is_minibatch(input):
            self.output = input.view(input.size(0), *self.size)
        else:
            self.output = input.view(*self.size)
        return self.output

    def updateGradInput(self, input, gradOutput):
        _require_gpu(input, gradOutput)
        self.gradInput = gradOutput.view(*input.size())
        return self.gradInput


class Reshape(Module):
    """nn.Reshape(sizes..., [batchMode]) (mcw_nn/Reshape.lua:1-70): like View, but a non-contiguous input or
    gradOutput is copied into a dense buffer first."""

    def __init__(self, *args):
        Module.__init__(self)
        args = list(args)
        self.batchMode = None
        if args and isinstance(args[-1], bool):
            self.batchMode = args.pop()
        if len(args) == 1 and not np.isscalar(args[0]):
            args = list(args[0])
        self.size = tuple(int(v) for v in args)
        self.nelement = int(np.prod(self.size, dtype=np.int64))
        self._input = FloatTensor()
        self._gradOutput = FloatTensor()

    def updateOutput(self, input):
        _require_gpu(input, self._input)
        if not input.isContiguous():
            self._input.resizeAs(input)
            self._input.copy(input)
            input = self._input
        if self.batchMode is False or (self.batchMode is None and input.nElement() == self.nelement and
                                       input.size(0) != 1):
            self.output = input.view(*self.size)
        else:
            self.output = input.view(input.size(0), *self.size)
        return self.output

    def updateGradInput(self, input, gradOutput):
        _require_gpu(input, gradOutput, self._gradOutput)
        if not gradOutput.isContiguous():
            self._gradOutput.resizeAs(gradOutput)
            self._gradOutput.copy(gradOutput)
            gradOutput = self._gradOutput
        self.gradInput = gradOutput.viewAs(input)
        return self.gradInput


class LogSoftMax(Module):
    """nn.LogSoftMax() (mcw_nn/LogSoftMax.lua:1-9): vector or matrix of frames."""

    def updateOutput(self, input):
        _require_gpu(input, self.output)
        _lib.check_status(lib.thgpu_LogSoftMax_updateOutput(input._p, self.output._p))
        return self.output

    def updateGradInput(self, input, gradOutput):
        _require_gpu(gradOutput, self.output, self.gradInput)
        _lib.check_status(lib.thgpu_LogSoftMax_updateGradInput(gradOutput._p, self.output._p, self.gradInput._p))
        return self.gradInput


class Criterion(object):
    """nn.Criterion (mcw_nn/Criterion.lua:1-44)."""

    def __init__(self):
        self.gradInput = FloatTensor()
        self.output = 0

    def forward(self, input, target):
        return self.updateOutput(input, target)

    def backward(self, input, target):
        return self.updateGradInput(input, target)

    def type(self, type_name):
        for key, val in list(self.__dict__.items()):
            self.__dict__[key] = _convert(val, type_name)
        return self

    def gpu(self):
        return self.type("torch.GPUTensor")

    def float(self):
        return self.type("torch.FloatTensor")


class ClassNLLCriterion(Criterion):
    """nn.ClassNLLCriterion() on GPU tensors (mcw_nn/ClassNLLCriterion.lua:3-72): target holds 1-based class numbers,
    one per frame; sizeAverage defaults to true.  Class weights have no GPU implementation in the reference (its Lua
    falls back to element-by-element tensor indexing) and are not accepted here."""

    def __init__(self, weights=None):
        Criterion.__init__(self)
        if weights is not None:
            raise THGPUError("nn.ClassNLLCriterion: class weights are not supported on GPU tensors")
        self.sizeAverage = True
        self.outputTensor = FloatTensor(1)

    def updateOutput(self, input, target):
        _require_gpu(input, target, self.outputTensor)
        _lib.check_status(lib.thgpu_ClassNLLCriterion_updateOutput(input._p, target._p, self.outputTensor._p,
                                                                   1 if self.sizeAverage else 0))
        self.output = float(self.outputTensor[0])
        return self.output

    def updateGradInput(self, input, target):
        _require_gpu(input, target, self.gradInput)
        self.gradInput.resizeAs(input)
        self.gradInput.zero()
        _lib.check_status(lib.thgpu_ClassNLLCriterion_updateGradInput(input._p, target._p, self.gradInput._p,
                                                                      1 if self.sizeAverage else 0))
        return self.gradInput
