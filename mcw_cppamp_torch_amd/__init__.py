"""MI355X implementation of the gputorch/gpunn convolution hot path.

    from mcw_cppamp_torch_amd import gputorch, nn
    conv = nn.SpatialConvolutionMM(3, 64, 11, 11, 4, 4, 2).gpu()
    out = conv.forward(gputorch.FloatTensor(x).gpu()).float()

Importing the package loads libthgpu.so (built by `python -m
mcw_cppamp_torch_amd.build`); the import fails if the library is missing.
"""
from . import _lib, gputorch, nn, stacks  # noqa: F401
from ._lib import THGPUError  # noqa: F401
from .gputorch import FloatTensor, GPUStorage, GPUTensor  # noqa: F401
