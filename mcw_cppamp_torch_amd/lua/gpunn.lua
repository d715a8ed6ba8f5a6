-- gpunn on libthgpu: loaded as the package's init.lua in place of the reference's gpunn/init.lua:1-5.  The operators
-- register themselves under torch.GPUTensor's `nn` table when libgpunn is opened (lua/gpunn_glue.cpp), so the Lua
-- modules of nn dispatch to them through input.nn.<Op>_<method> unchanged (mcw_nn/SpatialConvolutionMM.lua:48-60).
require 'gputorch'
require 'nn'
require 'libgpunn'

gpunn = gpunn or {}
torch.include('gpunn', 'fuse.lua')     -- gpunn.fuse(net) / gpunn.unfuse(net)
return gpunn
