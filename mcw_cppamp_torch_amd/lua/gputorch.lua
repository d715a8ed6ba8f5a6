-- gputorch on libthgpu: the Lua half of the tensor package.  Loaded as the package's init.lua in place of the
-- reference's gputorch/init.lua:1-11, Tensor.lua:1-47 and FFI.lua:1-50; the C half is lua/gputorch_glue.cpp
-- (luaopen_libgputorch).
require 'torch'
gputorch = require 'libgputorch'

torch.GPUStorage.__tostring__ = torch.FloatStorage.__tostring__
torch.GPUTensor.__tostring__ = torch.FloatTensor.__tostring__

local GPUTensor = torch.getmetatable('torch.GPUTensor')

-- Type conversion: tensor:type(name) makes a tensor of the named class with the same sizes and copies into it
-- (the :copy of every class accepts every other, see the glue); :gpu() / :float() / :double() name the class.
local function convert(self, name)
   local current = torch.typename(self)
   if not name then return current end
   if name == current then return self end
   local made = torch.getmetatable(name).new()
   if self:nElement() > 0 then made:resize(self:size()):copy(self) end
   return made
end
local function to_gpu(self) return self:type('torch.GPUTensor') end

rawset(GPUTensor, 'type', convert)
rawset(GPUTensor, 'typeAs', function(self, other) return self:type(other:type()) end)
rawset(GPUTensor, 'gpu', to_gpu)
rawset(GPUTensor, 'float', function(self) return self:type('torch.FloatTensor') end)
rawset(GPUTensor, 'double', function(self) return self:type('torch.DoubleTensor') end)
rawset(torch.getmetatable('torch.FloatTensor'), 'gpu', to_gpu)
rawset(torch.getmetatable('torch.DoubleTensor'), 'gpu', to_gpu)

-- Element-wise callbacks run on the host: the values make a round trip through a FloatTensor (the binding template's
-- own apply / map / map2 walk host pointers, which device memory does not offer).
local function staged(self) return torch.FloatTensor(self:size()):copy(self) end
rawset(GPUTensor, 'apply', function(self, func)
   local host = staged(self)
   host:apply(func)
   return self:copy(host)
end)
rawset(GPUTensor, 'map', function(self, other, func)
   local host = staged(self)
   host:map(staged(other), func)
   return self:copy(host)
end)
rawset(GPUTensor, 'map2', function(self, a, b, func)
   local host = staged(self)
   host:map2(staged(a), staged(b), func)
   return self:copy(host)
end)

-- The shape helpers torch defines on top of the class methods.
for _, name in ipairs{'expand', 'expandAs', 'view', 'viewAs', 'repeatTensor'} do
   rawset(GPUTensor, name, torch[name])
end

-- LuaJIT: direct views of the two structs (their layout is part of the library's ABI; `data` is a DEVICE pointer,
-- to be handed to kernels, never dereferenced from Lua).
if jit then
   local ffi = require 'ffi'
   ffi.cdef[[
typedef struct THGPUStorage {
    float *data;
    long size;
    int refcount;
    char flag;
    THAllocator *allocator;
    void *allocatorContext;
} THGPUStorage;
typedef struct THGPUTensor {
    long *size;
    long *stride;
    int nDimension;
    THGPUStorage *storage;
    long storageOffset;
    int refcount;
    char flag;
} THGPUTensor;
]]
   local GPUStorage = torch.getmetatable('torch.GPUStorage')
   local storage_pp, tensor_pp = ffi.typeof('THGPUStorage**'), ffi.typeof('THGPUTensor**')
   rawset(GPUStorage, 'cdata', function(self) return storage_pp(self)[0] end)
   rawset(GPUStorage, 'data', function(self) return storage_pp(self)[0].data end)
   rawset(GPUTensor, 'cdata', function(self) return tensor_pp(self)[0] end)
   rawset(GPUTensor, 'data', function(self)
      local t = tensor_pp(self)[0]
      if t.storage == nil then return nil end
      return t.storage.data + t.storageOffset
   end)
end

return gputorch
