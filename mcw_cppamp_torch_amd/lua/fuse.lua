-- gpunn.fuse(net): lets the neighbours of every nn.Threshold / nn.ReLU of an nn.Sequential do its work while they
-- store their own results (see include/thgpu.h, thgpu_SpatialConvolutionMM_updateOutputThreshold and the *Masked
-- entry points).  The Threshold modules stay in place and pass tensors through, so nn.Sequential:updateOutput /
-- :updateGradInput (mcw_nn/Sequential.lua:33-68) and every result downstream are unchanged bit for bit.
-- Needs value <= threshold (true of nn.ReLU, mcw_nn/ReLU.lua:4).  gpunn.unfuse(net) undoes it.
require 'nn'
gpunn = gpunn or {}

local function isa(m, name) return torch.typename(m) == name end
local function threshold(m) return isa(m, 'nn.Threshold') or isa(m, 'nn.ReLU') end

function gpunn.unfuse(net)
   for _, m in ipairs(net.modules) do
      if m.modules then gpunn.unfuse(m) end
      if threshold(m) and (m.fusedForward or m.fusedBackward) then
         m.output = m.output.new()
         m.gradInput = m.gradInput.new()
         m.updateOutput, m.updateGradInput = nil, nil      -- back to the class methods
      end
      m.fusedForward, m.fusedBackward, m.fusedThreshold, m.fusedValue, m.inputThreshold = nil, nil, nil, nil, nil
   end
   return net
end

function gpunn.fuse(net)
   gpunn.unfuse(net)
   local mods = net.modules
   for i, m in ipairs(mods) do
      if m.modules then gpunn.fuse(m) end
      if threshold(m) and m.val <= m.threshold then
         local before, after = mods[i - 1], mods[i + 1]
         if before and isa(before, 'nn.SpatialConvolutionMM') and before.fusedThreshold == nil then
            before.fusedThreshold, before.fusedValue = m.threshold, m.val
            m.fusedForward = true
            m.updateOutput = function(self, input) self.output = input; return input end
         end
         if after and (isa(after, 'nn.SpatialConvolutionMM') or isa(after, 'nn.SpatialMaxPooling')) then
            after.inputThreshold = m.threshold
            m.fusedBackward = true
            m.updateGradInput = function(self, input, gradOutput) self.gradInput = gradOutput; return gradOutput end
         end
      end
   end
   return net
end
