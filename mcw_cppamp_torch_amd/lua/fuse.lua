-- gpunn.fuse(net): lets the neighbours of every nn.Threshold / nn.ReLU of an nn.Sequential do its work while they
-- store their own results (see include/thgpu.h, thgpu_SpatialConvolutionMM_updateOutputFused / _updateGradInputFused
-- and thgpu_SpatialMaxPooling_updateGradInputMasked).  The Threshold modules stay in place and pass tensors through, so nn.Sequential:updateOutput /
-- :updateGradInput (mcw_nn/Sequential.lua:33-68) and every result downstream are unchanged bit for bit.
-- Needs value <= threshold (true of nn.ReLU, mcw_nn/ReLU.lua:4).  gpunn.unfuse(net) undoes it.
require 'nn'
gpunn = gpunn or {}

local function isa(m, name) return torch.typename(m) == name end
local function threshold(m) return isa(m, 'nn.Threshold') or isa(m, 'nn.ReLU') end

-- The layer in front of a convolution that gathers from its padded input writes that padded image itself: before
-- every forward pass its `output` is made a view into a zero-bordered buffer of the right size (the operators leave an
-- output that already has the right sizes as it is), and the convolution is told so (inputInPaddedBuffer).
local function output_sizes(m, input)
   local n = input:dim()
   local H, W = input:size(n - 1), input:size(n)
   if isa(m, 'nn.SpatialConvolutionMM') then
      local pW, pH = m.padW or m.padding, m.padH or m.padding
      return m.nOutputPlane, math.floor((H + 2 * pH - m.kH) / m.dH) + 1, math.floor((W + 2 * pW - m.kW) / m.dW) + 1
   end
   return input:size(n - 2), math.floor((H - m.kH) / m.dH) + 1, math.floor((W - m.kW) / m.dW) + 1
end

local function link(producer, consumer)
   local class_updateOutput = producer.updateOutput
   producer.updateOutput = function(self, input)
      local C, H, W = output_sizes(self, input)
      local B = input:dim() == 4 and input:size(1) or 1
      local pW, pH = consumer.padW or consumer.padding, consumer.padH or consumer.padding
      local want = (pW > 0 or pH > 0) and H > 0 and W > 0 and thgpu.convGathers(B, C, H, W, consumer.nOutputPlane,
                   consumer.kW, consumer.kH, consumer.dW, consumer.dH, pW, pH)
      if want then
         local b = self.paddedOutput
         if not (b and b:dim() == input:dim() and b:size(b:dim()) == W + 2 * pW and b:size(b:dim() - 1) == H + 2 * pH
                 and b:size(b:dim() - 2) == C and (input:dim() == 3 or b:size(1) == B)) then
            b = input:dim() == 4 and input.new(B, C, H + 2 * pH, W + 2 * pW) or input.new(C, H + 2 * pH, W + 2 * pW)
            b:zero()
            self.paddedOutput = b
            self.output = b:narrow(b:dim() - 1, pH + 1, H):narrow(b:dim(), pW + 1, W)
         end
      else
         if self.paddedOutput then self.output = input.new(); self.paddedOutput = nil end
      end
      return class_updateOutput(self, input)
   end
   producer.linkedConsumer = consumer
   -- The consumer decides call by call whether its input lies in the padded buffer: only the producer's own current
   -- output view does (the very object nn.Sequential hands on, mcw_nn/Sequential.lua:33-68); any other input, e.g.
   -- net:get(i):forward(x) on a tensor of the caller's, takes the ordinary route.
   local function in_padded_buffer(input)
      return producer.paddedOutput ~= nil and rawequal(input, producer.output) or nil
   end
   local consumer_updateOutput, consumer_accGradParameters = consumer.updateOutput, consumer.accGradParameters
   consumer.updateOutput = function(self, input)
      self.inputInPaddedBuffer = in_padded_buffer(input)
      return consumer_updateOutput(self, input)
   end
   consumer.accGradParameters = function(self, input, gradOutput, scale)
      self.inputInPaddedBuffer = in_padded_buffer(input)
      return consumer_accGradParameters(self, input, gradOutput, scale)
   end
   consumer.linkedProducer = producer
end

-- Backward inside a fused container: the module whose gradInput is a convolution's gradOutput (gradConsumer) also
-- stores it in the padded layout that convolution's gradInput product gathers from, through the view
-- SpatialConvolutionMM_gradOutputTwin hands out, and the convolution is told so -- only here, where nothing can touch
-- either copy in between.  The loop is nn.Sequential:updateGradInput's (mcw_nn/Sequential.lua:45-57).
local function fused_updateGradInput(self, input, gradOutput)
   local mods = self.modules
   local current = gradOutput
   local ready_for = nil              -- the convolution whose fgradInput already holds `current` in padded form
   for i = #mods, 1, -1 do
      local m = mods[i]
      local m_input = i > 1 and mods[i - 1].output or input
      local consumer = m.gradConsumer and mods[m.gradConsumer]
      local twin = nil
      if consumer then
         local c_input = m.gradConsumer > 1 and mods[m.gradConsumer - 1].output or input
         consumer.gradOutputTwin = consumer.gradOutputTwin or c_input.new()
         twin = c_input.nn.SpatialConvolutionMM_gradOutputTwin(consumer, c_input)
      end
      m.twinTarget = twin
      m.gradOutputInTwin = (ready_for == m) or nil
      m.wroteTwin = nil
      current = m:updateGradInput(m_input, current)
      local passes_on = threshold(m) and m.fusedBackward
      if twin and m.wroteTwin then ready_for = consumer elseif not passes_on then ready_for = nil end
      m.twinTarget, m.gradOutputInTwin = nil, nil
   end
   self.gradInput = current
   return current
end

function gpunn.unfuse(net)
   net.updateGradInput = nil           -- back to the class method
   for _, m in ipairs(net.modules) do
      m.gradConsumer, m.twinTarget, m.gradOutputInTwin, m.wroteTwin = nil, nil, nil, nil
      if m.modules then gpunn.unfuse(m) end
      if m.linkedConsumer then
         m.linkedConsumer, m.updateOutput = nil, nil
         if m.paddedOutput then m.output = m.output.new(); m.paddedOutput = nil end
      end
      if m.linkedProducer then
         m.linkedProducer, m.inputInPaddedBuffer = nil, nil
         m.updateOutput, m.accGradParameters = nil, nil     -- back to the class methods
      end
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
   for i, m in ipairs(mods) do
      if isa(m, 'nn.SpatialConvolutionMM') or isa(m, 'nn.SpatialMaxPooling') then
         local j = i + 1
         if mods[j] and threshold(mods[j]) and mods[j].fusedForward then j = j + 1 end
         if mods[j] and isa(mods[j], 'nn.SpatialConvolutionMM') then link(m, mods[j]) end
      end
   end
   -- backward: the module whose gradInput reaches a convolution's updateGradInput unchanged
   local any = false
   for i, m in ipairs(mods) do
      if isa(m, 'nn.SpatialConvolutionMM') and m.gradInput then
         local j = i + 1
         if mods[j] and threshold(mods[j]) and mods[j].fusedBackward then j = j + 1 end
         local p = mods[j]
         if p and (isa(p, 'nn.SpatialConvolutionMM') or isa(p, 'nn.SpatialMaxPooling'))
            and (j == i + 1 or p.inputThreshold ~= nil) then
            p.gradConsumer = i
            any = true
         end
      end
   end
   if any then net.updateGradInput = fused_updateGradInput end
   return net
end
