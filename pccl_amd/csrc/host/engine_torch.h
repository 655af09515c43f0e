// engine_torch.h -- the at::Tensor form of Engine::exeOp, header-only.
//
// The reference declares `void exeOp(const std::string &name, at::Tensor &input,
// at::Tensor output)` (include/engine.h:19) and exposes it to Python unchanged
// (csrc/python_api.cc:17).  The engine of this build takes raw device addresses so that
// libpccl_engine.so needs neither torch nor HIP headers; a caller that has torch includes
// this header and gets the reference's signature as a free function and as a thin class.
// The stream is torch's current HIP stream of the input tensor's device, like the
// reference's CUDA plugin takes the device from the current torch stream
// (csrc/plugins/cuda_executor/device.cc:63).
#pragma once

#include <ATen/Tensor.h>
#include <c10/hip/HIPStream.h>
#include <c10/util/Exception.h>

#include <string>

#include "engine.h"

namespace engine_c {

inline void exeOp(Engine &engine, const std::string &name, at::Tensor &input, at::Tensor output) {
  TORCH_CHECK(input.is_cuda() && output.is_cuda(), "exeOp: input and output must be device tensors");
  TORCH_CHECK(input.is_contiguous() && output.is_contiguous(), "exeOp: input and output must be contiguous");
  TORCH_CHECK(input.get_device() == output.get_device(), "exeOp: input and output live on different devices");
  void *stream = (void *)c10::hip::getCurrentHIPStream(input.get_device()).stream();
  engine.exeOp(name, input.data_ptr(), output.data_ptr(), (long)input.nbytes(), (long)output.nbytes(), stream);
}

// Engine with the reference's exact method set, for code written against include/engine.h.
class TorchEngine : public Engine {
public:
  using Engine::Engine;
  using Engine::exeOp;
  void exeOp(const std::string &name, at::Tensor &input, at::Tensor output) {
    engine_c::exeOp(*this, name, input, output);
  }
};

}  // namespace engine_c
