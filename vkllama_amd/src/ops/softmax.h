// Softmax: interface of the reference's src/ops/softmax.h:14-32.
#ifndef __VKLLAMA_SOFTMAX_H__
#define __VKLLAMA_SOFTMAX_H__
#include "src/ops/op.h"

namespace vkllama
{
class Softmax : public Op
{
public:
  Softmax (GPUDevice *dev, Command *command, bool seq_mask = false,
           const float temp = 1.0, Tensor::DType const dtype = FP16);
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  absl::StatusOr<Tensor> operator() (Tensor a, size_t offset = 0) noexcept;

private:
  bool seq_mask_;
  Tensor::DType dtype_;
  float temp_; // stored and unused, as in the reference (softmax.cpp:15-18)
  Tensor out_;
};
}
#endif
