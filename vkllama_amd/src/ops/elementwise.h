// ElementWise: interface of the reference's src/ops/elementwise.h:16-34.
// type 0..3 = add, sub, mul, div.
#ifndef __VKLLAMA_ELEMENTWISE_H__
#define __VKLLAMA_ELEMENTWISE_H__

#include "src/ops/op.h"

namespace vkllama
{
class ElementWise : public Op
{
public:
  ElementWise (GPUDevice *dev, Command *command_, const int type,
               Tensor::DType dtype = FP16);
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  // y = x op y, written into y, returns y (src/ops/elementwise.cpp:66-101)
  absl::StatusOr<Tensor> operator() (Tensor x, Tensor y) noexcept;
  // x = x op y in place
  absl::StatusOr<Tensor> operator() (Tensor x, float y) noexcept;

private:
  const int type_;
  Tensor::DType dtype_;
};
}
#endif
