// Transpose: interface of the reference's src/ops/transpose.h:14-30.
#ifndef __VKLLAMA_TRANSPOSE_H__
#define __VKLLAMA_TRANSPOSE_H__
#include "src/ops/op.h"

namespace vkllama
{
class Transpose : public Op
{
public:
  Transpose (GPUDevice *gpu, Command *command, const int type,
             Tensor::DType const dtype = FP16);
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  absl::StatusOr<Tensor> operator() (Tensor in) noexcept;

private:
  Tensor::DType dtype_;
  Tensor out_;
  int trans_type_;
};
}
#endif
