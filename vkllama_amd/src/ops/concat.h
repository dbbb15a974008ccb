// Concat: interface of the reference's src/ops/concat.h:10-27.
#ifndef __VKLLAMA_CONCAT_H__
#define __VKLLAMA_CONCAT_H__
#include "src/ops/op.h"
#include <vector>

namespace vkllama
{
class Concat : public Op
{
public:
  Concat (GPUDevice *gpu, Command *command, const int num, const int axis,
          Tensor::DType const dtype = FP16);
  absl::Status init () noexcept override;
  absl::StatusOr<Tensor>
  operator() (std::vector<Tensor> const &inputs) noexcept;
  uint64_t time () noexcept override;

private:
  const int num_;
  int axis_;
  Tensor::DType dtype_;
  Tensor out_;
};
}
#endif
