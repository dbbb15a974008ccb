// Cast: interface of the reference's src/ops/cast.h:15-31.
#ifndef __VKLLAMA_CAST_H__
#define __VKLLAMA_CAST_H__
#include "src/ops/op.h"

namespace vkllama
{
class Cast : public Op
{
public:
  Cast (GPUDevice *dev, Command *command, const Tensor::DType from,
        const Tensor::DType to);
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  absl::StatusOr<Tensor> operator() (Tensor from) noexcept;

private:
  Tensor::DType from_;
  Tensor::DType to_;
  Tensor out_;
};
}
#endif
