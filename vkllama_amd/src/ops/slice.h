// Slice: interface of the reference's src/ops/slice.h:13-29.
#ifndef __VKLLAMA_SLICE_H__
#define __VKLLAMA_SLICE_H__
#include "src/ops/op.h"
#include <array>

namespace vkllama
{
class Slice : public Op
{
public:
  Slice (GPUDevice *gpu, Command *command, Tensor::DType dtype);
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  absl::StatusOr<Tensor> operator() (
      Tensor in, const std::array<uint32_t, 3> &starts,
      const std::array<uint32_t, 3> &extents) noexcept;

private:
  Tensor::DType dtype_;
  Tensor out_;
};
}
#endif
