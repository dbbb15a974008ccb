// RMSNorm: interface of the reference's src/ops/rms_norm.h:12-28.
#ifndef __VKLLAMA_RMSNORM_H__
#define __VKLLAMA_RMSNORM_H__
#include "src/core/tensor.h"
#include "src/ops/op.h"

namespace vkllama
{
class RMSNorm : public Op
{
public:
  RMSNorm (GPUDevice *dev, Command *command, Tensor weight,
           const float eps = 1e-3, const Tensor::DType dtype = FP16);
  absl::StatusOr<Tensor> operator() (Tensor a) noexcept;
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  // for fused callers
  Tensor &weight () { return weight_; }
  float eps () const { return eps_; }

private:
  Tensor weight_;
  Tensor::DType dtype_;
  float eps_;
  Tensor out_;
};
}
#endif
