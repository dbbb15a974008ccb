// FeedForward: interface of the reference's src/ops/feed_forward.h:17-35.
// w1 = gate, w2 = down, w3 = up (models/llama2.h:633-640).
#ifndef __VKLLAMA_FEED_FORWARD__
#define __VKLLAMA_FEED_FORWARD__

#include "src/core/tensor.h"
#include "src/ops/elementwise.h"
#include "src/ops/mat_mul.h"
#include "src/ops/op.h"
#include <memory>

namespace vkllama
{
class FeedForward : public Op
{
public:
  FeedForward (GPUDevice *, Command *, Tensor, Tensor, Tensor,
               const bool transposed_weight = false,
               const Tensor::DType dtype = FP16);
  absl::StatusOr<Tensor> operator() (Tensor X) noexcept;
  // the next call only: the residual is added in the down projection's launch
  void set_residual (const Tensor *r) noexcept { residual_ = r; }
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  Tensor &w1 () { return w1_; }
  Tensor &w2 () { return w2_; }
  Tensor &w3 () { return w3_; }

private:
  const Tensor *residual_ = nullptr;
  Tensor t0_;
  Tensor w1_;
  Tensor w2_;
  Tensor w3_;
  std::unique_ptr<MatMul> down_op_;
  Tensor::DType dtype_;
  bool transposed_weight_;
  bool inited_;
};
}
#endif
