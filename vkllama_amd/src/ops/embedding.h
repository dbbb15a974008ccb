// Embedding: interface of the reference's src/ops/embedding.h:13-29.
#ifndef __VKLLAMA_EMBEDDING_H__
#define __VKLLAMA_EMBEDDING_H__
#include "src/ops/op.h"

namespace vkllama
{
class Embedding : public Op
{
public:
  Embedding (GPUDevice *dev, Command *command, Tensor vocab,
             const uint32_t UNK, Tensor::DType dtype = FP16);
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  absl::StatusOr<Tensor> operator() (Tensor indices) noexcept;
  Tensor &vocab () { return vocab_; }

private:
  Tensor vocab_;
  Tensor out_;
  const uint32_t UNK_;
  Tensor::DType dtype_;
};
}
#endif
