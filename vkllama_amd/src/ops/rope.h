// Rope: interface of the reference's src/ops/rope.h:15-34.
#ifndef __VKLLAMA_ROPE_H__
#define __VKLLAMA_ROPE_H__

#include "src/core/float.h"
#include "src/core/tensor.h"
#include "src/ops/op.h"
#include <vector>

namespace vkllama
{
class Rope : public Op
{
public:
  Rope (GPUDevice *dev, Command *command, const int maxlen, const int dim,
        const Tensor::DType dtype = FP16);

  absl::StatusOr<Tensor> operator() (Tensor query,
                                     const size_t offset = 0) noexcept;
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  // cos / sin tables, fp32 [maxlen, dim/2]
  Tensor &freqc () { return freqc_; }
  Tensor &freqs () { return freqs_; }
  // host computation of the tables (src/ops/rope.cpp:19-47)
  static void compute_freq (size_t dim, size_t maxlen,
                            std::vector<float> &freqc,
                            std::vector<float> &freqs);

private:
  const int maxlen_;
  const int dim_;
  const Tensor::DType dtype_;
  Tensor freqc_;
  Tensor freqs_;
};
}
#endif
