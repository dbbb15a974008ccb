// UpdateKVCache: interface of the reference's src/ops/update_kv_cache.h:13-26.
#ifndef __VKLLAMA_UPDATE_KV_CACHE_H__
#define __VKLLAMA_UPDATE_KV_CACHE_H__
#include "src/ops/op.h"

namespace vkllama
{
class UpdateKVCache : public Op
{
public:
  UpdateKVCache (GPUDevice *gpu, Command *command, const Tensor::DType dtype);
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;
  absl::Status operator() (Tensor cache, Tensor key_or_value,
                           const uint32_t offset) noexcept;

private:
  Tensor::DType dtype_;
};
}
#endif
