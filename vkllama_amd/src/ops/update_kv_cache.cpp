// Follows src/ops/update_kv_cache.cpp:15-76 of the reference:
// cache[c, (offset + y) % cache.height, :] = kv[c, y, :].
#include "src/ops/update_kv_cache.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
UpdateKVCache::UpdateKVCache (GPUDevice *gpu, Command *command,
                              const Tensor::DType dtype)
    : Op (gpu, command), dtype_ (dtype)
{
}

absl::Status
UpdateKVCache::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "UpdateKVCache op: only fp16 is supported.");
  return absl::OkStatus ();
}

uint64_t
UpdateKVCache::time () noexcept
{
  return timer_.micros ();
}

absl::Status
UpdateKVCache::operator() (Tensor cache, Tensor key_or_value,
                           const uint32_t offset) noexcept
{
  if (cache.height () < key_or_value.height ()
      || cache.channels () < key_or_value.channels ()
      || cache.width () != key_or_value.width ())
    return absl::OutOfRangeError (
        absl::StrFormat ("size of value is larger than cache. value.shape = "
                         "(%zu, %zu, %zu), cache.shape = (%zu, %zu, %zu)",
                         key_or_value.channels (), key_or_value.height (),
                         key_or_value.width (), cache.channels (),
                         cache.height (), cache.width ()));
  if (cache.dtype () != dtype_ || key_or_value.dtype () != dtype_)
    return absl::InvalidArgumentError (
        "UpdateKVCache op: cache and value must be fp16");
  timer_.start (dev_);
  const int err = vkl_kv_update_f16 (
      cache.data (), key_or_value.data (), (int)key_or_value.channels (),
      (int)cache.height (), (int)key_or_value.height (),
      (int)key_or_value.width (), offset, dev_->stream ());
  timer_.stop (dev_);
  return launch_status ("update_kv_cache", err);
}
}
