// Follows src/ops/read_kvcache_op.cpp:9-71 of the reference: `len` rows of
// every channel of a ring cache [C, H, W], starting at row offset % H.
#include "src/ops/read_kvcache_op.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
ReadKVCache::ReadKVCache (GPUDevice *gpu, Command *command) : Op (gpu, command)
{
}

absl::Status
ReadKVCache::init () noexcept
{
  return absl::OkStatus ();
}

uint64_t
ReadKVCache::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
ReadKVCache::operator() (Tensor cache, uint32_t offset, uint32_t len) noexcept
{
  if (len > cache.height ())
    return absl::OutOfRangeError (absl::StrFormat (
        "read %d len but size of cache is %zu", int (len), cache.height ()));
  if (cache.dtype () != FP16)
    return absl::InvalidArgumentError ("ReadKVCache: only fp16 caches");
  auto out = Tensor (cache.channels (), len, cache.width (), dev_,
                     cache.dtype (), false);
  VKLLAMA_STATUS_OK (out.create ());
  if (out.size () == 0)
    return out;
  timer_.start (dev_);
  const int err = vkl_read_kvcache_f16 (
      cache.data (), (int)cache.channels (), (int)cache.height (),
      (int)cache.width (), offset, len, out.data (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("read_kvcache", err));
  return out;
}
}
