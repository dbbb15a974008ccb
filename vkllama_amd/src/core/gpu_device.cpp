#include "src/core/gpu_device.h"
#include "absl/strings/str_format.h"
#include "vkl_hip.h"
#include <stdlib.h>

namespace vkllama
{
GPUDevice::GPUDevice (int dev)
    : dev_ (dev), stream_ (nullptr), compute_units_ (0), wavefront_ (64),
      total_mem_ (0), timing_ (false)
{
}

GPUDevice::~GPUDevice ()
{
  if (stream_)
    {
      vkl_stream_sync (stream_);
      trim ();
      vkl_stream_destroy (stream_);
    }
}

namespace
{
// size classes: 256 B steps below 1 MiB, 64 KiB steps above
size_t
size_class (size_t bytes)
{
  if (bytes == 0)
    bytes = 1;
  const size_t step = bytes < ((size_t)1 << 20) ? 256 : ((size_t)64 << 10);
  return (bytes + step - 1) / step * step;
}
constexpr size_t kPoolLimit = (size_t)8 << 30;  // bytes kept for reuse
constexpr size_t kPoolBlockMax = (size_t)1 << 30; // larger blocks go straight back
}

int
GPUDevice::alloc (void **p, size_t bytes, bool host_visible)
{
  const size_t cls = size_class (bytes);
  auto it = pool_.find ({ cls, host_visible });
  if (it != pool_.end () && !it->second.empty ())
    {
      *p = it->second.back ();
      it->second.pop_back ();
      pooled_bytes_ -= cls;
      return 0;
    }
  int e = host_visible ? vkl_host_malloc_h (p, cls) : vkl_malloc (p, cls);
  if (e && pooled_bytes_)
    {
      // out of memory with blocks parked in the pool: give them back, retry
      vkl_stream_sync (stream_);
      trim ();
      e = host_visible ? vkl_host_malloc_h (p, cls) : vkl_malloc (p, cls);
    }
  return e;
}

void
GPUDevice::release (void *p, size_t bytes, bool host_visible)
{
  if (!p)
    return;
  const size_t cls = size_class (bytes);
  if (cls > kPoolBlockMax || pooled_bytes_ + cls > kPoolLimit)
    {
      if (host_visible)
        vkl_host_free_h (p);
      else
        vkl_free (p);
      return;
    }
  pool_[{ cls, host_visible }].push_back (p);
  pooled_bytes_ += cls;
}

void
GPUDevice::trim ()
{
  for (auto &kv : pool_)
    {
      for (void *p : kv.second)
        {
          if (kv.first.second)
            vkl_host_free_h (p);
          else
            vkl_free (p);
        }
      kv.second.clear ();
    }
  pooled_bytes_ = 0;
}

absl::Status
GPUDevice::init ()
{
  vkl_device_info info;
  if (int e = vkl_device_open (dev_, &info))
    return absl::InternalError (absl::StrFormat (
        "GPUDevice: cannot open HIP device %d: %s", dev_,
        vkl_error_string (e)));
  compute_units_ = info.compute_units;
  wavefront_ = info.wavefront_size;
  total_mem_ = info.total_mem;
  name_ = info.name;
  if (wavefront_ != 64)
    return absl::InternalError (absl::StrFormat (
        "GPUDevice: kernels are written for wave64, device reports %d",
        wavefront_));
  if (int e = vkl_stream_create (&stream_))
    return absl::InternalError (absl::StrFormat (
        "GPUDevice: cannot create stream: %s", vkl_error_string (e)));
  const char *t = getenv ("VKLLAMA_OP_TIMING");
  timing_ = t && t[0] == '1';
  return absl::OkStatus ();
}

bool GPUDevice::support_descriptor_templ_update () const { return true; }
bool GPUDevice::support_16bit_storage () const { return true; }
bool GPUDevice::support_8bit_storage () const { return true; }
bool GPUDevice::support_fp16_arithmetic () const { return false; }
bool GPUDevice::support_int8_arithmetic () const { return true; }
bool GPUDevice::support_pipeline_statistics () const { return timing_; }
size_t GPUDevice::subgroup_size () const { return (size_t)wavefront_; }
}
