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
      vkl_stream_destroy (stream_);
    }
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
