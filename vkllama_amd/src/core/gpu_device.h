// GPUDevice: interface of the reference's src/core/gpu_device.h:13-37 with the
// Vulkan instance/device/allocator replaced by a HIP device and ONE in-order
// stream (the reference submits every command buffer to queue 0 of one queue
// family, src/core/command.h:42-44, so a single stream keeps its ordering).
#ifndef __VKLLAMA_CPP_GPU_DEVICE_H__
#define __VKLLAMA_CPP_GPU_DEVICE_H__
#include "absl/status/status.h"
#include <map>
#include <stddef.h>
#include <string>
#include <utility>
#include <vector>

namespace vkllama
{
class GPUDevice
{
public:
  GPUDevice (int dev = 0);
  ~GPUDevice ();
  GPUDevice (const GPUDevice &) = delete;
  GPUDevice &operator= (const GPUDevice &) = delete;

  absl::Status init ();
  bool support_descriptor_templ_update () const;
  bool support_16bit_storage () const;
  bool support_8bit_storage () const;
  // false: products are formed in fp32 (the reference's non-"fp16a" shader
  // variants, src/ops/mat_mul.cpp:75-97 pick by this flag)
  bool support_fp16_arithmetic () const;
  bool support_int8_arithmetic () const;
  // true when per-op event timing is on (environment VKLLAMA_OP_TIMING=1)
  bool support_pipeline_statistics () const;
  size_t subgroup_size () const;

  // HIP-side accessors
  void *stream () const { return stream_; }
  int device_id () const { return dev_; }
  int compute_units () const { return compute_units_; }
  size_t total_memory () const { return total_mem_; }
  const std::string &name () const { return name_; }

  // Pooled memory for tensors (the job VMA does in the reference,
  // src/core/allocator.cpp): freed blocks are kept by size class and handed
  // out again, so that the operator chain does not pay a driver allocation
  // and release per intermediate tensor and pass.  All work runs on the one
  // in-order stream, so a block reused by a later launch cannot be written
  // before earlier launches have finished reading it.
  int alloc (void **p, size_t bytes, bool host_visible);
  void release (void *p, size_t bytes, bool host_visible);
  // returns pooled blocks to the driver
  void trim ();

private:
  const int dev_;
  void *stream_;
  int compute_units_;
  int wavefront_;
  size_t total_mem_;
  bool timing_;
  std::string name_;
  std::map<std::pair<size_t, bool>, std::vector<void *>> pool_;
  size_t pooled_bytes_ = 0;
};
}
#endif
