// Op base class: interface of the reference's src/ops/op.h:14-25.
#ifndef __VKLLAMA_OP_H__
#define __VKLLAMA_OP_H__

#include "absl/status/status.h"
#include "absl/status/statusor.h"
#include "absl/strings/str_format.h"
#include "src/core/tensor.h"
#include <stdint.h>

namespace vkllama
{
class GPUDevice;
class Command;

// Event pair around an operator's launches; the counterpart of the
// reference's per-pipeline timestamp queries (src/core/pipeline.cpp:425-445).
// Active only when GPUDevice::support_pipeline_statistics() is true.
class OpTimer
{
public:
  OpTimer ();
  ~OpTimer ();
  OpTimer (const OpTimer &) = delete;
  OpTimer &operator= (const OpTimer &) = delete;
  void start (GPUDevice *dev);
  void stop (GPUDevice *dev);
  // microseconds of the last recorded span; waits for it to finish
  uint64_t micros ();

private:
  void *ev0_, *ev1_;
  bool recorded_;
};

class Op
{
public:
  Op (GPUDevice *dev, Command *command) noexcept;
  virtual absl::Status init () noexcept = 0;
  virtual uint64_t time () noexcept = 0;
  virtual ~Op (){};

protected:
  // maps a vkl_* return code to a Status
  static absl::Status launch_status (const char *what, int err);
  GPUDevice *dev_;
  Command *command_;
  OpTimer timer_;
};

}

#endif
