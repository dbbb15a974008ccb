#include "src/ops/op.h"
#include "src/core/command.h"
#include "src/core/gpu_device.h"
#include "vkl_hip.h"

namespace vkllama
{
OpTimer::OpTimer () : ev0_ (nullptr), ev1_ (nullptr), recorded_ (false) {}

OpTimer::~OpTimer ()
{
  if (ev0_)
    vkl_event_destroy (ev0_);
  if (ev1_)
    vkl_event_destroy (ev1_);
}

void
OpTimer::start (GPUDevice *dev)
{
  if (!dev->support_pipeline_statistics ())
    return;
  if (!ev0_ && (vkl_event_create (&ev0_) || vkl_event_create (&ev1_)))
    return;
  vkl_event_record (ev0_, dev->stream ());
}

void
OpTimer::stop (GPUDevice *dev)
{
  if (!dev->support_pipeline_statistics () || !ev1_)
    return;
  vkl_event_record (ev1_, dev->stream ());
  recorded_ = true;
}

uint64_t
OpTimer::micros ()
{
  if (!recorded_)
    return 0;
  float ms = 0.f;
  if (vkl_event_sync (ev1_) || vkl_event_elapsed_ms (ev0_, ev1_, &ms))
    return 0;
  return (uint64_t)(ms * 1000.0f);
}

Op::Op (GPUDevice *dev, Command *command) noexcept
    : dev_ (dev), command_ (command)
{
}

absl::Status
Op::launch_status (const char *what, int err)
{
  if (err == 0)
    return absl::OkStatus ();
  if (err == 1) // hipErrorInvalidValue: rejected before any launch
    return absl::InvalidArgumentError (
        absl::StrFormat ("%s: shapes rejected by the HIP layer", what));
  return absl::InternalError (
      absl::StrFormat ("%s: %s", what, vkl_error_string (err)));
}
}
