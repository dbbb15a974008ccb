// Follows src/ops/rms_norm.cpp:23-91 of the reference: fp16 activations,
// FP32 weights required, output cached per instance.
#include "src/ops/rms_norm.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
RMSNorm::RMSNorm (GPUDevice *dev, Command *command, Tensor weight,
                  const float eps, const Tensor::DType dtype)
    : Op (dev, command), weight_ (weight), dtype_ (dtype), eps_ (eps)
{
}

absl::Status
RMSNorm::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "RMSNorm op: only fp16 dtype is supported.");
  if (weight_.dtype () != FP32)
    return absl::InvalidArgumentError (absl::StrFormat (
        "rms_norm op defined with %d dtype but the dtype of weight is %d",
        int (dtype_), int (weight_.dtype ())));
  return absl::OkStatus ();
}

uint64_t
RMSNorm::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
RMSNorm::operator() (Tensor x) noexcept
{
  if (x.dtype () != dtype_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "rms_norm op defined with %d dtype but the dtype of input0 is %d",
        int (dtype_), int (x.dtype ())));
  if (weight_.size () < x.width ())
    return absl::InvalidArgumentError (absl::StrFormat (
        "rms_norm weight has %zu elements but input0 width is %zu",
        weight_.size (), x.width ()));
  if (out_.channels () != x.channels () || out_.height () != x.height ()
      || out_.width () != x.width ())
    {
      out_ = Tensor (x.channels (), x.height (), x.width (), dev_, dtype_,
                     false);
      VKLLAMA_STATUS_OK (out_.create ());
    }
  timer_.start (dev_);
  const int err = vkl_rmsnorm_f16 (
      x.data (), (const float *)weight_.data (),
      (int)(x.channels () * x.height ()), (int)x.width (), eps_, out_.data (),
      dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("rms_norm", err));
  return out_;
}
}
