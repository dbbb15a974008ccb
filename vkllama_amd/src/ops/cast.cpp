// Follows src/ops/cast.cpp:13-77 of the reference (fp32<->fp16 only).  The
// output tensor is reused while the shape stays the same.
#include "src/ops/cast.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
Cast::Cast (GPUDevice *dev, Command *command, const Tensor::DType from,
            const Tensor::DType to)
    : Op (dev, command), from_ (from), to_ (to)
{
}

absl::Status
Cast::init () noexcept
{
  if (!((from_ == FP32 && to_ == FP16) || (from_ == FP16 && to_ == FP32)))
    return absl::InvalidArgumentError (
        "only fp32 -> fp16 and fp16 -> fp32 are supported.");
  return absl::OkStatus ();
}

uint64_t
Cast::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
Cast::operator() (Tensor from) noexcept
{
  if (from.dtype () != from_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "operator defined as casting from %d dtype but %d given",
        int (from_), int (from.dtype ())));
  if (out_.channels () != from.channels () || out_.height () != from.height ()
      || out_.width () != from.width ())
    {
      out_ = Tensor (from.channels (), from.height (), from.width (), dev_,
                     to_);
      VKLLAMA_STATUS_OK (out_.create ());
    }
  timer_.start (dev_);
  const int err
      = from_ == FP16
            ? vkl_cast_f16_f32 (from.data (), (float *)out_.data (),
                                from.size (), dev_->stream ())
            : vkl_cast_f32_f16 ((const float *)from.data (), out_.data (),
                                from.size (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("cast", err));
  return out_;
}
}
