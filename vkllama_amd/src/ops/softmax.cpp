// Follows src/ops/softmax.cpp:21-92 of the reference.
#include "src/ops/softmax.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
Softmax::Softmax (GPUDevice *dev, Command *command, bool seq_mask, float temp,
                  const Tensor::DType dtype)
    : Op (dev, command), seq_mask_ (seq_mask), dtype_ (dtype), temp_ (temp)
{
}

absl::Status
Softmax::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "Softmax op: only fp16 dtype is supported");
  return absl::OkStatus ();
}

uint64_t
Softmax::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
Softmax::operator() (Tensor a, size_t offset) noexcept
{
  if (a.dtype () != dtype_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "softmax op defined with %d dtype but input0's dtype = %d",
        int (dtype_), int (a.dtype ())));
  if (out_.channels () != a.channels () || out_.height () != a.height ()
      || out_.width () != a.width ())
    {
      out_ = Tensor::like (a);
      VKLLAMA_STATUS_OK (out_.create ());
    }
  timer_.start (dev_);
  const int err = vkl_softmax_f16 (
      a.data (), (int)a.channels (), (int)a.height (), (int)a.width (),
      seq_mask_ ? 1 : 0, (uint32_t)offset, out_.data (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("softmax", err));
  return out_;
}
}
