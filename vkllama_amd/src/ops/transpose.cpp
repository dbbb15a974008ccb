// Follows src/ops/transpose.cpp:13-85 of the reference: type 0 maps
// [C, H, W] to [H, C, W]; other types are Unimplemented.
#include "src/ops/transpose.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
Transpose::Transpose (GPUDevice *gpu, Command *command, const int type,
                      Tensor::DType const dtype)
    : Op (gpu, command), dtype_ (dtype), trans_type_ (type)
{
}

absl::Status
Transpose::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "Transpose op: only fp16 is supported.");
  return absl::OkStatus ();
}

uint64_t
Transpose::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
Transpose::operator() (Tensor in) noexcept
{
  if (in.dtype () != dtype_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "transpose op defined with %d dtype but the dtype of input0 is %d",
        int (dtype_), int (in.dtype ())));
  if (trans_type_ != 0)
    return absl::UnimplementedError (
        "only transpose type 0 is supported now.");
  if (out_.channels () != in.height () || out_.height () != in.channels ()
      || out_.width () != in.width ())
    {
      out_ = Tensor (in.height (), in.channels (), in.width (), dev_,
                     in.dtype ());
      VKLLAMA_STATUS_OK (out_.create ());
    }
  if (out_.size () == 0)
    return out_;
  timer_.start (dev_);
  const int err = vkl_transpose102_f16 (
      in.data (), (int)in.channels (), (int)in.height (), (int)in.width (),
      out_.data (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("transpose", err));
  return out_;
}
}
