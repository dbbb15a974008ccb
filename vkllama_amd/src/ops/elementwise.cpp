// Follows src/ops/elementwise.cpp of the reference.  The tensor-scalar form
// is given a launch here (the reference never sets its dispatch size,
// src/ops/elementwise.cpp:104-133).
#include "src/ops/elementwise.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
ElementWise::ElementWise (GPUDevice *dev, Command *command, const int type,
                          Tensor::DType dtype)
    : Op (dev, command), type_ (type), dtype_ (dtype)
{
}

absl::Status
ElementWise::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "ElementWise op: only fp16 is supported");
  if (type_ < 0 || type_ > 3)
    return absl::InvalidArgumentError (
        absl::StrFormat ("ElementWise op: type %d is unsupported", type_));
  return absl::OkStatus ();
}

uint64_t
ElementWise::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
ElementWise::operator() (Tensor x, Tensor y) noexcept
{
  if (x.dtype () != y.dtype () || x.dtype () != dtype_)
    return absl::InvalidArgumentError (
        "elementwise op: x.dtype() != y.dtype()");
  if (x.channels () != y.channels () || x.height () != y.height ()
      || x.width () != y.width ())
    return absl::InvalidArgumentError (
        absl::StrFormat ("elementwise op: shape error. shape of x = (%zu, "
                         "%zu, %zu), y = (%zu, %zu, %zu)",
                         x.channels (), x.height (), x.width (),
                         y.channels (), y.height (), y.width ()));
  timer_.start (dev_);
  const int err = vkl_elementwise_f16 (x.data (), y.data (), x.size (), type_,
                                       dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("elementwise", err));
  return y;
}

absl::StatusOr<Tensor>
ElementWise::operator() (Tensor x, float y) noexcept
{
  if (x.dtype () != dtype_)
    return absl::InvalidArgumentError (
        "elementwise op: x.dtype() differs from the op's dtype");
  timer_.start (dev_);
  const int err = vkl_elementwise_const_f16 (x.data (), y, x.size (), type_,
                                             x.data (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("elementwise", err));
  return x;
}
}
