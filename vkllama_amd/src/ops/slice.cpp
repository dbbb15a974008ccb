// Follows src/ops/slice.cpp:13-77 of the reference.
#include "src/ops/slice.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
Slice::Slice (GPUDevice *gpu, Command *command, Tensor::DType dtype)
    : Op (gpu, command), dtype_ (dtype)
{
}

absl::Status
Slice::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "Slice op: only fp16 dtype is supported");
  return absl::OkStatus ();
}

uint64_t
Slice::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
Slice::operator() (Tensor in, const std::array<uint32_t, 3> &starts,
                   const std::array<uint32_t, 3> &extents) noexcept
{
  if (starts[0] + extents[0] > in.channels ()
      || starts[1] + extents[1] > in.height ()
      || starts[2] + extents[2] > in.width ())
    return absl::OutOfRangeError (absl::StrFormat (
        "slice starts = (%zu, %zu, %zu) from (%zu, %zu, %zu) shape tensor",
        size_t (starts[0]), size_t (starts[1]), size_t (starts[2]),
        in.channels (), in.height (), in.width ()));
  if (in.dtype () != dtype_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "slice op defined with %d dtype but the dtype of input0 is %d",
        int (dtype_), int (in.dtype ())));
  if (out_.channels () != extents[0] || out_.height () != extents[1]
      || out_.width () != extents[2])
    {
      out_ = Tensor (extents[0], extents[1], extents[2], dev_, dtype_);
      VKLLAMA_STATUS_OK (out_.create ());
    }
  if (out_.size () == 0)
    return out_;
  timer_.start (dev_);
  const int err = vkl_slice_f16 (
      in.data (), (int)in.channels (), (int)in.height (), (int)in.width (),
      (int)starts[0], (int)starts[1], (int)starts[2], (int)extents[0],
      (int)extents[1], (int)extents[2], out_.data (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("slice", err));
  return out_;
}
}
