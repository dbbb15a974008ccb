// ArgOp / ArgMax / ArgMin: interface of the reference's src/ops/argop.h:13-156.
// The index of the first maximum (op 0) or minimum (op 1) of every row; the
// reference's two-stage reduction also lets the lowest index win ties
// (src/shaders/argmax_stage0_fp16.comp:69-76, argmax_stage1.comp:44).
#ifndef __VKLLAMA_ARGMAX_H__
#define __VKLLAMA_ARGMAX_H__
#include "src/core/command.h"
#include "src/ops/op.h"
#include "vkl_hip.h"

namespace vkllama
{
template <int op_type> class ArgOp : public Op
{
public:
  ArgOp (GPUDevice *gpu, Command *command, const Tensor::DType dtype = FP16)
      : Op (gpu, command), dtype_ (dtype)
  {
  }

  absl::Status
  init () noexcept override
  {
    if (dtype_ != FP16)
      return absl::InvalidArgumentError (
          absl::StrFormat ("dtype %i is unsupported", int (dtype_)));
    return absl::OkStatus ();
  }

  absl::StatusOr<Tensor>
  operator() (Tensor in) noexcept
  {
    if (in.dtype () != dtype_)
      return absl::InvalidArgumentError (
          absl::StrFormat ("operator defined as %d dtype but %d given.",
                           int (dtype_), int (in.dtype ())));
    Tensor out (in.channels (), in.height (), 1, dev_, UINT32);
    VKLLAMA_STATUS_OK (out.create ());
    timer_.start (dev_);
    const int err = vkl_argop_f16 (
        in.data (), (int)(in.channels () * in.height ()), (int)in.width (),
        op_type, (uint32_t *)out.data (), dev_->stream ());
    timer_.stop (dev_);
    VKLLAMA_STATUS_OK (launch_status ("argop", err));
    return out;
  }

  uint64_t
  time () noexcept override
  {
    return timer_.micros ();
  }

private:
  Tensor::DType dtype_;
};

using ArgMax = ArgOp<0>;
using ArgMin = ArgOp<1>;
}
#endif
