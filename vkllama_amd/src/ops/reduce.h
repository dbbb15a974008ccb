// Reduce over the last axis: interface of the reference's src/ops/reduce.h:17-120
// (op_type 0 sum, 1 max, 2 min, 3 mean; [C,H,W] -> [C,H,1]).
#ifndef __VKLLAMA_REDUCE_H__
#define __VKLLAMA_REDUCE_H__
#include "src/core/command.h"
#include "src/ops/op.h"
#include "vkl_hip.h"

namespace vkllama
{
class Reduce : public Op
{
public:
  Reduce (GPUDevice *gpu, Command *command, int op_type,
          Tensor::DType const dtype = FP16)
      : Op (gpu, command), op_type_ (op_type), dtype_ (dtype)
  {
  }

  absl::Status
  init () noexcept override
  {
    if (dtype_ != FP16)
      return absl::InvalidArgumentError (
          "Reduce op: only fp16 dtype is supported");
    if (op_type_ < 0 || op_type_ > 3)
      return absl::InvalidArgumentError (
          absl::StrFormat ("reduce op_type %d is unsupported", op_type_));
    return absl::OkStatus ();
  }

  uint64_t
  time () noexcept override
  {
    return timer_.micros ();
  }

  absl::StatusOr<Tensor>
  operator() (Tensor a)
  {
    if (a.dtype () != dtype_)
      return absl::InternalError (absl::StrFormat (
          "reduce op defined with %d dtype but the dtype of input0 is %d",
          int (dtype_), int (a.dtype ())));
    auto b = Tensor (a.channels (), a.height (), 1, dev_, dtype_);
    VKLLAMA_STATUS_OK (b.create ());
    if (a.size () == 0)
      return b;
    timer_.start (dev_);
    const int err = vkl_reduce_f16 (a.data (), (int)a.channels (),
                                    (int)a.height (), (int)a.width (),
                                    op_type_, b.data (), dev_->stream ());
    timer_.stop (dev_);
    VKLLAMA_STATUS_OK (launch_status ("reduce", err));
    return b;
  }

private:
  const int op_type_;
  const Tensor::DType dtype_;
};
}
#endif
