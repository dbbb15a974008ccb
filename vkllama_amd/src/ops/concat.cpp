// Follows src/ops/concat.cpp:13-200 of the reference: `num` inputs joined
// along axis 0 (channels), 1 (height) or 2 (width); every input is one
// strided copy into its place in the output.
#include "src/ops/concat.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
Concat::Concat (GPUDevice *gpu, Command *command, const int num,
                const int axis, Tensor::DType const dtype)
    : Op (gpu, command), num_ (num), axis_ (axis), dtype_ (dtype)
{
}

absl::Status
Concat::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "Concat op: only fp16 dtype is supported");
  if (axis_ < 0 || axis_ > 2)
    return absl::InvalidArgumentError (
        absl::StrFormat ("axis %d is unsupported.", axis_));
  return absl::OkStatus ();
}

uint64_t
Concat::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
Concat::operator() (std::vector<Tensor> const &inputs) noexcept
{
  if (inputs.size () != (size_t)num_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "operator has %zu inputs but %zu are given", (size_t)num_,
        inputs.size ()));
  if (inputs.empty ())
    return absl::InvalidArgumentError ("concat of no inputs");
  const Tensor &first = inputs.front ();
  size_t dims[3] = { first.channels (), first.height (), first.width () };
  for (size_t i = 0; i < inputs.size (); ++i)
    {
      const Tensor &t = inputs[i];
      if (t.dtype () != dtype_)
        return absl::InvalidArgumentError ("dtype of inputs are unsupported.");
      const size_t d[3] = { t.channels (), t.height (), t.width () };
      for (int ax = 0; ax < 3; ++ax)
        if (ax != axis_ && d[ax] != dims[ax])
          return absl::InvalidArgumentError (
              absl::StrFormat ("inputs shape error on axis %d", axis_));
      if (i > 0)
        dims[axis_] += d[axis_];
    }
  if (out_.channels () != dims[0] || out_.height () != dims[1]
      || out_.width () != dims[2])
    {
      out_ = Tensor (dims[0], dims[1], dims[2], dev_, dtype_);
      VKLLAMA_STATUS_OK (out_.create ());
    }
  // where input i starts in the output, in elements (concat.cpp:143-166)
  size_t offset = 0;
  timer_.start (dev_);
  int err = 0;
  for (const Tensor &t : inputs)
    {
      if (t.size () > 0)
        err = vkl_concat_part_f16 (
            t.data (), (int)t.channels (), (int)t.height (), (int)t.width (),
            t.cs () / 2, t.hs () / 2, out_.data (), out_.cs () / 2,
            out_.hs () / 2, offset, dev_->stream ());
      if (err)
        break;
      offset += axis_ == 0   ? t.channels () * (out_.cs () / 2)
                : axis_ == 1 ? t.height () * (out_.hs () / 2)
                             : t.width ();
    }
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("concat", err));
  return out_;
}
}
