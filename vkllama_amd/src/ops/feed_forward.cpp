// Follows src/ops/feed_forward.cpp of the reference: one fused launch for
// T = fp16(silu(X W1^T) * (X W3^T)) (:106-120), then the down projection
// through a MatMul (:122-128).  Only transposed ([out, in]) weights exist on
// the HIP layer; the reference's MatMul rejects the other orientation for
// Q8_0 as well (src/ops/mat_mul.cpp:98-109).
#include "src/ops/feed_forward.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
FeedForward::FeedForward (GPUDevice *dev, Command *command, Tensor w1,
                          Tensor w2, Tensor w3, const bool transposed_weight,
                          const Tensor::DType dtype)
    : Op (dev, command), w1_ (w1), w2_ (w2), w3_ (w3), dtype_ (dtype),
      transposed_weight_ (transposed_weight), inited_ (false)
{
  down_op_.reset (new MatMul (dev_, command_, w2_, 1.0, .0, 0, 0,
                              transposed_weight_, FP16, dtype_));
}

absl::Status
FeedForward::init () noexcept
{
  if (dtype_ != FP16 && dtype_ != Q8_0)
    return absl::InvalidArgumentError (
        "FeedForward op: only fp16 and q8_0 are supported.");
  if (w1_.dtype () != w2_.dtype () || w2_.dtype () != w3_.dtype ()
      || dtype_ != w1_.dtype ())
    return absl::InvalidArgumentError (
        absl::StrFormat ("feed_forward op defined with %d dtype but "
                         "w1.dtype = %d, w2.dtype = %d, w3.dtype = %d",
                         int (dtype_), int (w1_.dtype ()), int (w2_.dtype ()),
                         int (w3_.dtype ())));
  if (!transposed_weight_)
    return absl::InvalidArgumentError (
        "feed_forward op: only transposed ([out, in]) weights are supported");
  if (w1_.channels () != 1 || w3_.channels () != 1
      || w1_.height () != w3_.height () || w1_.width () != w3_.width ()
      || w2_.width () != w1_.height () || w2_.height () != w1_.width ())
    return absl::InvalidArgumentError (absl::StrFormat (
        "feed_forward op: weight shapes w1 = (%zu, %zu, %zu), w2 = (%zu, "
        "%zu, %zu), w3 = (%zu, %zu, %zu) do not fit",
        w1_.channels (), w1_.height (), w1_.width (), w2_.channels (),
        w2_.height (), w2_.width (), w3_.channels (), w3_.height (),
        w3_.width ()));
  VKLLAMA_STATUS_OK (down_op_->init ());
  inited_ = true;
  return absl::OkStatus ();
}

uint64_t
FeedForward::time () noexcept
{
  return down_op_->time () + timer_.micros ();
}

absl::StatusOr<Tensor>
FeedForward::operator() (Tensor X) noexcept
{
  if (X.dtype () != FP16)
    return absl::InvalidArgumentError (absl::StrFormat (
        "feed_forward op defined with FP16 input but input X.dtype() = %d",
        int (X.dtype ())));
  if (!inited_)
    return absl::InternalError ("feed_forward op used before init()");
  if (X.width () != w1_.width () || X.channels () != 1)
    return absl::InvalidArgumentError (absl::StrFormat (
        "feed_forward shape error. X.shape = (%zu, %zu, %zu), w1.shape = "
        "(%zu, %zu, %zu)",
        X.channels (), X.height (), X.width (), w1_.channels (),
        w1_.height (), w1_.width ()));
  if (t0_.channels () != X.channels () || t0_.height () != X.height ()
      || t0_.width () != w1_.height ())
    {
      t0_ = Tensor (X.channels (), X.height (), w1_.height (), dev_, FP16,
                    false);
      VKLLAMA_STATUS_OK (t0_.create ());
    }
  timer_.start (dev_);
  int err;
  if (dtype_ == Q8_0)
    err = vkl_ffn_upgate_q8_0 (X.data (), w3_.data (), w1_.data (),
                               (int)X.height (), (int)w1_.height (),
                               (int)X.width (), t0_.data (), dev_->stream ());
  else
    err = vkl_ffn_upgate_f16 (X.data (), w3_.data (), w1_.data (),
                              (int)X.height (), (int)w1_.height (),
                              (int)X.width (), t0_.data (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("feed_forward up/gate", err));
  down_op_->set_residual (residual_);
  residual_ = nullptr;
  return (*down_op_) (t0_);
}
}
