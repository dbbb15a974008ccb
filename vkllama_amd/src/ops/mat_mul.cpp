// MatMul on the HIP layer.  Behaviour follows the reference's
// src/ops/mat_mul.cpp: dtype/shape checks and their status codes (:28-125,
// :159-183, :230-249), the cached output tensor (:185-194), and the kernel
// choice by (a_dtype, b_dtype, transpose_b) (:71-109).
#include "src/ops/mat_mul.h"
#include "src/core/command.h"
#include "vkl_hip.h"
#include <algorithm>

namespace vkllama
{
MatMul::MatMul (GPUDevice *dev, Command *command, Tensor weight,
                const float scale, const float bias, const int act,
                const int broadcast_type, const bool transpose_b,
                const Tensor::DType a_dtype, const Tensor::DType b_dtype)
    : Op (dev, command), weight_ (weight), broadcast_type_ (broadcast_type),
      act_ (act), transpose_b_ (transpose_b), a_dtype_ (a_dtype),
      b_dtype_ (b_dtype), scale_ (scale), bias_ (bias), inited_ (false)
{
}

MatMul::MatMul (GPUDevice *dev, Command *command, const float scale,
                const float bias, const int act, const int broadcast_type,
                const bool transpose_b, const Tensor::DType a_dtype,
                const Tensor::DType b_dtype)
    : Op (dev, command), broadcast_type_ (broadcast_type), act_ (act),
      transpose_b_ (transpose_b), a_dtype_ (a_dtype), b_dtype_ (b_dtype),
      scale_ (scale), bias_ (bias), inited_ (false)
{
}

absl::Status
MatMul::init () noexcept
{
  if (a_dtype_ != FP16)
    return absl::InvalidArgumentError (absl::StrFormat (
        "MatMul op: %d a_dtype is unsupported", int (a_dtype_)));
  if (weight_.size () > 0 && weight_.dtype () != b_dtype_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "matmul operator defined as %d b_dtype but dtype of "
        "weight tensor is %d",
        int (b_dtype_), int (weight_.dtype ())));
  if (broadcast_type_ < 0 || broadcast_type_ > 2)
    return absl::InvalidArgumentError (absl::StrFormat (
        "broadcast_type %d is unsupported.", broadcast_type_));
  const bool f16 = b_dtype_ == FP16;
  const bool q8 = b_dtype_ == Q8_0 && transpose_b_ && broadcast_type_ == 0;
  if (!f16 && !q8)
    return absl::InvalidArgumentError (
        absl::StrFormat ("%d a_dtype and %d b_dtype is unsupported",
                         int (a_dtype_), int (b_dtype_)));
  if (act_ != 0 && act_ != 1)
    return absl::InvalidArgumentError (
        absl::StrFormat ("activation %d is unsupported", act_));
  inited_ = true;
  return absl::OkStatus ();
}

uint64_t
MatMul::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
MatMul::operator() (Tensor a) noexcept
{
  if (weight_.size () == 0 || a.dtype () != a_dtype_)
    return absl::InvalidArgumentError (
        absl::StrFormat ("matmul op defined with %d a dtype but %d given.",
                         int (a_dtype_), int (a.dtype ())));
  if (broadcast_type_ == 0 && weight_.channels () != a.channels ())
    return absl::InvalidArgumentError (absl::StrFormat (
        "matmul op defined with broadcast_type = %d but weight channels = "
        "%zu != a.channels = %zu",
        broadcast_type_, weight_.channels (), a.channels ()));
  if (broadcast_type_ == 1 && weight_.channels () != 1)
    return absl::InvalidArgumentError (
        absl::StrFormat ("matmul op defined with broadcast_type = %d but "
                         "weight channels = %zu != 1",
                         broadcast_type_, weight_.channels ()));
  return run_ (a, weight_);
}

absl::StatusOr<Tensor>
MatMul::operator() (Tensor a, Tensor b) noexcept
{
  if (b.size () == 0 || a.dtype () != a_dtype_ || b.dtype () != b_dtype_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "matmul op defined with %d a_dtype and %d b_dtype but inputs "
        "a.dtype() = %d, b.dtype() = %d",
        int (a_dtype_), int (b_dtype_), int (a.dtype ()), int (b.dtype ())));
  if ((broadcast_type_ == 0 && b.channels () != a.channels ())
      || (broadcast_type_ == 1 && b.channels () != 1))
    return absl::InvalidArgumentError (
        absl::StrFormat ("matmul defined with %d broadcast_type but "
                         "a.channels() = %zu, b.channels() = %zu",
                         broadcast_type_, a.channels (), b.channels ()));
  return run_ (a, b);
}

absl::StatusOr<Tensor>
MatMul::run_ (Tensor &a, Tensor &b) noexcept
{
  if (!inited_)
    return absl::InternalError ("matmul op used before init()");
  const size_t K = a.width ();
  const size_t bk = transpose_b_ ? b.width () : b.height ();
  if (bk != K)
    return absl::InvalidArgumentError (absl::StrFormat (
        "matmul shape error. a.shape = (%zu, %zu, %zu), b.shape = (%zu, "
        "%zu, %zu), transpose_b = %d",
        a.channels (), a.height (), a.width (), b.channels (), b.height (),
        b.width (), int (transpose_b_)));
  const size_t out_c = std::max (a.channels (), b.channels ());
  const size_t out_h = a.height ();
  const size_t out_w = transpose_b_ ? b.height () : b.width ();
  if (out_.channels () != out_c || out_.height () != out_h
      || out_.width () != out_w)
    {
      out_ = Tensor (out_c, out_h, out_w, dev_, FP16, false);
      VKLLAMA_STATUS_OK (out_.create ());
    }
  if (out_.size () == 0)
    return out_;

  const Tensor *res = residual_;
  residual_ = nullptr;
  if (res
      && (res->channels () != out_c || res->height () != out_h || res->width () != out_w
          || res->hs () != out_.hs () || res->dtype () != FP16
          || (b_dtype_ != Q8_0 && !transpose_b_) || out_c != 1))
    return absl::InvalidArgumentError ("matmul residual operand does not fit the product");

  void *s = dev_->stream ();
  int err = 0;
  timer_.start (dev_);
  if (b_dtype_ == Q8_0)
    {
      // the planar Q8_0 layout is defined per matrix: one channel only
      if (out_c != 1)
        return absl::InvalidArgumentError (absl::StrFormat (
            "matmul with Q8_0 weights supports channels = 1, got %zu", out_c));
      err = vkl_matmul_q8_0 (a.data (), b.data (), (int)out_h, (int)out_w,
                             (int)K, a.hs () / 2, out_.hs () / 2, scale_,
                             bias_, act_, res ? res->data () : nullptr,
                             out_.data (), nullptr, s);
    }
  else
    {
      // a broadcast operand gets channel stride 0
      const size_t acs
          = a.channels () == 1 && out_c > 1 ? 0 : a.cs () / 2;
      const size_t bcs
          = b.channels () == 1 && out_c > 1 ? 0 : b.cs () / 2;
      if (transpose_b_)
        err = vkl_matmul_f16_tb (a.data (), b.data (), (int)out_c, (int)out_h,
                                 (int)out_w, (int)K, acs, a.hs () / 2, bcs,
                                 b.hs () / 2, out_.cs () / 2, out_.hs () / 2,
                                 scale_, bias_, act_, res ? res->data () : nullptr,
                                 out_.data (), nullptr, s);
      else
        err = vkl_matmul_f16_nn (a.data (), b.data (), (int)out_c, (int)out_h,
                                 (int)out_w, (int)K, acs, a.hs () / 2, bcs,
                                 b.hs () / 2, out_.cs () / 2, out_.hs () / 2,
                                 scale_, bias_, act_, out_.data (), s);
    }
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("matmul", err));
  return out_;
}
}
