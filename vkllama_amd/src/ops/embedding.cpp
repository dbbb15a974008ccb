// Follows src/ops/embedding.cpp:17-114 of the reference: indices [1, H, W]
// UINT32 -> output [H, W, vocab.width] FP16; ids >= vocab rows map to UNK.
#include "src/ops/embedding.h"
#include "src/core/command.h"
#include "vkl_hip.h"

namespace vkllama
{
Embedding::Embedding (GPUDevice *dev, Command *command, Tensor vocab,
                      const uint32_t UNK, const Tensor::DType dtype)
    : Op (dev, command), vocab_ (vocab), UNK_ (UNK), dtype_ (dtype)
{
}

absl::Status
Embedding::init () noexcept
{
  if (dtype_ != FP16 && dtype_ != Q8_0)
    return absl::InvalidArgumentError (
        "Embedding op: only fp16 and q8_0 are supported.");
  return absl::OkStatus ();
}

uint64_t
Embedding::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
Embedding::operator() (Tensor indices) noexcept
{
  if (vocab_.channels () != 1 || indices.channels () != 1)
    return absl::InvalidArgumentError (absl::StrFormat (
        "only channels = 1 is supported. vocab channels = %zu, indices "
        "channels = %zu\n",
        vocab_.channels (), indices.channels ()));
  if (indices.dtype () != UINT32 || vocab_.dtype () != dtype_)
    return absl::InvalidArgumentError (
        "only indices.dtype = UINT32 is supported");
  if (UNK_ >= vocab_.height ())
    return absl::InvalidArgumentError (absl::StrFormat (
        "UNK = %u is outside the vocabulary of %zu rows", UNK_,
        vocab_.height ()));
  if (out_.channels () != indices.height ()
      || out_.height () != indices.width ()
      || out_.width () != vocab_.width ())
    {
      out_ = Tensor (indices.height (), indices.width (), vocab_.width (),
                     dev_, FP16);
      VKLLAMA_STATUS_OK (out_.create ());
    }
  const uint32_t n = (uint32_t)(indices.height () * indices.width ());
  timer_.start (dev_);
  int err;
  if (dtype_ == Q8_0)
    err = vkl_embed_q8_0 (vocab_.data (), (uint32_t)vocab_.height (),
                          (uint32_t)vocab_.width (),
                          (const uint32_t *)indices.data (), n, UNK_,
                          out_.data (), dev_->stream ());
  else
    err = vkl_embed_f16 (vocab_.data (), (uint32_t)vocab_.height (),
                         (uint32_t)vocab_.width (),
                         (const uint32_t *)indices.data (), n, UNK_,
                         out_.data (), dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("embedding", err));
  return out_;
}
}
