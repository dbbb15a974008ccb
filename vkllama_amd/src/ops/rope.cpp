// Follows src/ops/rope.cpp of the reference.  The cos/sin tables are built on
// the host in float exactly as there (:19-47: freq[k] = 1/pow(10000, 2k/dim),
// angle = freq[k] * float(pos), std::cos / std::sin of a float).  The
// reference allocates 2*maxlen rows and uploads the first half of the bytes
// (:73-92), i.e. positions [0, maxlen); the same positions are valid here and
// a position outside them is rejected instead of reading unwritten memory.
#include "src/ops/rope.h"
#include "src/core/command.h"
#include "vkl_hip.h"
#include <cmath>

namespace vkllama
{
Rope::Rope (GPUDevice *dev, Command *command, const int maxlen, const int dim,
            const Tensor::DType dtype)
    : Op (dev, command), maxlen_ (maxlen), dim_ (dim), dtype_ (dtype)
{
}

void
Rope::compute_freq (size_t dim, size_t maxlen, std::vector<float> &freqc,
                    std::vector<float> &freqs)
{
  const size_t half = dim / 2;
  std::vector<float> freq (half);
  float n = .0f;
  for (size_t k = 0; k < half; ++k)
    {
      freq[k] = 1.0f / std::pow (10000.0f, n / dim);
      n += 2.0;
    }
  freqs.resize (maxlen * half);
  freqc.resize (maxlen * half);
  for (size_t i = 0; i < maxlen; ++i)
    for (size_t k = 0; k < half; ++k)
      {
        const float f = freq[k] * static_cast<float> (i);
        freqc[i * half + k] = std::cos (f);
        freqs[i * half + k] = std::sin (f);
      }
}

absl::Status
Rope::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "Rope op: only fp16 dtype is supported.");
  if (maxlen_ <= 0 || dim_ <= 0 || (dim_ % 2) != 0)
    return absl::InvalidArgumentError (absl::StrFormat (
        "Rope op: bad maxlen = %d or dim = %d", maxlen_, dim_));
  freqc_ = Tensor (1, maxlen_, dim_ / 2, dev_, FP32, false);
  freqs_ = Tensor (1, maxlen_, dim_ / 2, dev_, FP32, false);
  VKLLAMA_STATUS_OK (freqc_.create ());
  VKLLAMA_STATUS_OK (freqs_.create ());
  std::vector<float> freqc, freqs;
  compute_freq (dim_, maxlen_, freqc, freqs);
  VKLLAMA_STATUS_OK (command_->upload (freqc.data (), freqc.size (), freqc_));
  VKLLAMA_STATUS_OK (command_->upload (freqs.data (), freqs.size (), freqs_));
  return absl::OkStatus ();
}

uint64_t
Rope::time () noexcept
{
  return timer_.micros ();
}

absl::StatusOr<Tensor>
Rope::operator() (Tensor query, const size_t offset) noexcept
{
  if (query.width () != (size_t)dim_ || query.height () > (size_t)maxlen_)
    return absl::InvalidArgumentError (absl::StrFormat (
        "rope shape error. input0.shape = (%zu, %zu, %zu)"
        " dim = %d, maxlen = %d",
        query.channels (), query.height (), query.width (), dim_, maxlen_));
  if (query.dtype () != dtype_)
    return absl::InvalidArgumentError (
        absl::StrFormat ("rope defined with dtype %d. but query.dtype = %d",
                         int (dtype_), int (query.dtype ())));
  if (offset + query.height () > (size_t)maxlen_)
    return absl::OutOfRangeError (absl::StrFormat (
        "rope positions [%zu, %zu) exceed maxlen = %d", offset,
        offset + query.height (), maxlen_));
  timer_.start (dev_);
  const int err = vkl_rope_f16 (
      query.data (), (int)query.channels (), (int)query.height (),
      (int)query.width (), (const float *)freqc_.data (),
      (const float *)freqs_.data (), (uint32_t)offset, dev_->stream ());
  timer_.stop (dev_);
  VKLLAMA_STATUS_OK (launch_status ("rope", err));
  return query;
}
}
