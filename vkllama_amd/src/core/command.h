// Command: interface of the reference's src/core/command.h:26-483.
// The reference records Vulkan commands and runs them at submit(); here each
// operator launch is enqueued on the device's in-order HIP stream as it is
// recorded, begin/end/submit only mark the span, and wait() synchronises the
// stream and then runs the deferred host tasks (downloads into user memory),
// which is when results become valid in both implementations.
#ifndef __VKLLAMA_COMMAND_H__
#define __VKLLAMA_COMMAND_H__

#include "absl/status/status.h"
#include "absl/strings/str_format.h"
#include "src/core/float.h"
#include "src/core/gpu_device.h"
#include "src/core/tensor.h"
#include "vkl_hip.h"
#include <functional>
#include <memory>
#include <numeric>
#include <stdio.h>
#include <string>
#include <vector>

namespace vkllama
{
class Command
{
public:
  Command (GPUDevice *dev) : dev_ (dev) {}
  ~Command () { defer_task_.clear (); }

  absl::Status
  init ()
  {
    if (!dev_ || !dev_->stream ())
      return absl::InternalError ("Command: device is not initialised");
    return absl::OkStatus ();
  }

  absl::Status begin () { return absl::OkStatus (); }
  absl::Status end () { return absl::OkStatus (); }
  absl::Status submit () { return absl::OkStatus (); }

  absl::Status
  submit_and_wait ()
  {
    if (auto ret = submit (); !ret.ok ())
      return ret;
    return wait ();
  }

  void *stream () const { return dev_->stream (); }

  template <typename T>
  absl::Status
  upload (T const *from, const size_t n, Tensor &to)
  {
    return upload_bytes (reinterpret_cast<const uint8_t *> (from),
                         n * sizeof (T), to);
  }

  // The host bytes are consumed before this returns.  Q8_0 tensors take the
  // GGUF 34-byte block stream and are repacked on the device into the planar
  // layout; the whole tensor must be uploaded at once.
  absl::Status
  upload_bytes (uint8_t const *from, const size_t bytes, Tensor &to)
  {
    if (to.bytes () < bytes)
      return absl::OutOfRangeError (absl::StrFormat (
          "to.size() = %zu but %zu bytes upload.", to.bytes (), bytes));
    if (!to.data ())
      return absl::InternalError ("upload into a tensor that was not created");
    if (to.dtype () == Q8_0)
      {
        if (bytes != to.bytes ())
          return absl::InvalidArgumentError (absl::StrFormat (
              "Q8_0 tensors are uploaded whole: %zu of %zu bytes given",
              bytes, to.bytes ()));
        void *staging = nullptr;
        if (int e = vkl_malloc (&staging, bytes))
          return hip_error_ ("allocating upload staging", e);
        int e = vkl_memcpy_h2d (staging, from, bytes, stream ());
        if (!e)
          e = vkl_stream_sync (stream ());
        if (!e)
          e = vkl_q8_0_pack (staging, to.data (),
                             to.channels () * to.height (), to.width (),
                             stream ());
        defer_task_.push_back ([staging] () {
          vkl_free (staging);
          return absl::OkStatus ();
        });
        return e ? hip_error_ ("uploading Q8_0 tensor", e) : absl::OkStatus ();
      }
    if (to.visable ())
      {
        ::memcpy (to.host (), from, bytes);
        return to.flush ();
      }
    int e = vkl_memcpy_h2d (to.data (), from, bytes, stream ());
    if (!e)
      e = vkl_stream_sync (stream ());
    return e ? hip_error_ ("uploading tensor", e) : absl::OkStatus ();
  }

  // Copies from.size() elements; the user buffer is filled when wait() runs
  // the deferred task.  Q8_0 tensors come back as GGUF blocks.
  template <typename T>
  absl::Status
  download (Tensor &from, T *to, const size_t n)
  {
    if (n < from.size ())
      return absl::InternalError (
          absl::StrFormat ("download bytes larger than source tensor. "
                           "from.size() = %zu, to.size() = %zu",
                           from.size (), n));
    if (from.visable ())
      {
        Tensor src = from;
        defer_task_.push_back ([src, to] () mutable {
          ::memcpy (to, src.host (), src.size () * sizeof (T));
          return absl::OkStatus ();
        });
        return absl::OkStatus ();
      }
    const size_t bytes
        = from.dtype () == Q8_0 ? from.bytes () : from.size () * sizeof (T);
    if (bytes > from.bytes ())
      return absl::InternalError (absl::StrFormat (
          "download of %zu bytes from a tensor of %zu", bytes, from.bytes ()));
    auto staging = std::make_shared<Tensor> (1, 1, (int)bytes, dev_, INT8, true);
    VKLLAMA_STATUS_OK (staging->create ());
    const void *src = from.data ();
    void *unpacked = nullptr;
    if (from.dtype () == Q8_0)
      {
        if (int e = vkl_malloc (&unpacked, bytes))
          return hip_error_ ("allocating download staging", e);
        if (int e = vkl_q8_0_unpack (from.data (), unpacked,
                                     from.channels () * from.height (),
                                     from.width (), stream ()))
          {
            vkl_free (unpacked);
            return hip_error_ ("unpacking Q8_0 tensor", e);
          }
        src = unpacked;
      }
    if (int e = vkl_memcpy_d2h (staging->host (), src, bytes, stream ()))
      return hip_error_ ("downloading tensor", e);
    defer_task_.push_back ([staging, to, bytes, unpacked] () {
      ::memcpy (reinterpret_cast<void *> (to), staging->host (), bytes);
      if (unpacked)
        vkl_free (unpacked);
      return absl::OkStatus ();
    });
    return absl::OkStatus ();
  }

  absl::Status
  print_tensor_mean (const std::string &msg, Tensor &t)
  {
    if (t.dtype () != FP16 && t.dtype () != FP32)
      return absl::InvalidArgumentError (
          "Command::print_tensor_mean: only fp16 and fp32 tensor is "
          "supported.");
    auto buf = std::make_shared<std::vector<uint8_t> > (t.bytes ());
    if (t.dtype () == FP32)
      {
        VKLLAMA_STATUS_OK (
            this->download (t, (float *)buf->data (), buf->size () / 4));
      }
    else
      {
        VKLLAMA_STATUS_OK (
            this->download (t, (uint16_t *)buf->data (), buf->size () / 2));
      }
    this->defer ([msg, buf, dtype = t.dtype (), n = t.size ()] () {
      float acc = .0f;
      if (dtype == FP32)
        {
          auto const *p = reinterpret_cast<const float *> (buf->data ());
          acc = std::accumulate (p, p + n, .0f);
        }
      else
        {
          auto const *p = reinterpret_cast<const uint16_t *> (buf->data ());
          for (size_t i = 0; i < n; ++i)
            acc += __fp16_to_fp32 (p[i]);
        }
      fprintf (stderr, "%s: %f\n", msg.c_str (), acc / n);
      return absl::OkStatus ();
    });
    return absl::OkStatus ();
  }

  absl::Status
  wait ()
  {
    if (int e = vkl_stream_sync (stream ()))
      {
        defer_task_.clear ();
        return hip_error_ ("waiting for the stream", e);
      }
    absl::Status defer_result = absl::OkStatus ();
    // tasks may enqueue further tasks; run what was queued at entry
    auto tasks = std::move (defer_task_);
    defer_task_.clear ();
    for (auto &fn : tasks)
      if (auto ret = fn (); !ret.ok ())
        defer_result = ret;
    return defer_result;
  }

  void
  defer (std::function<absl::Status (void)> &&fn)
  {
    defer_task_.push_back (std::move (fn));
  }

private:
  static absl::Status
  hip_error_ (const char *what, int e)
  {
    return absl::InternalError (
        absl::StrFormat ("failed at %s: %s", what, vkl_error_string (e)));
  }

  GPUDevice *dev_;
  std::vector<std::function<absl::Status (void)> > defer_task_;
};
}
#endif
