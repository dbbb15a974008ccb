// Tensor: interface of the reference's src/core/tensor.h:16-90.  A shared
// handle (last copy frees) on a 3-D array [c, h, w] with BYTE strides
// (cs, hs, ws); device memory comes from hipMalloc, "visable" tensors are
// pinned host memory that kernels read directly.  data() is the device
// pointer.  Q8_0 tensors hold the planar layout described in vkl_hip.h; their
// byte count equals the GGUF block layout's (34 bytes per 32 weights).
#ifndef __VKLLAMA_TENSOR__
#define __VKLLAMA_TENSOR__

#include "absl/status/status.h"
#include "src/core/common.h"
#include "src/core/gpu_device.h"
#include "src/core/shader_constants.h"
#include <array>
#include <atomic>
#include <stddef.h>

namespace vkllama
{
class Tensor
{
public:
  using DType = ::vkllama::DType;
  static Tensor like (Tensor const &);
  Tensor ();
  Tensor (const int c, const int h, const int w, GPUDevice *dev,
          DType const dtype = FP32, const bool visable = false);
  Tensor (const int c, const int h, const int w, const int cs, const int hs,
          const int ws, GPUDevice *dev, DType const dtype = FP32,
          const bool visable = false);

  Tensor &operator= (Tensor const &);
  Tensor (const Tensor &rhs);
  Tensor (Tensor &&rhs);
  ~Tensor ();

  // same storage and strides, new extents (src/core/tensor.cpp:293-302)
  Tensor view (size_t c, size_t h, size_t w);

  size_t channels () const;
  size_t height () const;
  size_t width () const;
  size_t cs () const;
  size_t hs () const;
  size_t ws () const;
  std::array<size_t, 3> shape () const;
  ShaderConstants shape_constant () const;
  size_t size () const;

  absl::Status reshape (size_t const c, size_t const h, size_t const w);

  void *data ();
  const void *data () const;

  absl::Status create ();
  size_t bytes () const;
  bool visable () const;
  DType dtype () const;
  size_t elem_bytes () const;
  absl::Status flush ();
  absl::Status invalid ();
  void *host ();
  GPUDevice *device () const { return dev_; }

private:
  void update_strides_ ();
  void release_ ();

  int c_, h_, w_;
  int cs_, hs_, ws_;
  GPUDevice *dev_;
  bool visable_;
  DType dtype_;
  void *data_;
  struct __TensorStatus
  {
    std::atomic<int> ref_;
    size_t bytes_ = 0; // size the block was requested with
  };
  __TensorStatus *status_;
};
}
#endif
