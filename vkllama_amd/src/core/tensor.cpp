#include "src/core/tensor.h"
#include "src/core/gpu_device.h"
#include "absl/strings/str_format.h"
#include "src/core/quants.h"
#include "vkl_hip.h"

namespace vkllama
{
DTypeProperty
get_dtype_property (const DType dtype)
{
  switch (dtype)
    {
    case FP32: return { 1, sizeof (float) };
    case FP16: return { 1, sizeof (uint16_t) };
    case UINT32: return { 1, sizeof (uint32_t) };
    case INT8: return { 1, sizeof (int8_t) };
    case Q8_0: return { 32, 34 };
    }
  return { 1, 0 };
}

Tensor::Tensor ()
    : c_ (0), h_ (0), w_ (0), cs_ (0), hs_ (0), ws_ (0), dev_ (nullptr),
      visable_ (false), dtype_ (FP32), data_ (nullptr), status_ (nullptr)
{
}

Tensor::Tensor (const int c, const int h, const int w, GPUDevice *dev,
                const DType dtype, const bool visable)
    : Tensor (c, h, w, 0, 0, 0, dev, dtype, visable)
{
}

Tensor::Tensor (const int c, const int h, const int w, const int cs,
                const int hs, const int ws, GPUDevice *dev, const DType dtype,
                const bool visable)
    : c_ (c), h_ (h), w_ (w), cs_ (cs), hs_ (hs), ws_ (ws), dev_ (dev),
      visable_ (visable), dtype_ (dtype), data_ (nullptr), status_ (nullptr)
{
}

Tensor::Tensor (const Tensor &rhs)
    : c_ (rhs.c_), h_ (rhs.h_), w_ (rhs.w_), cs_ (rhs.cs_), hs_ (rhs.hs_),
      ws_ (rhs.ws_), dev_ (rhs.dev_), visable_ (rhs.visable_),
      dtype_ (rhs.dtype_), data_ (rhs.data_), status_ (rhs.status_)
{
  if (status_)
    status_->ref_.fetch_add (1);
}

Tensor::Tensor (Tensor &&rhs)
    : c_ (rhs.c_), h_ (rhs.h_), w_ (rhs.w_), cs_ (rhs.cs_), hs_ (rhs.hs_),
      ws_ (rhs.ws_), dev_ (rhs.dev_), visable_ (rhs.visable_),
      dtype_ (rhs.dtype_), data_ (rhs.data_), status_ (rhs.status_)
{
  rhs.status_ = nullptr;
  rhs.data_ = nullptr;
}

Tensor &
Tensor::operator= (Tensor const &rhs)
{
  if (rhs.status_)
    rhs.status_->ref_.fetch_add (1);
  release_ ();
  c_ = rhs.c_, h_ = rhs.h_, w_ = rhs.w_;
  cs_ = rhs.cs_, hs_ = rhs.hs_, ws_ = rhs.ws_;
  dev_ = rhs.dev_;
  visable_ = rhs.visable_;
  dtype_ = rhs.dtype_;
  data_ = rhs.data_;
  status_ = rhs.status_;
  return *this;
}

Tensor::~Tensor () { release_ (); }

void
Tensor::release_ ()
{
  if (status_ && status_->ref_.fetch_sub (1) == 1)
    {
      if (data_)
        dev_->release (data_, status_->bytes_, visable_);
      delete status_;
    }
  status_ = nullptr;
  data_ = nullptr;
}

Tensor
Tensor::like (const Tensor &t)
{
  return Tensor (t.c_, t.h_, t.w_, t.dev_, t.dtype_, t.visable_);
}

size_t
Tensor::elem_bytes () const
{
  switch (dtype_)
    {
    case FP32: return sizeof (float);
    case UINT32: return sizeof (uint32_t);
    case FP16: return sizeof (uint16_t);
    case INT8:
    case Q8_0: return sizeof (int8_t);
    }
  return 0;
}

void
Tensor::update_strides_ ()
{
  const auto prop = get_dtype_property (dtype_);
  const auto blocks = (w_ + prop.items_per_block - 1) / prop.items_per_block;
  ws_ = (int)elem_bytes ();
  hs_ = (int)(blocks * prop.bytes_per_block);
  cs_ = h_ * hs_;
}

absl::Status
Tensor::create ()
{
  if (!dev_)
    return absl::InternalError ("Tensor::create: no device");
  if (c_ < 0 || h_ < 0 || w_ < 0)
    return absl::InvalidArgumentError (absl::StrFormat (
        "Tensor::create: negative extent (%d, %d, %d)", c_, h_, w_));
  release_ ();
  update_strides_ ();
  const size_t n = bytes ();
  void *p = nullptr;
  const int e = dev_->alloc (&p, n, visable_);
  if (e)
    return absl::InternalError (absl::StrFormat (
        "failed at allocating %zu bytes: %s", n, vkl_error_string (e)));
  data_ = p;
  status_ = new __TensorStatus ();
  status_->ref_.store (1);
  status_->bytes_ = n;
  return absl::OkStatus ();
}

size_t Tensor::bytes () const { return (size_t)c_ * (size_t)cs_; }
void *Tensor::host () { return visable_ ? data_ : nullptr; }
void *Tensor::data () { return data_; }
const void *Tensor::data () const { return data_; }
bool Tensor::visable () const { return visable_; }
size_t Tensor::channels () const { return c_; }
size_t Tensor::height () const { return h_; }
size_t Tensor::width () const { return w_; }
size_t Tensor::cs () const { return cs_; }
size_t Tensor::hs () const { return hs_; }
size_t Tensor::ws () const { return ws_; }
Tensor::DType Tensor::dtype () const { return dtype_; }

std::array<size_t, 3>
Tensor::shape () const
{
  return { channels (), height (), width () };
}

ShaderConstants
Tensor::shape_constant () const
{
  ShapeConstant shape = { (uint32_t)c_,  (uint32_t)h_,  (uint32_t)w_,
                          (uint32_t)cs_, (uint32_t)hs_, (uint32_t)ws_ };
  return shape;
}

size_t Tensor::size () const { return (size_t)c_ * h_ * w_; }

absl::Status
Tensor::reshape (size_t const c, size_t const h, size_t const w)
{
  if (c * h * w != (size_t)c_ * h_ * w_)
    return absl::OutOfRangeError (absl::StrFormat (
        "reshape from (%zu, %zu, %zu) to (%zu, %zu, %zu) error.", (size_t)c_,
        (size_t)h_, (size_t)w_, c, h, w));
  c_ = (int)c, h_ = (int)h, w_ = (int)w;
  update_strides_ ();
  return absl::OkStatus ();
}

Tensor
Tensor::view (size_t c, size_t h, size_t w)
{
  Tensor v = *this;
  v.c_ = (int)c, v.h_ = (int)h, v.w_ = (int)w;
  return v;
}

// Pinned host memory is coherent with the device at stream boundaries, so
// flush/invalid have nothing to do; they keep the reference's contract of
// failing on device-local tensors (src/core/tensor.cpp:313-317,335-339).
absl::Status
Tensor::flush ()
{
  if (!visable_)
    return absl::UnimplementedError ("cannot flush to invisable tensor");
  return absl::OkStatus ();
}

absl::Status
Tensor::invalid ()
{
  if (!visable_)
    return absl::UnimplementedError ("cannot invalid an invisable tensor");
  return absl::OkStatus ();
}
}
