// A flat list of 32-bit words describing tensor shapes, kept from the
// reference's src/core/shader_constants.h for source compatibility
// (Tensor::shape_constant() returns one).  The HIP layer takes shapes as
// plain arguments, so nothing consumes the packed bytes.
#ifndef __VKLLAMA_SHADER_CONSTANTS_H__
#define __VKLLAMA_SHADER_CONSTANTS_H__
#include "src/core/common.h"
#include <string.h>
#include <vector>

namespace vkllama
{
class ShaderConstants
{
public:
  ShaderConstants () = default;
  ShaderConstants (ShapeConstant const &s) { append (&s, sizeof (s)); }

  template <typename T>
  void
  push_back (T const v)
  {
    static_assert (sizeof (T) == 4, "constants are 32-bit words");
    append (&v, sizeof (v));
  }

  ShaderConstants &
  operator+= (ShaderConstants const &rhs)
  {
    words_.insert (words_.end (), rhs.words_.begin (), rhs.words_.end ());
    return *this;
  }

  friend ShaderConstants
  operator+ (ShaderConstants lhs, ShaderConstants const &rhs)
  {
    lhs += rhs;
    return lhs;
  }

  const uint8_t *data () const { return (const uint8_t *)words_.data (); }
  size_t bytes () const { return words_.size () * 4; }
  size_t elem_num () const { return words_.size (); }

private:
  void
  append (const void *p, size_t n)
  {
    const size_t old = words_.size ();
    words_.resize (old + n / 4);
    memcpy (words_.data () + old, p, n);
  }
  std::vector<uint32_t> words_;
};
}
#endif
