// Q8_0 host quantiser, interface of the reference's src/core/quants.h:17-139.
// Blocks are the 34-byte GGUF blocks the compute kernels read
// ({fp16 d; int8 q[32]}); the reference's host code writes a 36-byte block
// with an fp32 scale that its own shaders cannot read.
#ifndef __VKLLAMA_QUANTS_H__
#define __VKLLAMA_QUANTS_H__

#include "absl/status/status.h"
#include "src/core/common.h"
#include "src/core/float.h"
#include <algorithm>
#include <math.h>
#include <stddef.h>
#include <string.h>
#include <type_traits>
#include <vector>

namespace vkllama
{
struct DTypeProperty
{
  uint32_t items_per_block;
  uint32_t bytes_per_block;
};

extern DTypeProperty get_dtype_property (DType const dtype);

namespace detail
{
template <typename T>
inline float
load_as_f32 (const T *src, size_t i)
{
  if constexpr (std::is_same<typename std::remove_const<T>::type,
                             __vkllama_fp16_t>::value)
    return __fp16_to_fp32 (src[i].u16);
  else
    return (float)src[i];
}
}

// amax over the block, scale = amax/127, q = roundf(x * 127/amax), the tail of
// the last block is padded with zeros (src/core/quants.h:57-93).
template <typename T>
absl::Status
qint8_0_quantize_row (const T *src, int8_t *dst, const size_t n)
{
  const auto prop = get_dtype_property (Q8_0);
  const size_t per = prop.items_per_block;
  const size_t blocks = (n + per - 1) / per;
  for (size_t b = 0; b < blocks; ++b)
    {
      const size_t start = b * per, end = std::min (start + per, n);
      float amax = fabsf (detail::load_as_f32 (src, start));
      for (size_t i = start; i < end; ++i)
        amax = std::max (amax, fabsf (detail::load_as_f32 (src, i)));
      const float scale = amax / 127.0f;
      const float inverse = scale > 0 ? 127.0f / amax : .0f;
      const __vkllama_fp16_t d = __fp32_to_fp16_rne (scale);
      int8_t *blk = dst + b * prop.bytes_per_block;
      memcpy (blk, &d.u16, sizeof (uint16_t));
      int8_t *q = blk + sizeof (uint16_t);
      for (size_t i = 0; i < per; ++i)
        q[i] = start + i < n
                   ? (int8_t)roundf (detail::load_as_f32 (src, start + i)
                                     * inverse)
                   : int8_t (0);
    }
  return absl::OkStatus ();
}

template <typename T>
absl::Status
qint8_0_dequantize_row (const int8_t *src, T *dst, const size_t n)
{
  const auto prop = get_dtype_property (Q8_0);
  const size_t per = prop.items_per_block;
  const size_t blocks = (n + per - 1) / per;
  for (size_t b = 0; b < blocks; ++b)
    {
      const int8_t *blk = src + b * prop.bytes_per_block;
      uint16_t bits;
      memcpy (&bits, blk, sizeof (bits));
      const float d = __fp16_to_fp32 (bits);
      const int8_t *q = blk + sizeof (uint16_t);
      for (size_t i = 0; i < per && b * per + i < n; ++i)
        {
          const float v = (float)q[i] * d;
          if constexpr (std::is_same<typename std::remove_const<T>::type,
                                     __vkllama_fp16_t>::value)
            dst[b * per + i] = __fp32_to_fp16 (v);
          else
            dst[b * per + i] = v;
        }
    }
  return absl::OkStatus ();
}
}
#endif
