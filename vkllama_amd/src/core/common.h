// Interface kept from the reference's src/core/common.h:1-30.
#ifndef __VKLLAMA_COMMON_H__
#define __VKLLAMA_COMMON_H__
#include "absl/status/status.h"
#include "absl/status/statusor.h"
#include <stdint.h>
namespace vkllama
{
namespace detail
{
inline const absl::Status &
status_of (const absl::Status &s)
{
  return s;
}
template <typename T>
inline const absl::Status &
status_of (const absl::StatusOr<T> &s)
{
  return s.status ();
}
}
// Returns the error of a Status / StatusOr expression from the enclosing
// function (which may itself return a Status or any StatusOr).
#define VKLLAMA_STATUS_OK(__expr)                                             \
  if (auto __s = (__expr); !__s.ok ())                                        \
    {                                                                         \
      return ::vkllama::detail::status_of (__s);                              \
    }

#ifndef __VKLLAMA_LOG_COST
#define __VKLLAMA_LOG_COST 0
#endif
typedef enum : int
{
  FP32 = 0,
  FP16,
  UINT32,
  INT8,
  Q8_0, // block-wise quantize
} DType;

struct ShapeConstant
{
  uint32_t c, h, w, cs, hs, ws;
} __attribute__ ((packed));
}

#endif
