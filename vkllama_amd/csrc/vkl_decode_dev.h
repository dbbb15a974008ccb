// Shared declarations of the fused one-token decode step (device side).
#ifndef VKL_DECODE_DEV_H
#define VKL_DECODE_DEV_H
#include "../../include/vkl_decode.h"
#include "vkl_common.h"

namespace vkl
{
constexpr int kDecWaves = 8;
constexpr int kDecThreads = kDecWaves * VKL_WAVE;

struct QMat
{
  const uint8_t *q;  // int8 plane [N, Kp]
  const uint16_t *d; // scale plane [N, Kp/32]
};

__device__ __forceinline__ QMat
qmat (const void *planar, int N, int K)
{
  const int nb = (K + 31) >> 5;
  const uint8_t *p = (const uint8_t *)planar;
  return QMat{ p, (const uint16_t *)(p + (size_t)N * nb * 32) };
}

// Loads and stores that other compute units must see without a kernel
// boundary in between go through agent-scope relaxed atomics: they bypass the
// per-XCD L2 instead of relying on cache write-back / invalidate.
__device__ __forceinline__ uint32_t
ld_coherent_u32 (const uint32_t *p)
{
  return __hip_atomic_load (p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ void
st_coherent_u32 (uint32_t *p, uint32_t v)
{
  __hip_atomic_store (p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
} // namespace vkl
#endif
