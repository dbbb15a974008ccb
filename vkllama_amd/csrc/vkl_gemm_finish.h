// Shared epilogue of the prompt GEMM kernels that walk their results row-wise,
// eight neighbouring output columns per lane.
#ifndef VKL_GEMM_FINISH_H
#define VKL_GEMM_FINISH_H
#include "vkl_common.h"
#include "vkl_gemm.h"

namespace vkl
{
// Eight neighbouring outputs of row m from column ncol0 on: v the fp32 sums (for
// the fused pair: up; g: gate), then scale, bias, activation, rounding,
// residual, the stores.
template <bool UPGATE>
__device__ __forceinline__ void
gemm_finish8 (const GemmArgs &a, float (&v)[8], const float (&g)[8], int m, int ncol0, int zmat, int vec,
              float *part)
{
  if (!UPGATE && part)
    {
      // one part of a split k range: the raw sums, dense [M, N] fp32; the
      // reduction kernel adds the parts in order and applies the rest
      if (m >= a.M || ncol0 >= a.N)
        return;
      float *dst = part + (size_t)m * a.N + ncol0;
      if ((a.N % 4) == 0 && ncol0 + 8 <= a.N)
        {
          typedef float f32x4 __attribute__ ((ext_vector_type (4)));
          f32x4 w0 = { v[0], v[1], v[2], v[3] }, w1 = { v[4], v[5], v[6], v[7] };
          *(VKL_GLOBAL f32x4 *)dst = w0;
          *(VKL_GLOBAL f32x4 *)(dst + 4) = w1;
        }
      else
        for (int e = 0; e < 8 && ncol0 + e < a.N; ++e)
          dst[e] = v[e];
      return;
    }
  uint16_t *y = a.y[UPGATE ? 0 : zmat];
  const bool plain = a.nmat != 1; // one of three fused outputs: no scale, activation, residual
  if (UPGATE)
    {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v[e] = silu (g[e]) * v[e];
    }
  else if (!plain)
    {
#pragma unroll
      for (int e = 0; e < 8; ++e)
        v[e] = v[e] * a.scale + a.bias;
      if (a.act == 1)
        {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = silu (v[e]);
        }
    }
  if (m >= a.M || ncol0 >= a.N)
    return;
  uint16_t h[8];
#pragma unroll
  for (int e = 0; e < 8; ++e)
    h[e] = f2h (v[e]);
  const size_t o = (size_t)m * a.ys + ncol0;
  const bool res = !UPGATE && !plain && a.residual;
  float *y32 = !UPGATE && !plain && a.y32 ? a.y32 + (size_t)m * a.N + ncol0 : nullptr;
  if (vec && ncol0 + 8 <= a.N)
    {
      if (res)
        {
          const uint4 rv = ldg4 (a.residual + o);
          const uint32_t rw[4] = { rv.x, rv.y, rv.z, rv.w };
#pragma unroll
          for (int e = 0; e < 8; ++e)
            h[e] = f2h (h2f (h[e]) + h2f ((uint16_t)(rw[e >> 1] >> ((e & 1) * 16))));
        }
      vkl_u32x4 pk;
      pk.x = h[0] | ((uint32_t)h[1] << 16), pk.y = h[2] | ((uint32_t)h[3] << 16);
      pk.z = h[4] | ((uint32_t)h[5] << 16), pk.w = h[6] | ((uint32_t)h[7] << 16);
      *(VKL_GLOBAL vkl_u32x4 *)(y + o) = pk;
      if (y32)
        {
          typedef float f32x4 __attribute__ ((ext_vector_type (4)));
          f32x4 w0 = { h2f (h[0]), h2f (h[1]), h2f (h[2]), h2f (h[3]) };
          f32x4 w1 = { h2f (h[4]), h2f (h[5]), h2f (h[6]), h2f (h[7]) };
          *(VKL_GLOBAL f32x4 *)y32 = w0;
          *(VKL_GLOBAL f32x4 *)(y32 + 4) = w1;
        }
      return;
    }
  // ragged end of a row, or operands that are not 16-byte aligned
  for (int e = 0; e < 8 && ncol0 + e < a.N; ++e)
    {
      uint16_t he = h[e];
      if (res)
        he = f2h (h2f (he) + h2f (ldg (a.residual + o + e)));
      y[o + e] = he;
      if (y32)
        y32[e] = h2f (he);
    }
}
} // namespace vkl
#endif
