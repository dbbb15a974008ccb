// Q8_0: host quantiser, GGUF-block <-> planar repack, embedding gather.
#include "../../include/vkl_hip.h"
#include "vkl_common.h"
#include <math.h>
#include <string.h>

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
static inline uint16_t
host_f32_to_f16_rne (float f)
{
  return __builtin_bit_cast (uint16_t, (_Float16)f);
}

static inline float
host_f16_to_f32 (uint16_t h)
{
  return (float)__builtin_bit_cast (_Float16, h);
}

extern "C" size_t
vkl_q8_0_row_bytes (size_t K)
{
  return (K + 31) / 32 * 34;
}

// Follows src/core/quants.h:35-96: amax over the block, scale = amax/127,
// inverse = 127/amax (0 when the block is all zero), q = roundf(x*inverse),
// tail padded with zeros.  The scale is stored as fp16 (RNE) in front of the
// 32 quants, the block the reference's shaders read.
extern "C" void
vkl_quantize_q8_0_h (const float *src, size_t n, uint8_t *dst)
{
  const size_t nb = (n + 31) / 32;
  for (size_t b = 0; b < nb; ++b)
    {
      const size_t start = b * 32;
      const size_t end = start + 32 < n ? start + 32 : n;
      float amax = fabsf (src[start]);
      for (size_t i = start; i < end; ++i)
        amax = fmaxf (amax, fabsf (src[i]));
      const float scale = amax / 127.0f;
      const float inv = scale > 0 ? 127.0f / amax : 0.0f;
      const uint16_t h = host_f32_to_f16_rne (scale);
      memcpy (dst, &h, 2);
      int8_t *q = (int8_t *)(dst + 2);
      for (size_t i = 0; i < 32; ++i)
        q[i] = start + i < n ? (int8_t)roundf (src[start + i] * inv) : 0;
      dst += 34;
    }
}

extern "C" void
vkl_dequantize_q8_0_h (const uint8_t *src, size_t n, float *dst)
{
  const size_t nb = (n + 31) / 32;
  for (size_t b = 0; b < nb; ++b)
    {
      uint16_t h;
      memcpy (&h, src + b * 34, 2);
      const float d = host_f16_to_f32 (h);
      const int8_t *q = (const int8_t *)(src + b * 34 + 2);
      for (size_t i = 0; i < 32 && b * 32 + i < n; ++i)
        dst[b * 32 + i] = (float)q[i] * d;
    }
}

// ---------------------------------------------------------------------------
// repack
// ---------------------------------------------------------------------------
// One thread per block.  Raw blocks are only 2-byte aligned, so they are read
// and written as 17 ushorts; the planar side is 32-byte aligned.
__global__ void
q8_pack_kernel (const uint16_t *__restrict__ raw, uint32_t *__restrict__ q,
                uint16_t *__restrict__ d, size_t nblocks)
{
  const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nblocks)
    return;
  const uint16_t *src = raw + b * 17;
  d[b] = src[0];
  uint32_t *dst = q + b * 8;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    dst[i] = (uint32_t)src[1 + 2 * i] | ((uint32_t)src[2 + 2 * i] << 16);
}

__global__ void
q8_unpack_kernel (const uint32_t *__restrict__ q,
                  const uint16_t *__restrict__ d, uint16_t *__restrict__ raw,
                  size_t nblocks)
{
  const size_t b = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= nblocks)
    return;
  uint16_t *dst = raw + b * 17;
  dst[0] = d[b];
  const uint32_t *src = q + b * 8;
#pragma unroll
  for (int i = 0; i < 8; ++i)
    {
      const uint32_t w = src[i];
      dst[1 + 2 * i] = (uint16_t)(w & 0xffffu);
      dst[2 + 2 * i] = (uint16_t)(w >> 16);
    }
}

extern "C" int
vkl_q8_0_pack (const void *raw, void *planar, size_t rows, size_t K,
               void *stream)
{
  VKL_CHECK_ARG (raw && planar);
  const size_t nb = (K + 31) / 32, nblocks = rows * nb;
  if (nblocks == 0)
    return 0;
  VKL_CHECK_ARG ((nblocks + 255) / 256 <= 0x7fffffffu);
  uint8_t *p = (uint8_t *)planar;
  q8_pack_kernel<<<dim3 ((unsigned)((nblocks + 255) / 256)), dim3 (256), 0,
                   (hipStream_t)stream>>> (
      (const uint16_t *)raw, (uint32_t *)p, (uint16_t *)(p + nblocks * 32),
      nblocks);
  return vkl_launch_status ();
}

extern "C" int
vkl_q8_0_unpack (const void *planar, void *raw, size_t rows, size_t K,
                 void *stream)
{
  VKL_CHECK_ARG (raw && planar);
  const size_t nb = (K + 31) / 32, nblocks = rows * nb;
  if (nblocks == 0)
    return 0;
  VKL_CHECK_ARG ((nblocks + 255) / 256 <= 0x7fffffffu);
  const uint8_t *p = (const uint8_t *)planar;
  q8_unpack_kernel<<<dim3 ((unsigned)((nblocks + 255) / 256)), dim3 (256), 0,
                     (hipStream_t)stream>>> (
      (const uint32_t *)p, (const uint16_t *)(p + nblocks * 32),
      (uint16_t *)raw, nblocks);
  return vkl_launch_status ();
}

// ---------------------------------------------------------------------------
// embedding
// ---------------------------------------------------------------------------
// grid (ceil(nb/256), n): one thread dequantises one 32-wide block of one
// token's row: out = fp16(float(q) * float(d)).
__global__ void
embed_q8_kernel (const uint8_t *__restrict__ q, const uint16_t *__restrict__ d,
                 uint32_t VH, uint32_t VW, uint32_t nb,
                 const uint32_t *__restrict__ toks, uint32_t unk,
                 uint16_t *__restrict__ out)
{
  const uint32_t b = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t t = blockIdx.y;
  if (b >= nb)
    return;
  uint32_t tok = toks[t];
  if (tok >= VH)
    tok = unk;
  const size_t blk = (size_t)tok * nb + b;
  const float scale = vkl::h2f (d[blk]);
  const uint4 *src = (const uint4 *)(q + blk * 32);
  const uint4 w0 = src[0], w1 = src[1];
  const uint32_t w[8] = { w0.x, w0.y, w0.z, w0.w, w1.x, w1.y, w1.z, w1.w };
  uint16_t *o = out + (size_t)t * VW + (size_t)b * 32;
#pragma unroll
  for (int i = 0; i < 32; ++i)
    {
      if (b * 32 + i < VW)
        {
          const int8_t v = (int8_t)((w[i >> 2] >> (8 * (i & 3))) & 0xff);
          o[i] = vkl::f2h ((float)v * scale);
        }
    }
}

__global__ void
embed_f16_kernel (const uint16_t *__restrict__ table, uint32_t VH, uint32_t VW,
                  const uint32_t *__restrict__ toks, uint32_t unk,
                  uint16_t *__restrict__ out)
{
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  const uint32_t t = blockIdx.y;
  if (i >= VW)
    return;
  uint32_t tok = toks[t];
  if (tok >= VH)
    tok = unk;
  out[(size_t)t * VW + i] = table[(size_t)tok * VW + i];
}

extern "C" int
vkl_embed_q8_0 (const void *table_planar, uint32_t VH, uint32_t VW,
                const uint32_t *toks, uint32_t n, uint32_t unk, void *out,
                void *stream)
{
  VKL_CHECK_ARG (table_planar && toks && out && VH > 0 && VW > 0);
  VKL_CHECK_ARG (unk < VH && n <= 65535);
  if (n == 0)
    return 0;
  const uint32_t nb = (VW + 31) / 32;
  const uint8_t *p = (const uint8_t *)table_planar;
  embed_q8_kernel<<<dim3 ((nb + 127) / 128, n), dim3 (128), 0,
                    (hipStream_t)stream>>> (
      p, (const uint16_t *)(p + (size_t)VH * nb * 32), VH, VW, nb, toks, unk,
      (uint16_t *)out);
  return vkl_launch_status ();
}

extern "C" int
vkl_embed_f16 (const void *table, uint32_t VH, uint32_t VW,
               const uint32_t *toks, uint32_t n, uint32_t unk, void *out,
               void *stream)
{
  VKL_CHECK_ARG (table && toks && out && VH > 0 && VW > 0);
  VKL_CHECK_ARG (unk < VH && n <= 65535);
  if (n == 0)
    return 0;
  embed_f16_kernel<<<dim3 ((VW + 255) / 256, n), dim3 (256), 0,
                     (hipStream_t)stream>>> ((const uint16_t *)table, VH, VW,
                                             toks, unk, (uint16_t *)out);
  return vkl_launch_status ();
}
