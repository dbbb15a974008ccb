// Host fp16 helpers with the behaviour of the reference's src/core/float.h:
// __fp32_to_fp16 truncates the mantissa (src/core/float.h:86-110), clamps
// magnitudes above 65504 to the largest normal (:65-71) and maps values below
// the smallest subnormal to +0 (:74-78); __fp16_to_fp32 is exact.
// __fp32_to_fp16_rne is the round-to-nearest-even conversion the device uses.
#ifndef __VKLLAMA_FLOAT_H__
#define __VKLLAMA_FLOAT_H__
#include <math.h>
#include <stdint.h>
#include <string.h>

typedef union
{
  uint16_t u16;
} __attribute__ ((packed)) __vkllama_fp16_t;

typedef __vkllama_fp16_t __pack16_t;

inline __vkllama_fp16_t
__fp32_to_fp16 (float fp32)
{
  uint32_t u;
  memcpy (&u, &fp32, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const uint32_t exp = (u >> 23) & 0xffu, frac = u & 0x7fffffu;
  const float mag = fabsf (fp32);
  __vkllama_fp16_t out = { 0 };
  if (exp == 0 && frac == 0)
    out.u16 = sign;
  else if (isnan (fp32))
    out.u16 = (uint16_t)(sign | 0x7c01u);
  else if (isinf (fp32))
    out.u16 = (uint16_t)(sign | 0x7c00u);
  else if (mag > 65504.0f)
    out.u16 = (uint16_t)(sign | 0x7bffu);
  else if (mag < 5.96046448e-8f)
    out.u16 = 0;
  else if (mag < 6.103515625e-5f)
    out.u16 = (uint16_t)(sign | (((frac >> 14) + 512u) & 0x3ffu));
  else
    out.u16 = (uint16_t)(sign | ((exp - 127u + 15u) << 10) | (frac >> 13));
  return out;
}

inline float
__fp16_to_fp32 (uint16_t const value)
{
  const uint32_t sign = ((uint32_t)value & 0x8000u) << 16;
  const uint32_t exp = (value >> 10) & 0x1fu, frac = value & 0x3ffu;
  uint32_t u;
  float f;
  if (exp == 0)
    {
      f = (float)frac * 5.9604644775390625e-8f;
      memcpy (&u, &f, 4);
      u |= sign;
    }
  else if (exp == 0x1f)
    u = sign | 0x7f800000u | (frac ? 1u : 0u);
  else
    u = sign | ((exp - 15u + 127u) << 23) | (frac << 13);
  memcpy (&f, &u, 4);
  return f;
}

inline __vkllama_fp16_t
__fp32_to_fp16_rne (float f)
{
  uint32_t x;
  memcpy (&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  x &= 0x7fffffffu;
  uint32_t o;
  if (x >= ((127u + 16u) << 23))
    o = x > (255u << 23) ? 0x7e00u : 0x7c00u;
  else if (x < (113u << 23))
    {
      const uint32_t magic_u = ((127u - 15u) + (23u - 10u) + 1u) << 23;
      float magic, v;
      memcpy (&magic, &magic_u, 4);
      memcpy (&v, &x, 4);
      v += magic;
      memcpy (&x, &v, 4);
      o = x - magic_u;
    }
  else
    {
      const uint32_t odd = (x >> 13) & 1u;
      x += ((uint32_t)(15 - 127) << 23) + 0xfffu + odd;
      o = x >> 13;
    }
  __vkllama_fp16_t out = { (uint16_t)(o | sign) };
  return out;
}
#endif
