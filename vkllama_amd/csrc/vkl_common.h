// Device-side helpers shared by the gfx950 kernels (wave64).
#ifndef VKL_COMMON_H
#define VKL_COMMON_H
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#define VKL_WAVE 64

#define VKL_CHECK_ARG(cond)                                                   \
  do                                                                          \
    {                                                                         \
      if (!(cond))                                                            \
        return (int)hipErrorInvalidValue;                                     \
    }                                                                         \
  while (0)

#define VKL_HIP(expr)                                                         \
  do                                                                          \
    {                                                                         \
      hipError_t e__ = (expr);                                                \
      if (e__ != hipSuccess)                                                  \
        return (int)e__;                                                      \
    }                                                                         \
  while (0)

static inline int
vkl_launch_status ()
{
  return (int)hipGetLastError ();
}

#include <mutex>
namespace vkl
{
// The dynamic-LDS limit of one kernel, raised when a launch needs more than
// any launch before it on that device (a function attribute is kept per
// device); safe to call from several host threads.
struct LdsLimit
{
  std::mutex mu;
  size_t set[16] = {};
  int
  raise (const void *kernel, size_t bytes)
  {
    int dev = 0;
    if (hipGetDevice (&dev) != hipSuccess || dev < 0 || dev >= 16)
      return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock (mu);
    if (bytes > set[dev])
      {
        const hipError_t e
            = hipFuncSetAttribute (kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
        if (e != hipSuccess)
          return (int)e;
        set[dev] = bytes;
      }
    return 0;
  }
};
}

typedef _Float16 h16;
typedef _Float16 h16x2 __attribute__ ((ext_vector_type (2)));

#define VKL_GLOBAL __attribute__ ((address_space (1)))
typedef uint32_t vkl_u32x4 __attribute__ ((ext_vector_type (4)));

namespace vkl
{
// Loads and stores through pointers that were themselves read from memory
// (e.g. a per-layer table of weight pointers) are FLAT accesses unless the
// address space is stated: a flat load also counts against the LDS counter,
// so that waiting for an LDS read would wait for every weight load in flight.
// These helpers pin the global address space.
template <typename T>
__device__ __forceinline__ T
ldg (const T *p)
{
  return *(const VKL_GLOBAL T *)p;
}

template <typename T>
__device__ __forceinline__ void
stg (T *p, T v)
{
  *(VKL_GLOBAL T *)p = v;
}

__device__ __forceinline__ uint4
ldg4 (const void *p)
{
  const vkl_u32x4 v = *(const VKL_GLOBAL vkl_u32x4 *)p;
  return make_uint4 (v.x, v.y, v.z, v.w);
}

// The same for data read once (a weight stream): the non-temporal hint keeps it
// from displacing what the caches hold for re-use.
__device__ __forceinline__ uint4
ldg4_stream (const void *p)
{
  const vkl_u32x4 v = __builtin_nontemporal_load ((const VKL_GLOBAL vkl_u32x4 *)p);
  return make_uint4 (v.x, v.y, v.z, v.w);
}

// Cross-lane data movement by DPP (a modifier of a VALU instruction, a few
// cycles) instead of ds_bpermute (a trip through the LDS crossbar that also
// counts against the LDS counter): v of the lane chosen by CTRL within the
// lane's row of 16.  0xB1 / 0x4E swap neighbours / pairs inside a quad, 0x141
// mirrors a half row (8 lanes), 0x140 a row.
template <int CTRL>
__device__ __forceinline__ float
dpp_get (float v)
{
  return __builtin_bit_cast (
      float, __builtin_amdgcn_update_dpp (0, __builtin_bit_cast (int, v), CTRL, 0xf, 0xf, false));
}

// sum / maximum over groups of LANES (4, 8 or 16) consecutive lanes; every
// lane of a group gets the group's result
template <int LANES>
__device__ __forceinline__ float
row_sum (float v)
{
  v += dpp_get<0xB1> (v);
  v += dpp_get<0x4E> (v);
  if (LANES >= 8)
    v += dpp_get<0x141> (v);
  if (LANES >= 16)
    v += dpp_get<0x140> (v);
  return v;
}

template <int LANES>
__device__ __forceinline__ float
row_max (float v)
{
  v = fmaxf (v, dpp_get<0xB1> (v));
  v = fmaxf (v, dpp_get<0x4E> (v));
  if (LANES >= 8)
    v = fmaxf (v, dpp_get<0x141> (v));
  if (LANES >= 16)
    v = fmaxf (v, dpp_get<0x140> (v));
  return v;
}

__device__ __forceinline__ float
lane_value (float v, int lane)
{
  return __builtin_bit_cast (float, __builtin_amdgcn_readlane (__builtin_bit_cast (int, v), lane));
}

// sum over the 64 lanes of a wave; every lane gets the total: the four rows
// of 16 by DPP, their results through scalar registers.
__device__ __forceinline__ float
wave_sum (float v)
{
  v = row_sum<16> (v);
  return (lane_value (v, 0) + lane_value (v, 16)) + (lane_value (v, 32) + lane_value (v, 48));
}

__device__ __forceinline__ float
wave_max (float v)
{
  v = row_max<16> (v);
  return fmaxf (fmaxf (lane_value (v, 0), lane_value (v, 16)),
                fmaxf (lane_value (v, 32), lane_value (v, 48)));
}

__device__ __forceinline__ float
h2f (uint16_t bits)
{
  return (float)__builtin_bit_cast (h16, bits);
}

__device__ __forceinline__ uint16_t
f2h (float f)
{
  return __builtin_bit_cast (uint16_t, (h16)f); // v_cvt_f16_f32: RNE
}

__device__ __forceinline__ float
silu (float v)
{
  return v / (1.0f + expf (-v));
}

// Four int8 packed in a dword -> two half2 holding the exact integer values.
// (b ^ 0x80) is the byte biased by 128; 0x6400 | byte is the fp16 number
// 1024 + byte, and subtracting 1152 gives the signed value exactly.
__device__ __forceinline__ void
i8x4_to_h2x2 (uint32_t w, h16x2 &lo, h16x2 &hi)
{
  const uint32_t u = w ^ 0x80808080u;
  const uint32_t l = __builtin_amdgcn_perm (0x64646464u, u, 0x04010400u);
  const uint32_t h = __builtin_amdgcn_perm (0x64646464u, u, 0x04030402u);
  const h16x2 bias = { (h16)1152.0f, (h16)1152.0f };
  lo = __builtin_bit_cast (h16x2, l) - bias;
  hi = __builtin_bit_cast (h16x2, h) - bias;
}

// sum_{i<16} x[i] * q[i] with fp32 accumulation (v_dot2_f32_f16: products of
// two fp16 numbers are exact in fp32).  w: 16 int8, x: 16 fp16 as 8 half2.
__device__ __forceinline__ float
dot16_q8 (const uint4 w, const h16x2 *x, float acc)
{
  h16x2 lo, hi;
  i8x4_to_h2x2 (w.x, lo, hi);
  acc = __builtin_amdgcn_fdot2 (lo, x[0], acc, false);
  acc = __builtin_amdgcn_fdot2 (hi, x[1], acc, false);
  i8x4_to_h2x2 (w.y, lo, hi);
  acc = __builtin_amdgcn_fdot2 (lo, x[2], acc, false);
  acc = __builtin_amdgcn_fdot2 (hi, x[3], acc, false);
  i8x4_to_h2x2 (w.z, lo, hi);
  acc = __builtin_amdgcn_fdot2 (lo, x[4], acc, false);
  acc = __builtin_amdgcn_fdot2 (hi, x[5], acc, false);
  i8x4_to_h2x2 (w.w, lo, hi);
  acc = __builtin_amdgcn_fdot2 (lo, x[6], acc, false);
  acc = __builtin_amdgcn_fdot2 (hi, x[7], acc, false);
  return acc;
}

// sum_{i<8} a[i]*b[i], both fp16 (one dwordx4 each)
__device__ __forceinline__ float
dot8_f16 (const uint4 a, const uint4 b, float acc)
{
  acc = __builtin_amdgcn_fdot2 (__builtin_bit_cast (h16x2, a.x),
                                __builtin_bit_cast (h16x2, b.x), acc, false);
  acc = __builtin_amdgcn_fdot2 (__builtin_bit_cast (h16x2, a.y),
                                __builtin_bit_cast (h16x2, b.y), acc, false);
  acc = __builtin_amdgcn_fdot2 (__builtin_bit_cast (h16x2, a.z),
                                __builtin_bit_cast (h16x2, b.z), acc, false);
  acc = __builtin_amdgcn_fdot2 (__builtin_bit_cast (h16x2, a.w),
                                __builtin_bit_cast (h16x2, b.w), acc, false);
  return acc;
}
} // namespace vkl
#endif
