// Small fp16 operators: RMSNorm, RoPE, KV-cache update, softmax, element-wise,
// casts, arg-max/min, slice, transpose.  All of them move a few KiB to a few
// MiB; they exist for the operator classes and for prefill, the decode step
// fuses most of them into its GEMV and attention kernels.
#include "../../include/vkl_hip.h"
#include "vkl_common.h"

namespace
{
// ---- RMSNorm: one workgroup (256 threads) per row ---------------------------
// general form: any row width, the row is read twice
__global__ __launch_bounds__ (256) void
rmsnorm_generic_kernel (const uint16_t *__restrict__ x, const float *__restrict__ w,
                        int W, float eps, uint16_t *__restrict__ out)
{
  __shared__ float part[4];
  const uint16_t *xr = x + (size_t)blockIdx.x * W;
  uint16_t *o = out + (size_t)blockIdx.x * W;
  float s = 0.f;
  for (int i = threadIdx.x; i < W; i += 256)
    {
      const float v = vkl::h2f (xr[i]);
      s += v * v;
    }
  s = vkl::wave_sum (s);
  if ((threadIdx.x & 63) == 0)
    part[threadIdx.x >> 6] = s;
  __syncthreads ();
  const float total = (part[0] + part[1]) + (part[2] + part[3]);
  const float alpha = 1.0f / sqrtf (total / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256)
    {
      const float v = vkl::h2f (xr[i]);
      o[i] = vkl::f2h (v * w[i] * alpha);
    }
}

// rows of W = 8 * n values, n <= 256 * VEC: the row stays in registers between
// the sum of squares and the scaling, and row and weights are requested at
// once (16-byte loads from clamped addresses, no branch around a load)
template <int VEC>
__global__ __launch_bounds__ (256) void
rmsnorm_kernel (const uint16_t *__restrict__ x, const float *__restrict__ w,
                int W, float eps, uint16_t *__restrict__ out)
{
  __shared__ float part[4];
  const uint16_t *xr = x + (size_t)blockIdx.x * W;
  uint16_t *o = out + (size_t)blockIdx.x * W;
  const int nv = W >> 3;
  uint4 v[VEC], g[VEC][2];
#pragma unroll
  for (int j = 0; j < VEC; ++j)
    v[j] = vkl::ldg4 (xr + (size_t)min ((int)threadIdx.x + j * 256, nv - 1) * 8);
#pragma unroll
  for (int j = 0; j < VEC; ++j)
    {
      const float *wp = w + (size_t)min ((int)threadIdx.x + j * 256, nv - 1) * 8;
      g[j][0] = vkl::ldg4 (wp), g[j][1] = vkl::ldg4 (wp + 4);
    }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < VEC; ++j)
    {
      const uint32_t h[4] = { v[j].x, v[j].y, v[j].z, v[j].w };
      float t = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        {
          const float a = vkl::h2f ((uint16_t)(h[i] & 0xffff)), b = vkl::h2f ((uint16_t)(h[i] >> 16));
          t += a * a;
          t += b * b;
        }
      s += (int)threadIdx.x + j * 256 < nv ? t : 0.f;
    }
  s = vkl::wave_sum (s);
  if ((threadIdx.x & 63) == 0)
    part[threadIdx.x >> 6] = s;
  __syncthreads ();
  const float total = (part[0] + part[1]) + (part[2] + part[3]);
  const float alpha = 1.0f / sqrtf (total / (float)W + eps);
#pragma unroll
  for (int j = 0; j < VEC; ++j)
    {
      const int idx = (int)threadIdx.x + j * 256;
      const uint32_t h[4] = { v[j].x, v[j].y, v[j].z, v[j].w };
      const uint32_t gw[8] = { g[j][0].x, g[j][0].y, g[j][0].z, g[j][0].w,
                               g[j][1].x, g[j][1].y, g[j][1].z, g[j][1].w };
      uint32_t r[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        {
          const float a = vkl::h2f ((uint16_t)(h[i] & 0xffff)), b = vkl::h2f ((uint16_t)(h[i] >> 16));
          r[i] = (uint32_t)vkl::f2h (a * __uint_as_float (gw[2 * i]) * alpha)
                 | ((uint32_t)vkl::f2h (b * __uint_as_float (gw[2 * i + 1]) * alpha) << 16);
        }
      if (idx < nv)
        *(uint4 *)(o + (size_t)idx * 8) = make_uint4 (r[0], r[1], r[2], r[3]);
    }
}

// ---- RoPE: one thread per (c, y, pair) --------------------------------------
__global__ void
rope_kernel (uint16_t *__restrict__ x, int H, int W,
             const float *__restrict__ fc, const float *__restrict__ fs,
             uint32_t offset, size_t total)
{
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total)
    return;
  const int half = W / 2;
  const int i = (int)(t % half);
  const size_t row = t / half; // c*H + y
  const int y = (int)(row % H);
  const size_t fi = ((size_t)y + offset) * half + i;
  const float c = fc[fi], s = fs[fi];
  uint32_t *p = (uint32_t *)(x + row * W + 2 * i);
  const uint32_t v = *p;
  const float q0 = vkl::h2f ((uint16_t)(v & 0xffff)), q1 = vkl::h2f ((uint16_t)(v >> 16));
  const float r0 = q0 * c - q1 * s;
  const float r1 = q0 * s + q1 * c;
  *p = (uint32_t)vkl::f2h (r0) | ((uint32_t)vkl::f2h (r1) << 16);
}

__global__ void
kv_update_kernel (uint16_t *__restrict__ cache, const uint16_t *__restrict__ kv,
                  int HO, int H, int W, uint32_t offset, size_t total)
{
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total)
    return;
  const int xw = (int)(t % W);
  const size_t row = t / W;
  const int y = (int)(row % H);
  const size_t c = row / H;
  const uint32_t uy = (offset + (uint32_t)y) % (uint32_t)HO;
  cache[(c * HO + uy) * W + xw] = kv[t];
}

// ---- softmax: one wave per row ----------------------------------------------
__global__ __launch_bounds__ (256) void
softmax_kernel (const uint16_t *__restrict__ x, int H, int W, int seq_mask,
                uint32_t offset, uint16_t *__restrict__ out, size_t rows)
{
  const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows)
    return;
  const int lane = threadIdx.x & 63;
  const uint32_t y = (uint32_t)(row % H);
  const uint16_t *r = x + row * W;
  uint16_t *o = out + row * W;
  // the maximum is taken over masked entries too, as the reference does
  float mx = vkl::h2f (r[0]);
  for (int i = lane; i < W; i += 64)
    mx = fmaxf (mx, vkl::h2f (r[i]));
  mx = vkl::wave_max (mx);
  const uint32_t last = seq_mask > 0 ? y + offset : 0xffffffffu;
  float s = 0.f;
  for (int i = lane; i < W; i += 64)
    if ((uint32_t)i <= last)
      s += expf (vkl::h2f (r[i]) - mx);
  s = vkl::wave_sum (s);
  for (int i = lane; i < W; i += 64)
    {
      uint16_t v = 0;
      if ((uint32_t)i <= last)
        v = vkl::f2h (expf (vkl::h2f (r[i]) - mx) / s);
      o[i] = v;
    }
}

__global__ void
elementwise_kernel (const uint16_t *__restrict__ x, uint16_t *y, size_t n,
                    int op)
{
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n)
    return;
  const float a = vkl::h2f (x[i]), b = vkl::h2f (y[i]);
  float v;
  switch (op)
    {
    case 0: v = a + b; break;
    case 1: v = a - b; break;
    case 2: v = a * b; break;
    default: v = a / b; break;
    }
  y[i] = vkl::f2h (v);
}

__global__ void
elementwise_const_kernel (const uint16_t *x, float alpha, size_t n, int op,
                          uint16_t *out)
{
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n)
    return;
  const float a = vkl::h2f (x[i]);
  float v;
  switch (op)
    {
    case 0: v = a + alpha; break;
    case 1: v = a - alpha; break;
    case 2: v = a * alpha; break;
    default: v = a / alpha; break;
    }
  out[i] = vkl::f2h (v);
}

__global__ void
cast_f16_f32_kernel (const uint16_t *__restrict__ x, float *__restrict__ out,
                     size_t n)
{
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    out[i] = vkl::h2f (x[i]);
}

__global__ void
cast_f32_f16_kernel (const float *__restrict__ x, uint16_t *__restrict__ out,
                     size_t n)
{
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n)
    out[i] = vkl::f2h (x[i]);
}

// ---- arg-max / arg-min: one workgroup per row; the lowest index wins ties ---
__device__ __forceinline__ bool
arg_better (float v, uint32_t i, float bv, uint32_t bi, int op)
{
  if (op == 0 ? v > bv : v < bv)
    return true;
  return v == bv && i < bi;
}

__global__ __launch_bounds__ (256) void
argop_kernel (const uint16_t *__restrict__ x, int W, int op,
              uint32_t *__restrict__ out)
{
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  const uint16_t *r = x + (size_t)blockIdx.x * W;
  float bv = vkl::h2f (r[0]);
  uint32_t bi = 0;
  for (int i = threadIdx.x; i < W; i += 256)
    {
      const float v = vkl::h2f (r[i]);
      if (arg_better (v, (uint32_t)i, bv, bi, op))
        {
          bv = v;
          bi = (uint32_t)i;
        }
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    {
      const float ov = __shfl_xor (bv, o, 64);
      const uint32_t oi = __shfl_xor (bi, o, 64);
      if (arg_better (ov, oi, bv, bi, op))
        {
          bv = ov;
          bi = oi;
        }
    }
  if ((threadIdx.x & 63) == 0)
    {
      sv[threadIdx.x >> 6] = bv;
      si[threadIdx.x >> 6] = bi;
    }
  __syncthreads ();
  if (threadIdx.x == 0)
    {
      for (int w = 1; w < 4; ++w)
        if (arg_better (sv[w], si[w], bv, bi, op))
          {
            bv = sv[w];
            bi = si[w];
          }
      out[blockIdx.x] = bi;
    }
}

__global__ void
slice_kernel (const uint16_t *__restrict__ x, int H, int W, int c0, int h0,
              int w0, int HE, int WE, uint16_t *__restrict__ out, size_t total)
{
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total)
    return;
  const int xw = (int)(t % WE);
  const size_t r = t / WE;
  const int y = (int)(r % HE);
  const size_t c = r / HE;
  out[t] = x[((c + c0) * H + (y + h0)) * W + (xw + w0)];
}

__global__ void
transpose102_kernel (const uint16_t *__restrict__ x, int C, int H, int W,
                     uint16_t *__restrict__ out, size_t total)
{
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total)
    return;
  const int xw = (int)(t % W);
  const size_t r = t / W;
  const int h = (int)(r % H);
  const size_t c = r / H;
  out[((size_t)h * C + c) * W + xw] = x[t];
}

// ---- strided copy of a [C, H, W] box (Concat, ReadKVCache) --------------------
// out[c*dcs + y*dhs + x + doff] = in[c*scs + ((y + h0) % HM)*shs + x]
__global__ void
copy_box_kernel (const uint16_t *__restrict__ in, int H, int W, size_t scs,
                 size_t shs, int h0, int HM, uint16_t *__restrict__ out,
                 size_t dcs, size_t dhs, size_t doff, size_t total)
{
  const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= total)
    return;
  const int xw = (int)(t % W);
  const size_t r = t / W;
  const int y = (int)(r % H);
  const size_t c = r / H;
  const size_t ys = (size_t)(((uint32_t)y + (uint32_t)h0) % (uint32_t)HM);
  out[c * dcs + (size_t)y * dhs + xw + doff] = in[c * scs + ys * shs + xw];
}

// ---- Reduce over the last axis: one wave per row ------------------------------
// op 0 sum, 1 max, 2 min; out = fp16(r * scale)
__global__ __launch_bounds__ (256) void
reduce_rows_kernel (const uint16_t *__restrict__ x, int W, int op, float scale,
                    uint16_t *__restrict__ out, size_t rows)
{
  const size_t row = (size_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows)
    return;
  const int lane = threadIdx.x & 63;
  const uint16_t *r = x + row * (size_t)W;
  float v = op == 0 ? 0.f : vkl::h2f (r[0]);
  for (int i = lane; i < W; i += 64)
    {
      const float e = vkl::h2f (r[i]);
      v = op == 0 ? v + e : (op == 1 ? fmaxf (v, e) : fminf (v, e));
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    {
      const float e = __shfl_xor (v, o, 64);
      v = op == 0 ? v + e : (op == 1 ? fmaxf (v, e) : fminf (v, e));
    }
  if (lane == 0)
    out[row] = vkl::f2h (v * scale);
}

inline unsigned
blocks_for (size_t n, int threads)
{
  return (unsigned)((n + threads - 1) / threads);
}
} // namespace

extern "C" {

int
vkl_rmsnorm_f16 (const void *x, const float *w, int rows, int W, float eps,
                 void *out, void *stream)
{
  VKL_CHECK_ARG (x && w && out && rows > 0 && W > 0);
  const hipStream_t s = (hipStream_t)stream;
  const uint16_t *xp = (const uint16_t *)x;
  uint16_t *op = (uint16_t *)out;
  const bool aligned = (W % 8) == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0
                       && ((uintptr_t)w % 16) == 0;
  if (aligned && W <= 2048)
    rmsnorm_kernel<1><<<dim3 ((unsigned)rows), dim3 (256), 0, s>>> (xp, w, W, eps, op);
  else if (aligned && W <= 4096)
    rmsnorm_kernel<2><<<dim3 ((unsigned)rows), dim3 (256), 0, s>>> (xp, w, W, eps, op);
  else if (aligned && W <= 8192)
    rmsnorm_kernel<4><<<dim3 ((unsigned)rows), dim3 (256), 0, s>>> (xp, w, W, eps, op);
  else
    rmsnorm_generic_kernel<<<dim3 ((unsigned)rows), dim3 (256), 0, s>>> (xp, w, W, eps, op);
  return vkl_launch_status ();
}

int
vkl_rope_f16 (void *x, int C, int H, int W, const float *freqc,
              const float *freqs, uint32_t offset, void *stream)
{
  VKL_CHECK_ARG (x && freqc && freqs && C > 0 && H > 0 && W > 0
                 && (W % 2) == 0);
  const size_t total = (size_t)C * H * (W / 2);
  rope_kernel<<<dim3 (blocks_for (total, 256)), dim3 (256), 0,
                (hipStream_t)stream>>> ((uint16_t *)x, H, W, freqc, freqs,
                                        offset, total);
  return vkl_launch_status ();
}

int
vkl_kv_update_f16 (void *cache, const void *kv, int C, int HO, int H, int W,
                   uint32_t offset, void *stream)
{
  VKL_CHECK_ARG (cache && kv && C > 0 && HO > 0 && H > 0 && W > 0);
  VKL_CHECK_ARG (H <= HO);
  const size_t total = (size_t)C * H * W;
  kv_update_kernel<<<dim3 (blocks_for (total, 256)), dim3 (256), 0,
                     (hipStream_t)stream>>> (
      (uint16_t *)cache, (const uint16_t *)kv, HO, H, W, offset, total);
  return vkl_launch_status ();
}

int
vkl_softmax_f16 (const void *x, int C, int H, int W, int seq_mask,
                 uint32_t offset, void *out, void *stream)
{
  VKL_CHECK_ARG (x && out && C > 0 && H > 0 && W > 0);
  const size_t rows = (size_t)C * H;
  softmax_kernel<<<dim3 (blocks_for (rows, 4)), dim3 (256), 0,
                   (hipStream_t)stream>>> ((const uint16_t *)x, H, W,
                                           seq_mask, offset, (uint16_t *)out,
                                           rows);
  return vkl_launch_status ();
}

int
vkl_elementwise_f16 (const void *x, void *y, size_t n, int op, void *stream)
{
  VKL_CHECK_ARG (x && y && op >= 0 && op <= 3);
  if (n == 0)
    return 0;
  elementwise_kernel<<<dim3 (blocks_for (n, 256)), dim3 (256), 0,
                       (hipStream_t)stream>>> ((const uint16_t *)x,
                                               (uint16_t *)y, n, op);
  return vkl_launch_status ();
}

int
vkl_elementwise_const_f16 (const void *x, float alpha, size_t n, int op,
                           void *out, void *stream)
{
  VKL_CHECK_ARG (x && out && op >= 0 && op <= 3);
  if (n == 0)
    return 0;
  elementwise_const_kernel<<<dim3 (blocks_for (n, 256)), dim3 (256), 0,
                             (hipStream_t)stream>>> (
      (const uint16_t *)x, alpha, n, op, (uint16_t *)out);
  return vkl_launch_status ();
}

int
vkl_cast_f16_f32 (const void *x, float *out, size_t n, void *stream)
{
  VKL_CHECK_ARG (x && out);
  if (n == 0)
    return 0;
  cast_f16_f32_kernel<<<dim3 (blocks_for (n, 256)), dim3 (256), 0,
                        (hipStream_t)stream>>> ((const uint16_t *)x, out, n);
  return vkl_launch_status ();
}

int
vkl_cast_f32_f16 (const float *x, void *out, size_t n, void *stream)
{
  VKL_CHECK_ARG (x && out);
  if (n == 0)
    return 0;
  cast_f32_f16_kernel<<<dim3 (blocks_for (n, 256)), dim3 (256), 0,
                        (hipStream_t)stream>>> (x, (uint16_t *)out, n);
  return vkl_launch_status ();
}

int
vkl_argop_f16 (const void *x, int rows, int W, int op, uint32_t *out,
               void *stream)
{
  VKL_CHECK_ARG (x && out && rows > 0 && W > 0 && (op == 0 || op == 1));
  argop_kernel<<<dim3 ((unsigned)rows), dim3 (256), 0,
                 (hipStream_t)stream>>> ((const uint16_t *)x, W, op, out);
  return vkl_launch_status ();
}

int
vkl_slice_f16 (const void *x, int C, int H, int W, int c0, int h0, int w0,
               int CE, int HE, int WE, void *out, void *stream)
{
  VKL_CHECK_ARG (x && out && C > 0 && H > 0 && W > 0);
  VKL_CHECK_ARG (c0 >= 0 && h0 >= 0 && w0 >= 0 && CE > 0 && HE > 0 && WE > 0);
  VKL_CHECK_ARG (c0 + CE <= C && h0 + HE <= H && w0 + WE <= W);
  const size_t total = (size_t)CE * HE * WE;
  slice_kernel<<<dim3 (blocks_for (total, 256)), dim3 (256), 0,
                 (hipStream_t)stream>>> ((const uint16_t *)x, H, W, c0, h0,
                                         w0, HE, WE, (uint16_t *)out, total);
  return vkl_launch_status ();
}

int
vkl_concat_part_f16 (const void *x, int C, int H, int W, size_t xcs,
                     size_t xhs, void *out, size_t ocs, size_t ohs,
                     size_t out_offset, void *stream)
{
  VKL_CHECK_ARG (x && out && C > 0 && H > 0 && W > 0);
  const size_t total = (size_t)C * H * W;
  copy_box_kernel<<<dim3 (blocks_for (total, 256)), dim3 (256), 0,
                    (hipStream_t)stream>>> ((const uint16_t *)x, H, W, xcs,
                                            xhs, 0, H, (uint16_t *)out, ocs,
                                            ohs, out_offset, total);
  return vkl_launch_status ();
}

int
vkl_read_kvcache_f16 (const void *cache, int C, int H, int W, uint32_t offset,
                      uint32_t len, void *out, void *stream)
{
  VKL_CHECK_ARG (cache && out && C > 0 && H > 0 && W > 0 && len > 0);
  VKL_CHECK_ARG (len <= (uint32_t)H);
  const size_t total = (size_t)C * len * W;
  copy_box_kernel<<<dim3 (blocks_for (total, 256)), dim3 (256), 0,
                    (hipStream_t)stream>>> (
      (const uint16_t *)cache, (int)len, W, (size_t)H * W, (size_t)W,
      (int)(offset % (uint32_t)H), H, (uint16_t *)out, (size_t)len * W,
      (size_t)W, 0, total);
  return vkl_launch_status ();
}

int
vkl_reduce_f16 (const void *x, int C, int H, int W, int op, void *out,
                void *stream)
{
  VKL_CHECK_ARG (x && out && C > 0 && H > 0 && W > 0 && op >= 0 && op <= 3);
  const size_t rows = (size_t)C * H;
  reduce_rows_kernel<<<dim3 (blocks_for (rows, 4)), dim3 (256), 0,
                       (hipStream_t)stream>>> (
      (const uint16_t *)x, W, op == 3 ? 0 : op,
      op == 3 ? 1.0f / (float)W : 1.0f, (uint16_t *)out, rows);
  return vkl_launch_status ();
}

int
vkl_transpose102_f16 (const void *x, int C, int H, int W, void *out,
                      void *stream)
{
  VKL_CHECK_ARG (x && out && C > 0 && H > 0 && W > 0);
  const size_t total = (size_t)C * H * W;
  transpose102_kernel<<<dim3 (blocks_for (total, 256)), dim3 (256), 0,
                        (hipStream_t)stream>>> ((const uint16_t *)x, C, H, W,
                                                (uint16_t *)out, total);
  return vkl_launch_status ();
}
}
