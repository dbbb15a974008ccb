// FP16 activations x Q8_0 (planar) weights: y = x W^T for small M.
//
// One wave owns R weight rows of each of the NMAT matrices and sweeps the
// whole K range: lane l handles the 16 quants at k = step*1024 + l*16 (one
// dwordx4 load, half a Q8_0 block), so a wave reads 1 KiB of contiguous
// weights per row and step.  The activation rows sit in LDS as fp16 and are
// shared by the 4 waves of the workgroup.  HBM-bound: 34 bytes per 32
// weights, nothing is read twice at M <= MT.
#include "../../include/vkl_hip.h"
#include "vkl_common.h"
#include "vkl_gemm.h"

namespace
{
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * VKL_WAVE;

struct GemvQ8Args
{
  const uint16_t *x; // [M, K], row stride xs
  size_t xs;
  const uint8_t *wq[3];  // int8 planes [N, Kp]
  const uint16_t *wd[3]; // scale planes [N, nb]
  uint16_t *y[3];        // [M, N], row stride ys
  size_t ys;
  const uint16_t *residual; // [M, N] stride ys, or null
  float *y32;               // [M, N] dense, or null
  int M, N, K, Kp, nb;
  float scale, bias;
  int act;
};

// MODE 0: NMAT=1 plain (scale, bias, act, residual, y32)
// MODE 1: NMAT=3 three independent outputs (k, q, v)
// MODE 2: NMAT=2 out = silu(mat1) * mat0   (mat0 = up, mat1 = gate)
template <int MODE, int NMAT, int R, int MT>
__global__ __launch_bounds__ (kThreads) void
gemv_q8_kernel (const GemvQ8Args a)
{
  extern __shared__ __align__ (16) uint16_t xs_lds[]; // [MT][Kp]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int m0 = blockIdx.y * MT;
  const int Kp = a.Kp;

  for (int i = threadIdx.x; i < MT * Kp; i += kThreads)
    {
      const int m = i / Kp, k = i - m * Kp;
      uint16_t v = 0;
      if (m0 + m < a.M && k < a.K)
        v = a.x[(size_t)(m0 + m) * a.xs + k];
      xs_lds[i] = v;
    }
  __syncthreads ();

  const int n0 = (blockIdx.x * kWaves + wave) * R;
  if (n0 >= a.N)
    return;

  float acc[NMAT][R][MT];
#pragma unroll
  for (int t = 0; t < NMAT; ++t)
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[t][r][m] = 0.f;

  size_t rowq[R], rowd[R];
#pragma unroll
  for (int r = 0; r < R; ++r)
    {
      const int n = min (n0 + r, a.N - 1);
      rowq[r] = (size_t)n * Kp;
      rowd[r] = (size_t)n * a.nb;
    }

  for (int kk = lane * 16; kk < Kp; kk += VKL_WAVE * 16)
    {
      uint4 w[NMAT][R];
      uint16_t d[NMAT][R];
#pragma unroll
      for (int t = 0; t < NMAT; ++t)
#pragma unroll
        for (int r = 0; r < R; ++r)
          {
            w[t][r] = *(const uint4 *)(a.wq[t] + rowq[r] + kk);
            d[t][r] = a.wd[t][rowd[r] + (kk >> 5)];
          }
#pragma unroll
      for (int m = 0; m < MT; ++m)
        {
          const uint4 *xp = (const uint4 *)(xs_lds + m * Kp + kk);
          const uint4 x0 = xp[0], x1 = xp[1];
          const h16x2 xv[8]
              = { __builtin_bit_cast (h16x2, x0.x), __builtin_bit_cast (h16x2, x0.y),
                  __builtin_bit_cast (h16x2, x0.z), __builtin_bit_cast (h16x2, x0.w),
                  __builtin_bit_cast (h16x2, x1.x), __builtin_bit_cast (h16x2, x1.y),
                  __builtin_bit_cast (h16x2, x1.z), __builtin_bit_cast (h16x2, x1.w) };
#pragma unroll
          for (int t = 0; t < NMAT; ++t)
#pragma unroll
            for (int r = 0; r < R; ++r)
              acc[t][r][m] += vkl::dot16_q8 (w[t][r], xv, 0.f) * vkl::h2f (d[t][r]);
        }
    }

#pragma unroll
  for (int t = 0; t < NMAT; ++t)
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m)
        acc[t][r][m] = vkl::wave_sum (acc[t][r][m]);

  if (lane != 0)
    return;
#pragma unroll
  for (int r = 0; r < R; ++r)
    {
      const int n = n0 + r;
      if (n >= a.N)
        break;
#pragma unroll
      for (int m = 0; m < MT; ++m)
        {
          if (m0 + m >= a.M)
            break;
          const size_t o = (size_t)(m0 + m) * a.ys + n;
          if (MODE == 0)
            {
              float v = acc[0][r][m] * a.scale + a.bias;
              if (a.act == 1)
                v = vkl::silu (v);
              uint16_t h = vkl::f2h (v);
              if (a.residual)
                h = vkl::f2h (vkl::h2f (h) + vkl::h2f (a.residual[o]));
              a.y[0][o] = h;
              if (a.y32)
                a.y32[(size_t)(m0 + m) * a.N + n] = vkl::h2f (h);
            }
          else if (MODE == 1)
            {
#pragma unroll
              for (int t = 0; t < NMAT; ++t)
                a.y[t][o] = vkl::f2h (acc[t][r][m]);
            }
          else
            {
              const float up = acc[0][r][m], g = acc[NMAT - 1][r][m];
              a.y[0][o] = vkl::f2h (vkl::silu (g) * up);
            }
        }
    }
}

template <int MODE, int NMAT>
int
launch (const GemvQ8Args &a, hipStream_t s)
{
  constexpr int R = 2;
  const unsigned gx = (unsigned)((a.N + kWaves * R - 1) / (kWaves * R));
  if (a.M == 1)
    {
      const size_t lds = (size_t)a.Kp * 2;
      gemv_q8_kernel<MODE, NMAT, R, 1>
          <<<dim3 (gx, 1), dim3 (kThreads), lds, s>>> (a);
    }
  else
    {
      constexpr int MT = 4;
      const size_t lds = (size_t)MT * a.Kp * 2;
      if (lds > 64 * 1024)
        {
          hipError_t e = hipFuncSetAttribute (
              (const void *)gemv_q8_kernel<MODE, NMAT, R, MT>,
              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
          if (e != hipSuccess)
            return (int)e;
        }
      gemv_q8_kernel<MODE, NMAT, R, MT>
          <<<dim3 (gx, (unsigned)((a.M + MT - 1) / MT)), dim3 (kThreads), lds,
             s>>> (a);
    }
  return vkl_launch_status ();
}

int
fill_common (GemvQ8Args &a, const void *x, int M, int N, int K, size_t xs,
             size_t ys)
{
  VKL_CHECK_ARG (x != nullptr && M > 0 && N > 0 && K > 0);
  VKL_CHECK_ARG (xs >= (size_t)K && ys >= (size_t)N);
  VKL_CHECK_ARG (M <= 65535 * 4);
  a.x = (const uint16_t *)x;
  a.xs = xs;
  a.ys = ys;
  a.M = M;
  a.N = N;
  a.K = K;
  a.nb = (K + 31) / 32;
  a.Kp = a.nb * 32;
  // 4 activation rows of Kp halves must fit the 160 KiB LDS of a CU
  VKL_CHECK_ARG ((size_t)a.Kp * 2 * (M == 1 ? 1 : 4) <= 160 * 1024);
  a.residual = nullptr;
  a.y32 = nullptr;
  a.scale = 1.f;
  a.bias = 0.f;
  a.act = 0;
  return 0;
}

// the same problem on the matrix cores when there are enough token rows
// the problem as the matrix-core launcher takes it
vkl::GemmArgs
gemm_args (const GemvQ8Args &a, int nmat, int upgate)
{
  vkl::GemmArgs g = {};
  g.x = a.x, g.xs = a.xs;
  g.M = a.M, g.N = a.N, g.K = a.K, g.Kp = a.Kp;
  g.wtype = 8, g.nmat = nmat, g.upgate = upgate;
  for (int t = 0; t < 3; ++t)
    g.wq[t] = a.wq[t], g.wd[t] = a.wd[t], g.y[t] = a.y[t];
  g.ys = a.ys;
  g.scale = a.scale, g.bias = a.bias, g.act = a.act;
  g.residual = a.residual, g.y32 = a.y32;
  return g;
}

bool
try_gemm (const GemvQ8Args &a, int nmat, int upgate, hipStream_t s, int &err,
          float *workspace = nullptr, size_t workspace_bytes = 0)
{
  if (a.M < vkl::kGemmMinRows)
    return false;
  vkl::GemmArgs g = gemm_args (a, nmat, upgate);
  g.workspace = workspace, g.workspace_bytes = workspace_bytes;
  if (!vkl::gemm_mfma_supported (g))
    return false;
  err = vkl::gemm_mfma_launch (g, s);
  return true;
}

void
set_mat (GemvQ8Args &a, int t, const void *w, void *y)
{
  const uint8_t *p = (const uint8_t *)w;
  a.wq[t] = p;
  a.wd[t] = (const uint16_t *)(p + (size_t)a.N * a.nb * 32);
  a.y[t] = (uint16_t *)y;
}
} // namespace

namespace
{
// no_alloc: scratch comes from the library's static device array or the call
// is refused; nothing is allocated
int
matmul_q8_0 (const void *x, const void *w_planar, int M, int N, int K, size_t xs,
             size_t ys, float scale, float bias, int act, const void *residual,
             void *y, float *y32, void *stream, bool no_alloc)
{
  GemvQ8Args a = {};
  if (int e = fill_common (a, x, M, N, K, xs, ys))
    return e;
  VKL_CHECK_ARG (w_planar && y && (act == 0 || act == 1));
  set_mat (a, 0, w_planar, y);
  a.wq[1] = a.wq[2] = a.wq[0];
  a.wd[1] = a.wd[2] = a.wd[0];
  a.y[1] = a.y[2] = a.y[0];
  a.scale = scale;
  a.bias = bias;
  a.act = act;
  a.residual = (const uint16_t *)residual;
  a.y32 = y32;
  // one row, plain epilogue: the decode step's streaming kernel
  if (M == 1 && scale == 1.0f && bias == 0.0f && act == 0 && !y32
      && ((uintptr_t)x % 16) == 0 && vkl::decode_gemv_supported (N, K, 8))
    return vkl::decode_gemv_launch (x, w_planar, 8, N, K, residual, y, (hipStream_t)stream);
  float *workspace = nullptr;
  size_t have = 0;
  if (no_alloc && M >= vkl::kGemmMinRows)
    {
      // The plan the allocating entry point would follow (same kernels, same
      // split: the results are then the same bit for bit) must fit the static
      // array; a problem whose partial sums exceed it is refused.
      vkl::GemmArgs g = gemm_args (a, 1, 0);
      workspace = vkl::gemm_static_scratch (&have);
      if (!workspace)
        return (int)hipErrorInvalidSymbol;
      if (vkl::gemm_plan (g).workspace_bytes > have)
        return (int)hipErrorInvalidValue;
    }
  int err = 0;
  if (try_gemm (a, 1, 0, (hipStream_t)stream, err, workspace, have))
    return err;
  return launch<0, 1> (a, (hipStream_t)stream);
}
} // namespace

extern "C" int
vkl_matmul_q8_0 (const void *x, const void *w_planar, int M, int N, int K,
                 size_t xs, size_t ys, float scale, float bias, int act,
                 const void *residual, void *y, float *y32, void *stream)
{
  return matmul_q8_0 (x, w_planar, M, N, K, xs, ys, scale, bias, act, residual, y, y32, stream,
                      false);
}

extern "C" int
vkl_matmul_q8_0_noalloc (const void *x, const void *w_planar, int M, int N, int K,
                         size_t xs, size_t ys, float scale, float bias, int act,
                         const void *residual, void *y, float *y32, void *stream)
{
  return matmul_q8_0 (x, w_planar, M, N, K, xs, ys, scale, bias, act, residual, y, y32, stream,
                      true);
}

extern "C" int
vkl_kqv_q8_0 (const void *x, const void *wk, const void *wq, const void *wv,
              int M, int N, int K, void *k, void *q, void *v, void *stream)
{
  GemvQ8Args a = {};
  if (int e = fill_common (a, x, M, N, K, (size_t)K, (size_t)N))
    return e;
  VKL_CHECK_ARG (wk && wq && wv && k && q && v);
  set_mat (a, 0, wk, k);
  set_mat (a, 1, wq, q);
  set_mat (a, 2, wv, v);
  int err = 0;
  if (try_gemm (a, 3, 0, (hipStream_t)stream, err))
    return err;
  return launch<1, 3> (a, (hipStream_t)stream);
}

extern "C" int
vkl_ffn_upgate_q8_0 (const void *x, const void *wup, const void *wgate, int M,
                     int N, int K, void *out, void *stream)
{
  GemvQ8Args a = {};
  if (int e = fill_common (a, x, M, N, K, (size_t)K, (size_t)N))
    return e;
  VKL_CHECK_ARG (wup && wgate && out);
  set_mat (a, 0, wup, out);
  set_mat (a, 1, wgate, out);
  a.wq[2] = a.wq[0];
  a.wd[2] = a.wd[0];
  a.y[2] = a.y[0];
  int err = 0;
  if (try_gemm (a, 1, 1, (hipStream_t)stream, err))
    return err;
  return launch<2, 2> (a, (hipStream_t)stream);
}
