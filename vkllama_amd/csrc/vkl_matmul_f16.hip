// fp16 x fp16 products with fp32 accumulation:
//   tb: Y[c,m,n] = act(scale * sum_k A[c,m,k] B[c,n,k] + bias)   (B transposed)
//   nn: Y[c,m,n] = act(scale * sum_k A[c,m,k] B[c,k,n] + bias)
// plus the fused FP16 up/gate product of the feed-forward block.  Operands are
// strided views (element strides), which is how the attention scores read the
// KV cache in place.
#include "../../include/vkl_hip.h"
#include "vkl_common.h"
#include "vkl_gemm.h"

namespace
{
struct TbArgs
{
  const uint16_t *a, *b, *b2; // b2: second matrix for the up/gate product
  uint16_t *y;
  const uint16_t *residual;
  float *y32;
  int C, M, N, K;
  size_t acs, ahs, bcs, bhs, ycs, yhs;
  float scale, bias;
  int act;
  int lpr_log2; // lanes per output = 1 << lpr_log2
  size_t total; // C*M*N
};

// A group of LPR lanes computes one output; lane j of the group takes the
// 8-element chunks j, j+LPR, ... of the K range (dwordx4 loads of both
// operands), then the group is reduced with xor-shuffles.
template <bool UPGATE, bool VEC>
__global__ __launch_bounds__ (256) void
matmul_tb_kernel (const TbArgs p)
{
  const int lpr = 1 << p.lpr_log2;
  const size_t gid = ((size_t)blockIdx.x * 256 + threadIdx.x) >> p.lpr_log2;
  const int sub = threadIdx.x & (lpr - 1);
  const bool live = gid < p.total;
  const size_t g = live ? gid : p.total - 1;
  const int n = (int)(g % p.N);
  const size_t cm = g / p.N;
  const int m = (int)(cm % p.M);
  const size_t c = cm / p.M;
  const uint16_t *ar = p.a + c * p.acs + (size_t)m * p.ahs;
  const uint16_t *br = p.b + c * p.bcs + (size_t)n * p.bhs;
  const uint16_t *br2 = UPGATE ? p.b2 + c * p.bcs + (size_t)n * p.bhs : br;
  float s0 = 0.f, s1 = 0.f;
  if (VEC)
    {
      for (int k = sub * 8; k < p.K; k += lpr * 8)
        {
          const uint4 av = *(const uint4 *)(ar + k);
          s0 = vkl::dot8_f16 (av, *(const uint4 *)(br + k), s0);
          if (UPGATE)
            s1 = vkl::dot8_f16 (av, *(const uint4 *)(br2 + k), s1);
        }
    }
  else
    {
      for (int k = sub; k < p.K; k += lpr)
        {
          const float av = vkl::h2f (ar[k]);
          s0 += av * vkl::h2f (br[k]);
          if (UPGATE)
            s1 += av * vkl::h2f (br2[k]);
        }
    }
  for (int o = lpr >> 1; o > 0; o >>= 1)
    {
      s0 += __shfl_xor (s0, o, 64);
      if (UPGATE)
        s1 += __shfl_xor (s1, o, 64);
    }
  if (!live || sub != 0)
    return;
  const size_t o = c * p.ycs + (size_t)m * p.yhs + n;
  if (UPGATE)
    {
      p.y[o] = vkl::f2h (vkl::silu (s1) * s0);
      return;
    }
  float v = s0 * p.scale + p.bias;
  if (p.act == 1)
    v = vkl::silu (v);
  uint16_t h = vkl::f2h (v);
  if (p.residual)
    h = vkl::f2h (vkl::h2f (h) + vkl::h2f (p.residual[g]));
  p.y[o] = h;
  if (p.y32)
    p.y32[g] = vkl::h2f (h);
}

struct NnArgs
{
  const uint16_t *a, *b;
  uint16_t *y;
  int C, M, N, K;
  size_t acs, ahs, bcs, bhs, ycs, yhs;
  float scale, bias;
  int act;
};

// grid (ceil(N/64), M, C), 256 threads: wave w takes k = w, w+4, ...; lane =
// output column, so B rows are read coalesced; partial sums meet in LDS.
__global__ __launch_bounds__ (256) void
matmul_nn_kernel (const NnArgs p)
{
  __shared__ float part[4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = blockIdx.x * 64 + lane;
  const int m = blockIdx.y, c = blockIdx.z;
  const uint16_t *ar = p.a + (size_t)c * p.acs + (size_t)m * p.ahs;
  const uint16_t *bc = p.b + (size_t)c * p.bcs + n;
  float s = 0.f;
  if (n < p.N)
    for (int k = wave; k < p.K; k += 4)
      s += vkl::h2f (ar[k]) * vkl::h2f (bc[(size_t)k * p.bhs]);
  part[wave][lane] = s;
  __syncthreads ();
  if (wave != 0 || n >= p.N)
    return;
  float v = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
  v = v * p.scale + p.bias;
  if (p.act == 1)
    v = vkl::silu (v);
  p.y[(size_t)c * p.ycs + (size_t)m * p.yhs + n] = vkl::f2h (v);
}

int
launch_tb (TbArgs &p, bool upgate, hipStream_t s)
{
  p.total = (size_t)p.C * p.M * p.N;
  const bool vec = (p.K % 8) == 0 && (p.acs % 8) == 0 && (p.ahs % 8) == 0
                   && (p.bcs % 8) == 0 && (p.bhs % 8) == 0
                   && ((uintptr_t)p.a % 16) == 0 && ((uintptr_t)p.b % 16) == 0
                   && (!upgate || ((uintptr_t)p.b2 % 16) == 0);
  const int chunks = vec ? (p.K + 7) / 8 : p.K;
  int l2 = 0;
  while ((1 << l2) < chunks && l2 < 6)
    ++l2;
  p.lpr_log2 = l2;
  const size_t threads = p.total << l2;
  const size_t blocks = (threads + 255) / 256;
  VKL_CHECK_ARG (blocks <= 0x7fffffffu);
  const dim3 g ((unsigned)blocks), b (256);
  if (upgate)
    {
      if (vec)
        matmul_tb_kernel<true, true><<<g, b, 0, s>>> (p);
      else
        matmul_tb_kernel<true, false><<<g, b, 0, s>>> (p);
    }
  else
    {
      if (vec)
        matmul_tb_kernel<false, true><<<g, b, 0, s>>> (p);
      else
        matmul_tb_kernel<false, false><<<g, b, 0, s>>> (p);
    }
  return vkl_launch_status ();
}
} // namespace

extern "C" int
vkl_matmul_f16_tb (const void *a, const void *b, int C, int M, int N, int K,
                   size_t acs, size_t ahs, size_t bcs, size_t bhs, size_t ycs,
                   size_t yhs, float scale, float bias, int act,
                   const void *residual, void *y, float *y32, void *stream)
{
  VKL_CHECK_ARG (a && b && y && C > 0 && M > 0 && N > 0 && K > 0);
  VKL_CHECK_ARG (act == 0 || act == 1);
  VKL_CHECK_ARG (ahs >= (size_t)K && bhs >= (size_t)K && yhs >= (size_t)N);
  TbArgs p = {};
  p.a = (const uint16_t *)a;
  p.b = (const uint16_t *)b;
  p.b2 = nullptr;
  p.y = (uint16_t *)y;
  p.residual = (const uint16_t *)residual;
  p.y32 = y32;
  p.C = C, p.M = M, p.N = N, p.K = K;
  p.acs = acs, p.ahs = ahs, p.bcs = bcs, p.bhs = bhs, p.ycs = ycs, p.yhs = yhs;
  p.scale = scale, p.bias = bias, p.act = act;
  if (M >= (C > 1 ? vkl::kGemmMinRowsBatched : vkl::kGemmMinRowsF16))
    {
      // many rows (a projection, or the scores of a prompt pass): matrix cores
      vkl::GemmArgs g = {};
      g.batch = C, g.xbs = acs, g.wbs = bcs, g.ybs = ycs;
      g.x = p.a, g.xs = ahs;
      g.M = M, g.N = N, g.K = K, g.Kp = (K + 31) / 32 * 32;
      g.wtype = 1, g.nmat = 1, g.upgate = 0;
      g.wh[0] = g.wh[1] = g.wh[2] = p.b;
      g.ws = bhs;
      g.y[0] = g.y[1] = g.y[2] = p.y;
      g.ys = yhs;
      g.scale = scale, g.bias = bias, g.act = act;
      g.residual = p.residual, g.y32 = y32;
      if (vkl::gemm_mfma_supported (g))
        return vkl::gemm_mfma_launch (g, (hipStream_t)stream);
    }
  return launch_tb (p, false, (hipStream_t)stream);
}

extern "C" int
vkl_ffn_upgate_f16 (const void *x, const void *wup, const void *wgate, int M,
                    int N, int K, void *out, void *stream)
{
  VKL_CHECK_ARG (x && wup && wgate && out && M > 0 && N > 0 && K > 0);
  TbArgs p = {};
  p.a = (const uint16_t *)x;
  p.b = (const uint16_t *)wup;
  p.b2 = (const uint16_t *)wgate;
  p.y = (uint16_t *)out;
  p.C = 1, p.M = M, p.N = N, p.K = K;
  p.acs = 0, p.ahs = (size_t)K, p.bcs = 0, p.bhs = (size_t)K;
  p.ycs = 0, p.yhs = (size_t)N;
  p.scale = 1.f, p.bias = 0.f, p.act = 0;
  if (M >= vkl::kGemmMinRowsF16)
    {
      vkl::GemmArgs g = {};
      g.x = p.a, g.xs = (size_t)K;
      g.M = M, g.N = N, g.K = K, g.Kp = (K + 31) / 32 * 32;
      g.wtype = 1, g.nmat = 1, g.upgate = 1;
      g.wh[0] = g.wh[2] = p.b, g.wh[1] = p.b2;
      g.ws = (size_t)K;
      g.y[0] = g.y[1] = g.y[2] = p.y;
      g.ys = (size_t)N;
      g.scale = 1.f;
      if (vkl::gemm_mfma_supported (g))
        return vkl::gemm_mfma_launch (g, (hipStream_t)stream);
    }
  return launch_tb (p, true, (hipStream_t)stream);
}

extern "C" int
vkl_matmul_f16_nn (const void *a, const void *b, int C, int M, int N, int K,
                   size_t acs, size_t ahs, size_t bcs, size_t bhs, size_t ycs,
                   size_t yhs, float scale, float bias, int act, void *y,
                   void *stream)
{
  VKL_CHECK_ARG (a && b && y && C > 0 && M > 0 && N > 0 && K > 0);
  VKL_CHECK_ARG (act == 0 || act == 1);
  VKL_CHECK_ARG (ahs >= (size_t)K && bhs >= (size_t)N && yhs >= (size_t)N);
  VKL_CHECK_ARG (M <= 65535 && C <= 65535);
  NnArgs p = {};
  p.a = (const uint16_t *)a;
  p.b = (const uint16_t *)b;
  p.y = (uint16_t *)y;
  p.C = C, p.M = M, p.N = N, p.K = K;
  p.acs = acs, p.ahs = ahs, p.bcs = bcs, p.bhs = bhs, p.ycs = ycs, p.yhs = yhs;
  p.scale = scale, p.bias = bias, p.act = act;
  if (M >= (C > 1 ? vkl::kGemmMinRowsBatched : vkl::kGemmMinRowsF16))
    {
      vkl::GemmArgs g = {};
      g.batch = C, g.xbs = acs, g.wbs = bcs, g.ybs = ycs;
      g.x = p.a, g.xs = ahs;
      g.M = M, g.N = N, g.K = K, g.Kp = (K + 31) / 32 * 32;
      g.wtype = 2, g.nmat = 1, g.upgate = 0;
      g.wh[0] = g.wh[1] = g.wh[2] = p.b;
      g.ws = bhs;
      g.y[0] = g.y[1] = g.y[2] = p.y;
      g.ys = yhs;
      g.scale = scale, g.bias = bias, g.act = act;
      if (vkl::gemm_mfma_supported (g))
        return vkl::gemm_mfma_launch (g, (hipStream_t)stream);
    }
  matmul_nn_kernel<<<dim3 ((unsigned)((N + 63) / 64), (unsigned)M, (unsigned)C),
                     dim3 (256), 0, (hipStream_t)stream>>> (p);
  return vkl_launch_status ();
}
