// y[M,N] = x[M,K] W[N,K]^T on the matrix cores (v_mfma_f32_32x32x16_f16),
// fp16 activations, planar Q8_0 or dense fp16 weights, fp32 accumulation.
//
// Workgroup = 4 waves on a BM x 128 output tile (BM = 128 or 64), k-steps of
// 32 (one Q8_0 block).  Per step the x tile and the weight tile go through
// LDS as fp16.  Q8_0 quants enter LDS as exact fp16 integers; the products of
// one block are summed by the MFMA from a zero accumulator and the block
// scale is applied afterwards in fp32 (acc += partial * d), which is the
// reference shader's arithmetic: sum over the block, then times d, in fp32.
// Global loads for step k+1 are issued before
// the MFMAs of step k and written to the other LDS buffer afterwards, so one
// barrier per step suffices.  Each wave owns a (BM/2) x 64 sub-tile: TM x 2
// accumulators of 32x32.
//
// Tiles are numbered so that workgroups that land on the same XCD (id % 8)
// walk neighbouring tiles with the token-row tile index fastest: the weight
// tile they share stays in that XCD's L2.
#include "vkl_common.h"
#include "vkl_gemm.h"

namespace vkl
{
namespace
{
typedef _Float16 half8 __attribute__ ((ext_vector_type (8)));
typedef float float16v __attribute__ ((ext_vector_type (16)));

constexpr int BN = 128, BK = 32;
constexpr int LDK = BK + 8; // LDS row stride in halves (80 B: conflict-free b128 reads)
constexpr int kGemmThreads = 256;

__device__ __forceinline__ uint4
ldg16 (const void *p)
{
  return ldg4 (p);
}

template <int BM, int WT>
struct TileLoads
{
  static constexpr int ACH = BM * 4 / kGemmThreads; // 16-byte chunks of x per thread
  uint4 a[ACH];
  uint4 b[2];  // fp16: two chunks; Q8_0: b[0] = 16 quants
  uint16_t bd; // Q8_0 block scale
};

// weight row (within matrix t) that virtual row v of this workgroup's tile maps to
__device__ __forceinline__ int
tile_row (const GemmArgs &a, int n0, int v, int &mat)
{
  if (a.upgate)
    {
      mat = v >> 6; // 64 up rows, then the matching 64 gate rows
      return n0 + (v & 63);
    }
  return n0 + v;
}

template <int BM, int WT>
__device__ __forceinline__ void
issue_tile (const GemmArgs &a, int zmat, int m0, int n0, int k0,
            TileLoads<BM, WT> &t)
{
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < TileLoads<BM, WT>::ACH; ++i)
    {
      const int c = tid + i * kGemmThreads;
      const int row = c >> 2, seg = c & 3;
      const int m = m0 + row, k = k0 + seg * 8;
      t.a[i] = make_uint4 (0, 0, 0, 0);
      if (m < a.M && k < a.K)
        t.a[i] = ldg16 (a.x + (size_t)m * a.xs + k);
    }
  if (WT == 8)
    {
      const int v = tid >> 1, seg = tid & 1;
      int mat = zmat;
      const int n = tile_row (a, n0, v, mat);
      t.b[0] = make_uint4 (0, 0, 0, 0);
      t.bd = 0;
      if (n < a.N)
        {
          t.b[0] = ldg16 (a.wq[mat] + (size_t)n * a.Kp + k0 + seg * 16);
          t.bd = ldg (a.wd[mat] + (size_t)n * (a.Kp >> 5) + (k0 >> 5));
        }
    }
  else
    {
#pragma unroll
      for (int i = 0; i < 2; ++i)
        {
          const int c = tid + i * kGemmThreads;
          const int v = c >> 2, seg = c & 3;
          int mat = zmat;
          const int n = tile_row (a, n0, v, mat);
          const int k = k0 + seg * 8;
          t.b[i] = make_uint4 (0, 0, 0, 0);
          if (n < a.N && k < a.K)
            t.b[i] = ldg16 (a.wh[mat] + (size_t)n * a.ws + k);
        }
    }
}

template <int BM, int WT>
__device__ __forceinline__ void
store_tile (const TileLoads<BM, WT> &t, uint16_t *As, uint16_t *Bs,
            uint16_t *Ds)
{
  const int tid = threadIdx.x;
#pragma unroll
  for (int i = 0; i < TileLoads<BM, WT>::ACH; ++i)
    {
      const int c = tid + i * kGemmThreads;
      const int row = c >> 2, seg = c & 3;
      *(uint4 *)(As + row * LDK + seg * 8) = t.a[i];
    }
  if (WT == 8)
    {
      const int v = tid >> 1, seg = tid & 1;
      if (seg == 0)
        Ds[v] = t.bd;
      const uint32_t w[4] = { t.b[0].x, t.b[0].y, t.b[0].z, t.b[0].w };
      uint32_t o[8];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        {
          h16x2 lo, hi;
          i8x4_to_h2x2 (w[j], lo, hi);
          o[2 * j] = __builtin_bit_cast (uint32_t, lo);
          o[2 * j + 1] = __builtin_bit_cast (uint32_t, hi);
        }
      uint4 *dst = (uint4 *)(Bs + v * LDK + seg * 16);
      dst[0] = make_uint4 (o[0], o[1], o[2], o[3]);
      dst[1] = make_uint4 (o[4], o[5], o[6], o[7]);
    }
  else
    {
#pragma unroll
      for (int i = 0; i < 2; ++i)
        {
          const int c = tid + i * kGemmThreads;
          const int v = c >> 2, seg = c & 3;
          *(uint4 *)(Bs + v * LDK + seg * 8) = t.b[i];
        }
    }
}

template <int BM, int WT>
__global__ __launch_bounds__ (kGemmThreads) void
gemm_mfma_kernel (const GemmArgs a, int tiles_m, int tiles_n, int per_xcd)
{
  constexpr int TM = BM / 64; // 32-row accumulators per wave along M
  __shared__ __align__ (16) uint16_t As[2][BM * LDK];
  __shared__ __align__ (16) uint16_t Bs[2][BN * LDK];
  __shared__ uint16_t Ds[2][BN]; // Q8_0 block scales of the tile rows

  // XCD-aware tile numbering
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int tile = xcd * per_xcd + j;
  if (j >= per_xcd || tile >= tiles_m * tiles_n)
    return;
  const int tn = tile / tiles_m, tm = tile - tn * tiles_m;
  const int bn_rows = a.upgate ? 64 : BN; // weight rows per matrix and tile
  const int m0 = tm * BM, n0 = tn * bn_rows;
  const int zmat = blockIdx.z;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // virtual weight-tile rows of this wave's two 32-column accumulators
  const int vb0 = a.upgate ? wn * 32 : wn * 64;
  const int vb1 = a.upgate ? 64 + wn * 32 : wn * 64 + 32;

  float16v acc[TM][2];
#pragma unroll
  for (int mi = 0; mi < TM; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[mi][ni][r] = 0.f;

  const int nk = (a.wtype == 8 ? a.Kp : ((a.K + BK - 1) / BK) * BK) / BK;
  TileLoads<BM, WT> t;
  issue_tile<BM, WT> (a, zmat, m0, n0, 0, t);
  store_tile<BM, WT> (t, As[0], Bs[0], Ds[0]);
  __syncthreads ();

  for (int kt = 0; kt < nk; ++kt)
    {
      const int cur = kt & 1;
      if (kt + 1 < nk)
        issue_tile<BM, WT> (a, zmat, m0, n0, (kt + 1) * BK, t);
      const uint16_t *Ac = As[cur], *Bc = Bs[cur];
      half8 af[2][TM], bf[2][2];
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
        {
          const int kof = ks * 16 + (lane >> 5) * 8;
#pragma unroll
          for (int mi = 0; mi < TM; ++mi)
            af[ks][mi] = *(const half8 *)(Ac + (wm * (BM / 2) + mi * 32 + (lane & 31)) * LDK + kof);
          bf[ks][0] = *(const half8 *)(Bc + (vb0 + (lane & 31)) * LDK + kof);
          bf[ks][1] = *(const half8 *)(Bc + (vb1 + (lane & 31)) * LDK + kof);
        }
      if (WT == 8)
        {
          const float sc[2] = { h2f (Ds[cur][vb0 + (lane & 31)]),
                                h2f (Ds[cur][vb1 + (lane & 31)]) };
#pragma unroll
          for (int mi = 0; mi < TM; ++mi)
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
              {
                float16v part;
#pragma unroll
                for (int r = 0; r < 16; ++r)
                  part[r] = 0.f;
                part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (
                    af[0][mi], bf[0][ni], part, 0, 0, 0);
                part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (
                    af[1][mi], bf[1][ni], part, 0, 0, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r)
                  acc[mi][ni][r] += part[r] * sc[ni];
              }
        }
      else
        {
#pragma unroll
          for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int mi = 0; mi < TM; ++mi)
#pragma unroll
              for (int ni = 0; ni < 2; ++ni)
                acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16 (
                    af[ks][mi], bf[ks][ni], acc[mi][ni], 0, 0, 0);
        }
      if (kt + 1 < nk)
        store_tile<BM, WT> (t, As[cur ^ 1], Bs[cur ^ 1], Ds[cur ^ 1]);
      __syncthreads ();
    }

  // epilogue: accumulator register r of lane l is row 8*(r/4) + 4*(l/32) +
  // r%4, column l%32 of its 32x32 block
  uint16_t *y = a.y[a.upgate ? 0 : zmat];
#pragma unroll
  for (int mi = 0; mi < TM; ++mi)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      {
        const int m = m0 + wm * (BM / 2) + mi * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m >= a.M)
          continue;
        if (a.upgate)
          {
            const int n = n0 + wn * 32 + (lane & 31);
            if (n < a.N)
              {
                const float up = acc[mi][0][r], g = acc[mi][1][r];
                y[(size_t)m * a.ys + n] = f2h (silu (g) * up);
              }
            continue;
          }
#pragma unroll
        for (int ni = 0; ni < 2; ++ni)
          {
            const int n = n0 + wn * 64 + ni * 32 + (lane & 31);
            if (n >= a.N)
              continue;
            float v = acc[mi][ni][r];
            const size_t o = (size_t)m * a.ys + n;
            if (a.nmat == 1)
              {
                v = v * a.scale + a.bias;
                if (a.act == 1)
                  v = silu (v);
              }
            uint16_t h = f2h (v);
            if (a.nmat == 1 && a.residual)
              h = f2h (h2f (h) + h2f (ldg (a.residual + o)));
            y[o] = h;
            if (a.nmat == 1 && a.y32)
              a.y32[(size_t)m * a.N + n] = h2f (h);
          }
      }
}

template <int BM, int WT>
int
launch_cfg (const GemmArgs &a, hipStream_t s)
{
  const int tiles_m = (a.M + BM - 1) / BM;
  const int tiles_n = (a.N + (a.upgate ? 64 : BN) - 1) / (a.upgate ? 64 : BN);
  const int tiles = tiles_m * tiles_n;
  const int per_xcd = (tiles + 7) / 8;
  gemm_mfma_kernel<BM, WT>
      <<<dim3 ((unsigned)(per_xcd * 8), 1, (unsigned)(a.upgate ? 1 : a.nmat)),
         dim3 (kGemmThreads), 0, s>>> (a, tiles_m, tiles_n, per_xcd);
  return (int)hipGetLastError ();
}
} // namespace

bool
gemm_mfma_supported (const GemmArgs &a)
{
  if (a.M < kGemmMinRows || a.N <= 0 || a.K <= 0)
    return false;
  // 16-byte vector loads of x (and of fp16 weights)
  if ((a.K % 8) != 0 || (a.xs % 8) != 0 || ((uintptr_t)a.x % 16) != 0)
    return false;
  if (a.wtype == 8)
    return (a.Kp % 32) == 0;
  if (a.wtype == 1)
    {
      if ((a.ws % 8) != 0)
        return false;
      for (int t = 0; t < (a.upgate ? 2 : a.nmat); ++t)
        if (((uintptr_t)a.wh[t] % 16) != 0)
          return false;
      return true;
    }
  return false;
}

int
gemm_mfma_launch (const GemmArgs &a, hipStream_t s)
{
  if (!gemm_mfma_supported (a))
    return (int)hipErrorInvalidValue;
  const bool small = a.M <= 64;
  if (a.wtype == 8)
    return small ? launch_cfg<64, 8> (a, s) : launch_cfg<128, 8> (a, s);
  return small ? launch_cfg<64, 1> (a, s) : launch_cfg<128, 1> (a, s);
}
} // namespace vkl
