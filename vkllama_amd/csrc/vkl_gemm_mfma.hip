// y[M,N] = x[M,K] W[N,K]^T on the matrix cores (v_mfma_f32_32x32x16_f16),
// fp16 activations, planar Q8_0 or dense fp16 weights, fp32 accumulation;
// also batched fp16 x fp16 products with the second operand stored [N, K]
// (attention scores) or [K, N] (probabilities times V).
//
// Workgroup = 4 waves on a BM x 128 output tile (BM = 128 or 64), k-steps of
// 32 (one Q8_0 block).  Per step the x tile and the weight tile go through
// LDS as fp16.  Q8_0 quants enter LDS as exact fp16 integers; the products of
// one block are summed by the MFMA from a zero accumulator and the block
// scale is applied afterwards in fp32 (acc += partial * d), which is the
// reference shader's arithmetic: sum over the block, then times d, in fp32.
// Global loads run several k-steps ahead in registers and are written to the
// other LDS buffer after the MFMAs of the current step, so one barrier per
// step suffices.  Each wave owns a (BM/2) x 64 sub-tile: TM x 2
// accumulators of 32x32.
//
// Tiles are numbered so that workgroups that land on the same XCD (id % 8)
// walk neighbouring tiles with the token-row tile index fastest: the weight
// tile they share stays in that XCD's L2.
#include "../../include/vkl_hip.h"
#include "vkl_common.h"
#include "vkl_gemm.h"
#include <algorithm>
#include <map>
#include <mutex>
#include <utility>

namespace vkl
{
namespace
{
typedef _Float16 half8 __attribute__ ((ext_vector_type (8)));
typedef float float16v __attribute__ ((ext_vector_type (16)));

constexpr int BN = 128;
// k extent of a step: 64.  For fp16 operands the eight 16-byte chunks of a
// tile row are then one full 128-byte cache line (with 32, every request is
// half a line and the L2 delivers half the bytes per cycle); for Q8_0 a step
// holds two blocks, each with its own scale (one block per step measured
// slower: half the products per barrier).
template <int WT> struct Geo
{
  static constexpr int BK = 64;
  static constexpr int CPR = BK / 8;  // 16-byte chunks per tile row
  static constexpr int LDK = BK + 8;  // LDS row stride in halves: 144 bytes,
                                      // conflict-free 16-byte accesses
  static constexpr int NB = WT == 8 ? 2 : BN * CPR / 256; // weight chunks per thread
};
constexpr int kGemmThreads = 256;
// fewer full-height tiles than this: half-height tiles; workgroups a launch
// should have at least (two per compute unit): else the k range is split too
constexpr int kGemmFewTiles = 384;
constexpr int kGemmSplitTarget = 512;
// k-tiles in flight in registers: more for the small-M configuration, where
// few workgroups run and each has to hide the memory latency alone
template <int BM> struct GemmDepth
{
  static constexpr int value = BM <= 64 ? 4 : 2;
};

__device__ __forceinline__ uint4
ldg16 (const void *p)
{
  return ldg4 (p);
}

__device__ __align__ (16) const uint32_t g_zero_chunk[4] = { 0, 0, 0, 0 };

template <int BM, int WT>
struct TileLoads
{
  static constexpr int ACH = BM * Geo<WT>::CPR / kGemmThreads; // 16-byte chunks of x per thread
  static constexpr int NB = Geo<WT>::NB;
  uint4 a[ACH];
  uint4 b[NB]; // fp16: weight chunks; Q8_0: the 32 quants of one block
  uint16_t bd; // Q8_0: its scale
};

// Per-thread source addresses of the tile loads.  They depend on k only
// through an added offset, so they are worked out once, before the k loop:
// in particular the choice among the matrices of a fused launch (a pointer
// picked from the argument block by a per-lane index) must not sit inside
// the loop, where the wait for that pointer would also wait for every tile
// load in flight.
template <int BM, int WT>
struct TileAddr
{
  static constexpr int ACH = BM * Geo<WT>::CPR / kGemmThreads;
  static constexpr int NB = Geo<WT>::NB;
  const uint16_t *a[ACH]; // x chunk at k = 0, or null beyond M
  int ak[ACH];            // its column offset within a k-step
  const uint8_t *bq;      // Q8_0: quants of this thread's row and block (0 or 1 of a step) at k = 0
  const uint16_t *bd;     // Q8_0: that block's scale
  int bko;                // Q8_0: 0 or 32, the block's offset within a step
  const uint16_t *b[NB];  // fp16: chunk pointers at k = 0
  int bk[NB];             // fp16 [N, K]: column offset; [K, N]: row offset
};

__device__ __forceinline__ const void *
pick3 (const void *p0, const void *p1, const void *p2, int i)
{
  return i == 0 ? p0 : (i == 1 ? p1 : p2);
}

template <int BM, int WT>
__device__ __forceinline__ void
tile_addresses (const GemmArgs &a, size_t xoff, size_t woff, int zmat, int m0,
                int n0, TileAddr<BM, WT> &ta)
{
  const int tid = threadIdx.x;
  constexpr int CPR = Geo<WT>::CPR, NB = Geo<WT>::NB;
#pragma unroll
  for (int i = 0; i < TileAddr<BM, WT>::ACH; ++i)
    {
      const int c = tid + i * kGemmThreads;
      const int m = m0 + c / CPR;
      ta.ak[i] = (c % CPR) * 8;
      ta.a[i] = m < a.M ? a.x + xoff + (size_t)m * a.xs + ta.ak[i] : nullptr;
    }
  ta.bq = nullptr, ta.bd = nullptr, ta.bko = 0;
#pragma unroll
  for (int i = 0; i < NB; ++i)
    ta.b[i] = nullptr, ta.bk[i] = 0;
  if (WT == 8)
    {
      const int v = tid >> 1, blk = tid & 1;
      const int mat = a.upgate ? (v >> 6) : zmat;
      const int n = a.upgate ? n0 + (v & 63) : n0 + v;
      ta.bko = blk * 32;
      if (n < a.N)
        {
          ta.bq = (const uint8_t *)pick3 (a.wq[0], a.wq[1], a.wq[2], mat)
                  + (size_t)n * a.Kp + blk * 32;
          ta.bd = (const uint16_t *)pick3 (a.wd[0], a.wd[1], a.wd[2], mat)
                  + (size_t)n * (a.Kp >> 5) + blk;
        }
    }
  else if (WT == 2)
    {
#pragma unroll
      for (int i = 0; i < NB; ++i)
        {
          const int c = tid + i * kGemmThreads;
          const int n = n0 + (c & 15) * 8;
          ta.bk[i] = c >> 4;
          if (n < a.N)
            ta.b[i] = (const uint16_t *)pick3 (a.wh[0], a.wh[1], a.wh[2], zmat)
                      + woff + (size_t)ta.bk[i] * a.ws + n;
        }
    }
  else
    {
#pragma unroll
      for (int i = 0; i < NB; ++i)
        {
          const int c = tid + i * kGemmThreads;
          const int v = c / CPR;
          const int mat = a.upgate ? (v >> 6) : zmat;
          const int n = a.upgate ? n0 + (v & 63) : n0 + v;
          ta.bk[i] = (c % CPR) * 8;
          if (n < a.N)
            ta.b[i] = (const uint16_t *)pick3 (a.wh[0], a.wh[1], a.wh[2], mat)
                      + woff + (size_t)n * a.ws + ta.bk[i];
        }
    }
}

// Every load is issued unconditionally: with no branch around a load the
// compiler can count the loads in flight and wait for exactly the tile it
// needs instead of for all of them.  A chunk outside the matrices (rows
// beyond M or N, columns beyond K) is read from a block of zeros instead, so
// nothing has to be masked after the load: a select on loaded data would be
// scheduled early and wait for the newest tile, which leaves one k-step of
// look-ahead whatever the depth.
template <int BM, int WT>
__device__ __forceinline__ void
issue_tile (const GemmArgs &a, const TileAddr<BM, WT> &ta, int k0,
            TileLoads<BM, WT> &t)
{
  const void *zeros = g_zero_chunk;
#pragma unroll
  for (int i = 0; i < TileLoads<BM, WT>::ACH; ++i)
    {
      const bool v = ta.a[i] != nullptr && k0 + ta.ak[i] < a.K;
      t.a[i] = ldg16 (v ? (const void *)(ta.a[i] + k0) : zeros);
    }
  if (WT == 8)
    {
      // rows beyond N, blocks beyond K: zero quants and a zero scale
      const bool v = ta.bq != nullptr && k0 + ta.bko < a.Kp;
      t.b[0] = ldg16 (v ? (const void *)(ta.bq + k0) : zeros);
      t.b[1] = ldg16 (v ? (const void *)(ta.bq + k0 + 16) : zeros);
      t.bd = ldg (v ? ta.bd + (k0 >> 5) : (const uint16_t *)zeros);
    }
  else
    {
#pragma unroll
      for (int i = 0; i < Geo<WT>::NB; ++i)
        {
          const bool v = ta.b[i] != nullptr && k0 + ta.bk[i] < a.K;
          t.b[i] = ldg16 (v ? (const void *)(ta.b[i] + (WT == 2 ? (size_t)k0 * a.ws : (size_t)k0))
                            : zeros);
        }
    }
}

template <int BM, int WT>
__device__ __forceinline__ void
store_tile (const TileLoads<BM, WT> &t, uint16_t *As, uint16_t *Bs,
            uint16_t *Ds)
{
  const int tid = threadIdx.x;
  constexpr int CPR = Geo<WT>::CPR, LDK = Geo<WT>::LDK, NB = Geo<WT>::NB;
#pragma unroll
  for (int i = 0; i < TileLoads<BM, WT>::ACH; ++i)
    {
      const int c = tid + i * kGemmThreads;
      const int row = c / CPR, seg = c % CPR;
      *(uint4 *)(As + row * LDK + seg * 8) = t.a[i];
    }
  if (WT == 8)
    {
      const int v = tid >> 1, blk = tid & 1;
      Ds[v * 2 + blk] = t.bd;
      const uint32_t w[8] = { t.b[0].x, t.b[0].y, t.b[0].z, t.b[0].w,
                              t.b[1].x, t.b[1].y, t.b[1].z, t.b[1].w };
      uint32_t o[16];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        {
          h16x2 lo, hi;
          i8x4_to_h2x2 (w[j], lo, hi);
          o[2 * j] = __builtin_bit_cast (uint32_t, lo);
          o[2 * j + 1] = __builtin_bit_cast (uint32_t, hi);
        }
      uint4 *dst = (uint4 *)(Bs + v * LDK + blk * 32);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        dst[j] = make_uint4 (o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]);
    }
  else if (WT == 2)
    {
      // transpose on the way in: LDS holds the tile as [column][k]
#pragma unroll
      for (int i = 0; i < NB; ++i)
        {
          const int c = tid + i * kGemmThreads;
          const int kr = c >> 4, v = (c & 15) * 8;
          const uint32_t w[4] = { t.b[i].x, t.b[i].y, t.b[i].z, t.b[i].w };
#pragma unroll
          for (int j = 0; j < 4; ++j)
            {
              Bs[(v + 2 * j) * LDK + kr] = (uint16_t)(w[j] & 0xffff);
              Bs[(v + 2 * j + 1) * LDK + kr] = (uint16_t)(w[j] >> 16);
            }
        }
    }
  else
    {
#pragma unroll
      for (int i = 0; i < NB; ++i)
        {
          const int c = tid + i * kGemmThreads;
          const int v = c / CPR, seg = c % CPR;
          *(uint4 *)(Bs + v * LDK + seg * 8) = t.b[i];
        }
    }
}

template <int BM, int WT>
__device__ __forceinline__ void
gemm_step (const GemmArgs &a, const TileAddr<BM, WT> &ta, int kbase, int kt, int nk,
           const uint16_t *Ac, const uint16_t *Bc, const uint16_t *Dc,
           uint16_t *An, uint16_t *Bn, uint16_t *Dn, TileLoads<BM, WT> &tn,
           float16v (&acc)[BM / 64][2], int wm, int vb0, int vb1)
{
  constexpr int TM = BM / 64;
  constexpr int D = GemmDepth<BM>::value;
  constexpr int BK = Geo<WT>::BK, LDK = Geo<WT>::LDK, KS = BK / 16;
  const int lane = threadIdx.x & 63;
  half8 af[KS][TM], bf[KS][2];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
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
      // the two blocks of the step in turn: block sum from a zero
      // accumulator, times the block's scale
      const uint32_t d0 = *(const uint32_t *)(Dc + (vb0 + (lane & 31)) * 2);
      const uint32_t d1 = *(const uint32_t *)(Dc + (vb1 + (lane & 31)) * 2);
      const float sc[2][2] = { { h2f ((uint16_t)(d0 & 0xffff)), h2f ((uint16_t)(d1 & 0xffff)) },
                               { h2f ((uint16_t)(d0 >> 16)), h2f ((uint16_t)(d1 >> 16)) } };
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
          for (int ni = 0; ni < 2; ++ni)
            {
              float16v part;
#pragma unroll
              for (int r = 0; r < 16; ++r)
                part[r] = 0.f;
              part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (af[2 * blk][mi], bf[2 * blk][ni], part, 0, 0, 0);
              part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (af[2 * blk + 1][mi], bf[2 * blk + 1][ni], part, 0, 0, 0);
#pragma unroll
              for (int r = 0; r < 16; ++r)
                acc[mi][ni][r] = __builtin_fmaf (part[r], sc[blk][ni], acc[mi][ni][r]);
            }
    }
  else
    {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
          for (int ni = 0; ni < 2; ++ni)
            acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_f16 (
                af[ks][mi], bf[ks][ni], acc[mi][ni], 0, 0, 0);
    }
  store_tile<BM, WT> (tn, An, Bn, Dn);
  const int knext = kbase + min (kt + 1 + D, nk - 1);
  issue_tile<BM, WT> (a, ta, knext * BK, tn);
  __syncthreads ();
}

template <int BM, int WT>
__global__ __launch_bounds__ (kGemmThreads, 2) void
gemm_mfma_kernel (const GemmArgs a, int tiles_m, int tiles_n, int per_xcd,
                  int ksplit, float *ws)
{
  // element offsets of this problem of the batch (the argument block itself
  // stays untouched in constant memory: it is indexed by a run-time matrix
  // number below)
  const size_t bi = a.batch > 1 ? blockIdx.y : 0;
  const size_t xoff = bi * a.xbs, woff = bi * a.wbs, yoff = bi * a.ybs;
  constexpr int TM = BM / 64; // 32-row accumulators per wave along M
  constexpr int BK = Geo<WT>::BK, LDK = Geo<WT>::LDK;
  __shared__ __align__ (16) uint16_t As[2][BM * LDK];
  __shared__ __align__ (16) uint16_t Bs[2][BN * LDK];
  __shared__ __align__ (4) uint16_t Ds[2][BN * 2]; // Q8_0: the two block scales of every tile row

  // XCD-aware tile numbering
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int tile = xcd * per_xcd + j;
  if (j >= per_xcd || tile >= tiles_m * tiles_n * ksplit)
    return;
  // ksplit > 1: the k range is divided among ksplit workgroups per output
  // tile; each writes its fp32 partial tile to the workspace and a second
  // kernel adds the parts in order and applies the epilogue
  const int ks = tile / (tiles_m * tiles_n), t2 = tile - ks * (tiles_m * tiles_n);
  const int tn = t2 / tiles_m, tm = t2 - tn * tiles_m;
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

  const int nk_all = ((a.wtype == 8 ? a.Kp : a.K) + BK - 1) / BK;
  const int kbase = (int)((long)nk_all * ks / ksplit);
  const int nk = (int)((long)nk_all * (ks + 1) / ksplit) - kbase; // k steps of this workgroup
  // D tiles are in flight in registers (tile k + 1 .. k + D while tile k is
  // being multiplied out of LDS): a k-step costs far less time than a trip to
  // memory, so one tile of look-ahead would leave every step waiting
  constexpr int D = GemmDepth<BM>::value;
  TileAddr<BM, WT> ta;
  tile_addresses<BM, WT> (a, xoff, woff, zmat, m0, n0, ta);
  TileLoads<BM, WT> t[D];
  issue_tile<BM, WT> (a, ta, kbase * BK, t[0]);
  store_tile<BM, WT> (t[0], As[0], Bs[0], Ds[0]);
  issue_tile<BM, WT> (a, ta, (kbase + min (1, nk - 1)) * BK, t[1 % D]);
  issue_tile<BM, WT> (a, ta, (kbase + min (2, nk - 1)) * BK, t[2 % D]);
  if (D > 2)
    {
      issue_tile<BM, WT> (a, ta, (kbase + min (3, nk - 1)) * BK, t[3]);
      issue_tile<BM, WT> (a, ta, (kbase + min (4, nk - 1)) * BK, t[0]);
    }
  __syncthreads ();

  // Each step multiplies tile kt out of LDS buffer kt & 1, moves tile kt + 1
  // (issued D steps earlier) from its registers to the other buffer and
  // reuses those registers for tile kt + 1 + D.  Stores and loads are
  // unconditional (past the end they repeat the last tile, which nothing
  // reads), so the waits in the unrolled body count loads exactly.
#define VKL_GEMM_STEP(d)                                                      \
  gemm_step<BM, WT> (a, ta, kbase, kt0 + (d), nk, As[(d) & 1], Bs[(d) & 1], \
                     Ds[(d) & 1], As[((d) & 1) ^ 1], Bs[((d) & 1) ^ 1],      \
                     Ds[((d) & 1) ^ 1], t[((d) + 1) % D], acc, wm, vb0, vb1)
  int kt0 = 0;
  for (; kt0 + D <= nk; kt0 += D)
    {
      VKL_GEMM_STEP (0);
      VKL_GEMM_STEP (1);
      if (D > 2)
        {
          VKL_GEMM_STEP (2);
          VKL_GEMM_STEP (3);
        }
    }
  if (kt0 + 0 < nk)
    VKL_GEMM_STEP (0);
  if (kt0 + 1 < nk)
    VKL_GEMM_STEP (1);
  if (D > 2 && kt0 + 2 < nk)
    VKL_GEMM_STEP (2);
#undef VKL_GEMM_STEP

  // epilogue: accumulator register r of lane l is row 8*(r/4) + 4*(l/32) +
  // r%4, column l%32 of its 32x32 block
  if (ksplit > 1)
    {
      // partial tile: matrix t of the launch (up = 0 and gate = 1 for the
      // fused pair), k part ks, dense [M, N] fp32
#pragma unroll
      for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          {
            const int m = m0 + wm * (BM / 2) + mi * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
            if (m >= a.M)
              continue;
#pragma unroll
            for (int ni = 0; ni < 2; ++ni)
              {
                const int n = a.upgate ? n0 + wn * 32 + (lane & 31)
                                       : n0 + wn * 64 + ni * 32 + (lane & 31);
                const int t = a.upgate ? ni : zmat;
                if (n < a.N)
                  ws[((size_t)(t * ksplit + ks) * a.M + m) * a.N + n] = acc[mi][ni][r];
              }
          }
      return;
    }
  uint16_t *y = a.y[a.upgate ? 0 : zmat] + yoff;
  const uint16_t *res = a.residual ? a.residual + yoff : nullptr;
  float *y32 = a.y32 ? a.y32 + bi * (size_t)a.M * a.N : nullptr;
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
            if (a.nmat == 1 && res)
              h = f2h (h2f (h) + h2f (ldg (res + o)));
            y[o] = h;
            if (a.nmat == 1 && y32)
              y32[(size_t)m * a.N + n] = h2f (h);
          }
      }
}

// ---------------------------------------------------------------------------
// few token rows (M <= 32): weight-streaming form, K split over workgroups
// ---------------------------------------------------------------------------
// A workgroup owns 32 weight rows and a 1024-wide slice of K: its 32 x 1024
// piece of x goes to LDS once (64 KiB, so two workgroups share a compute unit
// and one streams while the other reduces), each of the 8 waves requests ALL
// of its weights (4 Q8_0 blocks of 32 rows) at the start, in one round, and
// reads the x operand from LDS.  The slices' partial sums (fp32) go to a
// workspace and a second small kernel adds them in slice order and applies
// the epilogue, so the result does not depend on timing.  (An earlier form
// with the x fragments in registers next to the weights, one workgroup per 32
// weight rows over the whole of K, streamed at half the rate; from 33 rows on
// the tile kernel with its own k-split is faster than either.)
constexpr int kSk2Waves = 8;
constexpr int kSk2Slice = 1024;                // k extent of a workgroup
constexpr int kSk2Ldx = kSk2Slice + 8;         // LDS row stride of x in halves
constexpr size_t kSk2Workspace = 64u << 20;    // bytes, per stream

template <int WT>
__global__ __launch_bounds__ (kSk2Waves * 64) void
gemm_skinny2_kernel (const GemmArgs a, float *ws, int S)
{
  constexpr int UN = kSk2Slice / 32 / kSk2Waves; // blocks per wave: 4
  extern __shared__ __align__ (16) uint8_t lds[];
  uint16_t *xs = (uint16_t *)lds; // [32][kSk2Ldx]
  float *red = (float *)lds;      // after the products: [waves][32][33]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5;
  const int n0 = blockIdx.y * 32, slice = blockIdx.x, mat = blockIdx.z;
  const int k0 = slice * kSk2Slice;
  const int nrow = min (n0 + (lane & 31), a.N - 1); // clamped, masked at the end
  const void *zeros = g_zero_chunk;

  // The workgroup's piece of x first (it comes from the caches and returns
  // well before the weights: loads return in order), then all weights of the
  // wave; x goes to LDS while the weights are still on their way.
  constexpr int CPR = kSk2Slice / 8;               // chunks per x row
  constexpr int NCH = 32 * CPR / (kSk2Waves * 64); // per thread: 8
  uint4 xv[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    {
      const int c = tid + i * kSk2Waves * 64;
      const int row = c / CPR, k = k0 + (c % CPR) * 8;
      const bool v = row < a.M && k + 8 <= a.K;
      xv[i] = ldg16 (v ? (const void *)(a.x + (size_t)row * a.xs + k) : zeros);
    }
  __builtin_amdgcn_sched_barrier (0);
  uint4 wv[UN][WT == 8 ? 1 : 2];
  uint16_t dv[UN];
  const int bw = k0 / 32 + wave * UN; // first block of the wave
#pragma unroll
  for (int u = 0; u < UN; ++u)
    {
      const int k = (bw + u) * 32 + g * 16;
      if (WT == 8)
        {
          const bool v = k < a.Kp;
          const uint8_t *wq = (const uint8_t *)pick3 (a.wq[0], a.wq[1], a.wq[2], mat) + (size_t)nrow * a.Kp;
          const uint16_t *wd
              = (const uint16_t *)pick3 (a.wd[0], a.wd[1], a.wd[2], mat) + (size_t)nrow * (a.Kp >> 5);
          wv[u][0] = ldg16 (v ? (const void *)(wq + k) : zeros);
          dv[u] = ldg (v ? wd + (bw + u) : (const uint16_t *)zeros);
        }
      else
        {
          const bool v = k + 16 <= a.K;
          const uint16_t *wh = (const uint16_t *)pick3 (a.wh[0], a.wh[1], a.wh[2], mat) + (size_t)nrow * a.ws;
          wv[u][0] = ldg16 (v ? (const void *)(wh + k) : zeros);
          wv[u][WT == 8 ? 0 : 1] = ldg16 (v ? (const void *)(wh + k + 8) : zeros);
          dv[u] = 0;
        }
    }
  __builtin_amdgcn_sched_barrier (0);
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    {
      const int c = tid + i * kSk2Waves * 64;
      *(uint4 *)(xs + (c / CPR) * kSk2Ldx + (c % CPR) * 8) = xv[i];
    }
  __syncthreads ();

  float16v acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.f;
  const uint16_t *xa = xs + (lane & 31) * kSk2Ldx + wave * UN * 32 + g * 16;
#pragma unroll
  for (int u = 0; u < UN; ++u)
    {
      // operands: A = x (rows = tokens), B = weights (columns = rows n); a
      // lane's 16 consecutive k values feed two MFMAs
      const half8 a0 = *(const half8 *)(xa + u * 32), a1 = *(const half8 *)(xa + u * 32 + 8);
      half8 b0, b1;
      if (WT == 8)
        {
          const uint32_t w[4] = { wv[u][0].x, wv[u][0].y, wv[u][0].z, wv[u][0].w };
          uint32_t o[8];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            {
              h16x2 lo, hi;
              i8x4_to_h2x2 (w[j], lo, hi);
              o[2 * j] = __builtin_bit_cast (uint32_t, lo);
              o[2 * j + 1] = __builtin_bit_cast (uint32_t, hi);
            }
          b0 = __builtin_bit_cast (half8, make_uint4 (o[0], o[1], o[2], o[3]));
          b1 = __builtin_bit_cast (half8, make_uint4 (o[4], o[5], o[6], o[7]));
          // Q8_0: block sum from a zero accumulator, times the block scale
          float16v part;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            part[r] = 0.f;
          part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a0, b0, part, 0, 0, 0);
          part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a1, b1, part, 0, 0, 0);
          const float sc = h2f (dv[u]);
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[r] = __builtin_fmaf (part[r], sc, acc[r]);
        }
      else
        {
          b0 = __builtin_bit_cast (half8, wv[u][0]);
          b1 = __builtin_bit_cast (half8, wv[u][WT == 8 ? 0 : 1]);
          acc = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a0, b0, acc, 0, 0, 0);
          acc = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a1, b1, acc, 0, 0, 0);
        }
    }

  // add the waves' parts of the slice (x in LDS is no longer needed)
  __syncthreads ();
#pragma unroll
  for (int r = 0; r < 16; ++r)
    red[(wave * 32 + (r >> 2) * 8 + g * 4 + (r & 3)) * 33 + (lane & 31)] = acc[r];
  __syncthreads ();
  for (int i = tid; i < 32 * 32; i += kSk2Waves * 64)
    {
      const int m = i >> 5, nn = i & 31, n = n0 + nn;
      if (m < a.M && n < a.N)
        {
          float v = 0.f;
#pragma unroll
          for (int w = 0; w < kSk2Waves; ++w)
            v += red[(w * 32 + m) * 33 + nn];
          ws[((size_t)(mat * S + slice) * 32 + m) * a.N + n] = v;
        }
    }
}

// ---------------------------------------------------------------------------
// few token rows (M <= 32), Q8_0 weights: whole cache lines per weight row
// ---------------------------------------------------------------------------
// The kernel above has a lane fetch 16 bytes of "its" weight row, so a load
// instruction touches 32 rows with 32 contiguous bytes each; memory delivers
// such pieces at well under the rate of whole lines.  Here a workgroup owns 64
// weight rows and a 512-wide slice of K, wave (rb, kq) the 32 rows of row block
// rb and the 128-wide quarter kq of the slice: a load instruction fetches 8
// rows x 128 contiguous bytes (one line per row), four of them the wave's
// whole 32 x 128 piece.  The piece goes through a private LDS region of the
// wave (no workgroup barrier) to reach the matrix-core operand order (lane =
// row, 16 consecutive k).  The slice of x is half as large as above for the
// same weight bytes, and three workgroups fit a compute unit.  Partial sums
// and their reduction are as above (slices of 512).
constexpr int kR64Waves = 8;
constexpr int kR64Slice = 512;
constexpr int kR64Ldx = kR64Slice + 8;      // LDS row stride of x in halves
constexpr int kR64Tstride = 128 + 16;       // LDS row stride of a wave's weight piece in bytes
constexpr size_t kR64XBytes = (size_t)32 * kR64Ldx * 2;
constexpr size_t kR64TBytes = (size_t)kR64Waves * 32 * kR64Tstride;
constexpr size_t kR64RedBytes = (size_t)kR64Waves * 32 * 33 * 4;
constexpr size_t kR64Lds = kR64XBytes + (kR64TBytes > kR64RedBytes ? kR64TBytes : kR64RedBytes);
static_assert (2 * kR64RedBytes <= kR64Lds, "two passes' partial sums fit over x and the weight pieces");

#ifdef VKL_TRACE
__device__ unsigned long long *g_r64_trace = nullptr;
#define VKL_R64T(slot)                                                        \
  if (threadIdx.x == 0 && g_r64_trace)                                        \
    g_r64_trace[((size_t)(blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 8 + (slot)] \
        = wall_clock64 ();
#else
#define VKL_R64T(slot)
#endif

__global__ __launch_bounds__ (kR64Waves * 64) void
gemm_rows64_q8_kernel (const GemmArgs a, float *ws, int S)
{
  VKL_R64T (0)
  // row blocks a wave works through one after the other (the workgroup owns
  // 64 * PASSES weight rows, all loads requested at the start).  Two measured
  // slower than one on the 7B shapes (8.4 k against 9.0 k tok/s on a 32-token
  // prompt) although they double the bytes a workgroup has in flight.
  constexpr int PASSES = 1;
  extern __shared__ __align__ (16) uint8_t lds[];
  uint16_t *xs = (uint16_t *)lds;                 // [32][kR64Ldx]
  uint8_t *tr = lds + kR64XBytes;                 // [waves][32][kR64Tstride]
  // after the products: [PASSES][waves][32][33] (over the weight pieces and,
  // with two passes, the slice of x)
  float *red = (float *)(PASSES == 1 ? lds + kR64XBytes : lds);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int rb = wave >> 2, kq = wave & 3, g = lane >> 5;
  const int slice = blockIdx.x, mat = blockIdx.z;
  const int nwg = blockIdx.y * 64 * PASSES;       // first row of the workgroup
  const int k0 = slice * kR64Slice, kw = k0 + kq * 128; // first k of the slice / of the wave
  const void *zeros = g_zero_chunk;
  const uint8_t *wq = (const uint8_t *)pick3 (a.wq[0], a.wq[1], a.wq[2], mat);
  const uint16_t *wd = (const uint16_t *)pick3 (a.wd[0], a.wd[1], a.wd[2], mat);

  // the workgroup's piece of x first (from the caches, back before the
  // weights: loads return in order), then the scales, then the weights
  constexpr int CPR = kR64Slice / 8;                // 16-byte chunks per x row
  constexpr int NCH = 32 * CPR / (kR64Waves * 64);  // per thread: 4
  uint4 xv[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    {
      const int c = tid + i * kR64Waves * 64;
      const int row = c / CPR, k = k0 + (c % CPR) * 8;
      const bool v = row < a.M && k + 8 <= a.K;
      xv[i] = ldg16 (v ? (const void *)(a.x + (size_t)row * a.xs + k) : zeros);
    }
  // pass p of wave (rb, kq): rows nwg + (2 p + rb) * 32 ... + 31.
  // lane (n, g): the four block scales of row n of each pass in the wave's quarter
  uint16_t dv[PASSES][4];
#pragma unroll
  for (int p = 0; p < PASSES; ++p)
    {
      const int nrow = min (nwg + (2 * p + rb) * 32 + (lane & 31), a.N - 1); // clamped, masked at the end
#pragma unroll
      for (int u = 0; u < 4; ++u)
        {
          const int blk = (kw >> 5) + u;
          const bool v = blk * 32 < a.Kp;
          dv[p][u] = ldg (v ? wd + (size_t)nrow * (a.Kp >> 5) + blk : (const uint16_t *)zeros);
        }
    }
  __builtin_amdgcn_sched_barrier (0);
  // load j of a pass: rows 8 j .. 8 j + 7 of the row block, 128 contiguous bytes each
  uint4 wv[PASSES][4];
  const int lr = lane >> 3, lc = (lane & 7) * 16;
#pragma unroll
  for (int p = 0; p < PASSES; ++p)
#pragma unroll
    for (int j = 0; j < 4; ++j)
      {
        const int row = min (nwg + (2 * p + rb) * 32 + j * 8 + lr, a.N - 1);
        const bool v = kw + lc < a.Kp;
        wv[p][j] = ldg16 (v ? (const void *)(wq + (size_t)row * a.Kp + kw + lc) : zeros);
      }
  __builtin_amdgcn_sched_barrier (0);
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    {
      const int c = tid + i * kR64Waves * 64;
      *(uint4 *)(xs + (c / CPR) * kR64Ldx + (c % CPR) * 8) = xv[i];
    }
  VKL_R64T (1)
  __syncthreads ();
  VKL_R64T (2)

  uint8_t *tw = tr + (size_t)wave * 32 * kR64Tstride; // the wave's own LDS region
  const uint16_t *xa = xs + (lane & 31) * kR64Ldx + kq * 128 + g * 16;
  const uint8_t *tb = tw + (lane & 31) * kR64Tstride + g * 16;
  float16v acc[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; ++p)
    {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[p][r] = 0.f;
      // the pass's piece into the wave's LDS region, row-major, and back in
      // matrix-core order (a wave's LDS operations complete in order; no
      // other wave touches the region)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *(uint4 *)(tw + (j * 8 + lr) * kR64Tstride + lc) = wv[p][j];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        {
          // operands: A = x (rows = tokens), B = weights (columns = rows n); a
          // lane's 16 consecutive k values feed two MFMAs; Q8_0: block sum from
          // a zero accumulator, times the block scale
          const half8 a0 = *(const half8 *)(xa + u * 32), a1 = *(const half8 *)(xa + u * 32 + 8);
          const uint4 wq4 = *(const uint4 *)(tb + u * 32);
          const uint32_t w[4] = { wq4.x, wq4.y, wq4.z, wq4.w };
          uint32_t o[8];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            {
              h16x2 lo, hi;
              i8x4_to_h2x2 (w[j], lo, hi);
              o[2 * j] = __builtin_bit_cast (uint32_t, lo);
              o[2 * j + 1] = __builtin_bit_cast (uint32_t, hi);
            }
          const half8 b0 = __builtin_bit_cast (half8, make_uint4 (o[0], o[1], o[2], o[3]));
          const half8 b1 = __builtin_bit_cast (half8, make_uint4 (o[4], o[5], o[6], o[7]));
          float16v part;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            part[r] = 0.f;
          part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a0, b0, part, 0, 0, 0);
          part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a1, b1, part, 0, 0, 0);
          const float sc = h2f (dv[p][u]);
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[p][r] = __builtin_fmaf (part[r], sc, acc[p][r]);
        }
    }

  // add the four quarters of each row block (x and the weight pieces in LDS
  // are no longer needed)
#ifdef VKL_TRACE
  asm volatile("" ::"v"(acc[0][0]));
#endif
  VKL_R64T (3)
  __syncthreads ();
  VKL_R64T (4)
#pragma unroll
  for (int p = 0; p < PASSES; ++p)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      red[((p * kR64Waves + wave) * 32 + (r >> 2) * 8 + g * 4 + (r & 3)) * 33 + (lane & 31)] = acc[p][r];
  __syncthreads ();
  for (int i = tid; i < PASSES * 2 * 32 * 32; i += kR64Waves * 64)
    {
      // row block b of the workgroup = pass b / 2, waves 4 (b % 2) ... + 3
      const int b = i >> 10, m = (i >> 5) & 31, nn = i & 31, n = nwg + b * 32 + nn;
      if (m < a.M && n < a.N)
        {
          float v = 0.f;
#pragma unroll
          for (int q = 0; q < 4; ++q)
            v += red[(((b >> 1) * kR64Waves + (b & 1) * 4 + q) * 32 + m) * 33 + nn];
          ws[((size_t)(mat * S + slice) * 32 + m) * a.N + n] = v;
        }
    }
  VKL_R64T (5)
}

// The same with waves that do not wait for one another: a workgroup of four
// waves owns 128 weight rows and a 512-wide slice of K, each wave 32 rows over
// the whole slice (16 loads of 8 rows x 128 bytes, all requested at the
// start).  The only barrier follows the staging of x; a wave then works
// through its four 128-wide quarters as their loads arrive and stores its
// 32 x 32 partial sums from registers: no sum over waves.  In the form above
// the time from "weights arrived" to "workgroup done" (two barriers, the sum
// over the waves through LDS) was twice the load latency.
constexpr int kR128Waves = 4;
constexpr size_t kR128Lds = kR64XBytes + (size_t)kR128Waves * 32 * kR64Tstride;

__global__ __launch_bounds__ (kR128Waves * 64, 3) void
gemm_rows128_q8_kernel (const GemmArgs a, float *ws, int S)
{
  VKL_R64T (0)
  extern __shared__ __align__ (16) uint8_t lds[];
  uint16_t *xs = (uint16_t *)lds;                 // [32][kR64Ldx]
  uint8_t *tr = lds + kR64XBytes;                 // [waves][32][kR64Tstride]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 5;
  const int slice = blockIdx.x, mat = blockIdx.z;
  const int n0 = blockIdx.y * 128 + wave * 32;    // first row of the wave
  const int k0 = slice * kR64Slice;
  const void *zeros = g_zero_chunk;
  const uint8_t *wq = (const uint8_t *)pick3 (a.wq[0], a.wq[1], a.wq[2], mat);
  const uint16_t *wd = (const uint16_t *)pick3 (a.wd[0], a.wd[1], a.wd[2], mat);

  // the workgroup's piece of x first (from the caches, back before the
  // weights: loads return in order), then the scales, then the weights
  constexpr int CPR = kR64Slice / 8;                 // 16-byte chunks per x row
  constexpr int NCH = 32 * CPR / (kR128Waves * 64);  // per thread: 8
  uint4 xv[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    {
      const int c = tid + i * kR128Waves * 64;
      const int row = c / CPR, k = k0 + (c % CPR) * 8;
      const bool v = row < a.M && k + 8 <= a.K;
      xv[i] = ldg16 (v ? (const void *)(a.x + (size_t)row * a.xs + k) : zeros);
    }
  // lane (n, g): the 16 block scales of row n0 + n in this slice, 32
  // contiguous bytes (16-byte aligned: Kp is a multiple of 256 here; the
  // second half of the row's last slice may lie past K)
  const int nrow = min (n0 + (lane & 31), a.N - 1); // clamped, masked at the end
  const uint16_t *dp = wd + (size_t)nrow * (a.Kp >> 5) + (k0 >> 5);
  const uint4 d0 = ldg16 (k0 < a.Kp ? (const void *)dp : zeros);
  const uint4 d1 = ldg16 (k0 + 256 < a.Kp ? (const void *)(dp + 8) : zeros);
  __builtin_amdgcn_sched_barrier (0);
  // load (q, j): rows 8 j .. 8 j + 7 of the wave's rows, the 128 contiguous
  // bytes of quarter q each; two quarters are in flight
  // (two arrays passed by reference: an array reached through a pointer
  // would live in scratch memory instead of registers)
  uint4 wva[4], wvb[4];
  const int lr = lane >> 3, lc = (lane & 7) * 16;
  auto issue = [&] (int q, uint4 (&dst)[4]) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      {
        const int row = min (n0 + j * 8 + lr, a.N - 1);
        const int k = k0 + q * 128 + lc;
        dst[j] = ldg16 (k < a.Kp ? (const void *)(wq + (size_t)row * a.Kp + k) : zeros);
      }
  };
  issue (0, wva);
  issue (1, wvb);
  __builtin_amdgcn_sched_barrier (0);
#pragma unroll
  for (int i = 0; i < NCH; ++i)
    {
      const int c = tid + i * kR128Waves * 64;
      *(uint4 *)(xs + (c / CPR) * kR64Ldx + (c % CPR) * 8) = xv[i];
    }
  VKL_R64T (1)
  __syncthreads ();
  VKL_R64T (2)

  uint8_t *tw = tr + (size_t)wave * 32 * kR64Tstride; // the wave's own LDS region
  const uint16_t *xa = xs + (lane & 31) * kR64Ldx + g * 16;
  const uint8_t *tb = tw + (lane & 31) * kR64Tstride + g * 16;
  const uint32_t dw[8] = { d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w };
  float16v acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q)
    {
      // the quarter's piece into the wave's LDS region, row-major, and back in
      // matrix-core order (a wave's LDS operations complete in order; no
      // other wave touches the region); its registers then take the quarter
      // after next
#pragma unroll
      for (int j = 0; j < 4; ++j)
        *(uint4 *)(tw + (j * 8 + lr) * kR64Tstride + lc) = (q & 1) ? wvb[j] : wva[j];
      __builtin_amdgcn_sched_barrier (0);
      if (q + 2 < 4)
        {
          if (q & 1)
            issue (q + 2, wvb);
          else
            issue (q + 2, wva);
        }
      __builtin_amdgcn_sched_barrier (0);
#pragma unroll
      for (int u = 0; u < 4; ++u)
        {
          // operands: A = x (rows = tokens), B = weights (columns = rows n); a
          // lane's 16 consecutive k values feed two MFMAs; Q8_0: block sum from
          // a zero accumulator, times the block scale
          const half8 a0 = *(const half8 *)(xa + q * 128 + u * 32);
          const half8 a1 = *(const half8 *)(xa + q * 128 + u * 32 + 8);
          const uint4 wq4 = *(const uint4 *)(tb + u * 32);
          const uint32_t w[4] = { wq4.x, wq4.y, wq4.z, wq4.w };
          uint32_t o[8];
#pragma unroll
          for (int j = 0; j < 4; ++j)
            {
              h16x2 lo, hi;
              i8x4_to_h2x2 (w[j], lo, hi);
              o[2 * j] = __builtin_bit_cast (uint32_t, lo);
              o[2 * j + 1] = __builtin_bit_cast (uint32_t, hi);
            }
          const half8 b0 = __builtin_bit_cast (half8, make_uint4 (o[0], o[1], o[2], o[3]));
          const half8 b1 = __builtin_bit_cast (half8, make_uint4 (o[4], o[5], o[6], o[7]));
          float16v part;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            part[r] = 0.f;
          part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a0, b0, part, 0, 0, 0);
          part = __builtin_amdgcn_mfma_f32_32x32x16_f16 (a1, b1, part, 0, 0, 0);
          const int bi = q * 4 + u; // block of the slice
          const float sc = h2f ((uint16_t)(dw[bi >> 1] >> (16 * (bi & 1))));
#pragma unroll
          for (int r = 0; r < 16; ++r)
            acc[r] = __builtin_fmaf (part[r], sc, acc[r]);
          // (the sums are formed here and now: left alone, the compiler moves
          // these sixteen products down to the conditional stores at the end
          // and keeps every block's partial sums alive until then)
          asm volatile("" : "+v"(acc));
        }
    }
#ifdef VKL_TRACE
  asm volatile("" ::"v"(acc[0]));
#endif
  VKL_R64T (3)
  // the wave's 32 x 32 partial sums: accumulator r of lane (n, g) belongs to
  // token row (r / 4) * 8 + g * 4 + r % 4
  const int n = n0 + (lane & 31);
#pragma unroll
  for (int r = 0; r < 16; ++r)
    {
      const int m = (r >> 2) * 8 + g * 4 + (r & 3);
      if (m < a.M && n < a.N)
        ws[((size_t)(mat * S + slice) * 32 + m) * a.N + n] = acc[r];
    }
  VKL_R64T (5)
}

// sum over the slices in order, then the epilogue of the product
__global__ __launch_bounds__ (256) void
skinny2_reduce_kernel (const GemmArgs a, const float *ws, int S, int mrows)
{
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= (size_t)a.M * a.N)
    return;
  const int m = (int)(i / a.N), n = (int)(i % a.N);
  const int nm = a.upgate ? 2 : a.nmat;
  const size_t o = (size_t)m * a.ys + n;
  // the residual value and the parts are requested unconditionally, eight
  // parts at a time from clamped slices (a loop with a run-time bound around
  // single loads would make one trip to memory per part); a part past the
  // last counts as zero, so the parts are still added in slice order
  const uint16_t rs = ldg (a.residual ? a.residual + o : (const uint16_t *)ws);
  float v[3] = { 0.f, 0.f, 0.f };
  for (int t = 0; t < nm; ++t)
    for (int s0 = 0; s0 < S; s0 += 8)
      {
        float pc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          pc[j] = ldg (ws + ((size_t)(t * S + min (s0 + j, S - 1)) * mrows + m) * a.N + n);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          v[t] += s0 + j < S ? pc[j] : 0.f;
      }
  if (a.upgate)
    {
      a.y[0][o] = f2h (silu (v[1]) * v[0]);
      return;
    }
  if (a.nmat > 1)
    {
      for (int t = 0; t < a.nmat; ++t)
        a.y[t][o] = f2h (v[t]);
      return;
    }
  float r = v[0] * a.scale + a.bias;
  if (a.act == 1)
    r = silu (r);
  uint16_t h = f2h (r);
  if (a.residual)
    h = f2h (h2f (h) + h2f (rs));
  a.y[0][o] = h;
  if (a.y32)
    a.y32[(size_t)m * a.N + n] = h2f (h);
}

// fp32 workspace of the split forms: one per (device, stream), allocated on
// first use and freed when the stream is destroyed
std::mutex g_ws_mu;
std::map<std::pair<int, hipStream_t>, float *> g_ws_table;

float *
skinny2_workspace (hipStream_t s)
{
  std::lock_guard<std::mutex> lock (g_ws_mu);
  int dev = 0;
  if (hipGetDevice (&dev) != hipSuccess)
    return nullptr;
  auto it = g_ws_table.find ({ dev, s });
  if (it != g_ws_table.end ())
    return it->second;
  void *p = nullptr;
  if (hipMalloc (&p, kSk2Workspace) != hipSuccess)
    return nullptr;
  g_ws_table[{ dev, s }] = (float *)p;
  return (float *)p;
}

// Scratch for callers that must not allocate (vkl_matmul_q8_0_noalloc): a
// file-scope device array.  Every GPU the library runs on holds its own copy
// at its own address until the process ends; in host code the array's name is
// only a handle for hipGetSymbolAddress, never an address to pass to a kernel.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__ (256) unsigned char scratch[kStaticScratchBytes];
float *g_static_scratch[16] = {};

// K slices of the few-row form
template <int WT>
int
skinny2_slices (const GemmArgs &a)
{
  const int keff = WT == 8 ? a.Kp : a.K;
  return (keff + kSk2Slice - 1) / kSk2Slice;
}

// raises the kernel's LDS limit once per device
template <int WT>
bool
skinny2_prepare (size_t lds)
{
  static LdsLimit limit;
  return limit.raise ((const void *)gemm_skinny2_kernel<WT>, lds) == 0;
}

// the whole-line form for Q8_0 weights
bool
launch_rows64_q8 (const GemmArgs &a, hipStream_t s, int &err)
{
  if (a.wtype != 8 || a.M > 32 || a.batch > 1)
    return false;
  const int S = (a.Kp + kR64Slice - 1) / kR64Slice;
  const int nm = a.upgate ? 2 : a.nmat;
  const size_t need = (size_t)nm * S * 32 * a.N * sizeof (float);
  if (need > kSk2Workspace || (a.workspace && need > a.workspace_bytes))
    return false;
  static LdsLimit limit64, limit128;
  if (limit64.raise ((const void *)gemm_rows64_q8_kernel, kR64Lds) != 0
      || limit128.raise ((const void *)gemm_rows128_q8_kernel, kR128Lds) != 0)
    return false;
  float *ws = a.workspace ? a.workspace : skinny2_workspace (s);
  if (!ws)
    return false;
  // The form with independent waves reads a row's 16 scales of a slice as two
  // aligned 16-byte words: rows of scales must be multiples of 16 bytes.
  if ((a.Kp % 256) == 0)
    gemm_rows128_q8_kernel<<<dim3 ((unsigned)S, (unsigned)((a.N + 127) / 128), (unsigned)nm),
                             dim3 (kR128Waves * 64), kR128Lds, s>>> (a, ws, S);
  else
    gemm_rows64_q8_kernel<<<dim3 ((unsigned)S, (unsigned)((a.N + 63) / 64), (unsigned)nm),
                            dim3 (kR64Waves * 64), kR64Lds, s>>> (a, ws, S);
  const size_t total = (size_t)a.M * a.N;
  skinny2_reduce_kernel<<<dim3 ((unsigned)((total + 255) / 256)), dim3 (256), 0, s>>> (a, ws, S, 32);
  err = (int)hipGetLastError ();
  return true;
}

template <int WT>
bool
launch_skinny2 (const GemmArgs &a, hipStream_t s, int &err)
{
  if (a.M > 32 || a.batch > 1)
    return false;
  const int S = skinny2_slices<WT> (a);
  const int nm = a.upgate ? 2 : a.nmat;
  const size_t need = (size_t)nm * S * 32 * a.N * sizeof (float);
  if (need > kSk2Workspace || (a.workspace && need > a.workspace_bytes))
    return false;
  const size_t lds = (size_t)32 * kSk2Ldx * 2;
  if (!skinny2_prepare<WT> (lds))
    return false;
  float *ws = a.workspace ? a.workspace : skinny2_workspace (s);
  if (!ws)
    return false;
  gemm_skinny2_kernel<WT><<<dim3 ((unsigned)S, (unsigned)((a.N + 31) / 32), (unsigned)nm),
                           dim3 (kSk2Waves * 64), lds, s>>> (a, ws, S);
  const size_t total = (size_t)a.M * a.N;
  skinny2_reduce_kernel<<<dim3 ((unsigned)((total + 255) / 256)), dim3 (256), 0, s>>> (a, ws, S, 32);
  err = (int)hipGetLastError ();
  return true;
}

// parts the k range of a tile is split into (1: no split, no workspace)
template <int BM, int WT>
int
tile_ksplit (const GemmArgs &a)
{
  const int tiles_m = (a.M + BM - 1) / BM;
  const int tiles_n = (a.N + (a.upgate ? 64 : BN) - 1) / (a.upgate ? 64 : BN);
  const int nz = a.upgate ? 1 : a.nmat, nm = a.upgate ? 2 : a.nmat;
  const int nk = ((a.wtype == 8 ? a.Kp : a.K) + Geo<WT>::BK - 1) / Geo<WT>::BK;
  if (a.batch > 1 || WT == 2)
    return 1;
  // (measured on the 7B shapes: a split in two pays for Q8_0 weights, whose
  // steps are slower, and not for fp16 weights)
  const int want = kGemmSplitTarget / (tiles_m * tiles_n * nz);
  int ksplit = want < (WT == 8 ? 2 : 3) ? 1 : std::max (1, std::min (std::min (want, 8), nk / 8));
  // as far as the scratch holds the partial tiles (a caller's may be smaller
  // than the launcher's own)
  const size_t have = a.workspace ? std::min (a.workspace_bytes, kSk2Workspace) : kSk2Workspace;
  while (ksplit > 1 && (size_t)nm * ksplit * a.M * a.N * sizeof (float) > have)
    --ksplit;
  return ksplit;
}

template <int BM, int WT>
int
launch_cfg (const GemmArgs &a, int ksplit, hipStream_t s)
{
  const int tiles_m = (a.M + BM - 1) / BM;
  const int tiles_n = (a.N + (a.upgate ? 64 : BN) - 1) / (a.upgate ? 64 : BN);
  // Too few output tiles to occupy the compute units (a few hundred token
  // rows against a 4096-row matrix): the k range is split as well, into parts
  // of at least eight steps, as far as the fp32 workspace holds the partial
  // tiles.  Not for batched products (there are tiles enough).
  const int nz = a.upgate ? 1 : a.nmat;
  float *ws = nullptr;
  if (ksplit > 1 && !(ws = a.workspace ? a.workspace : skinny2_workspace (s)))
    ksplit = 1;
  const int tiles = tiles_m * tiles_n * ksplit;
  const int per_xcd = (tiles + 7) / 8;
  gemm_mfma_kernel<BM, WT>
      <<<dim3 ((unsigned)(per_xcd * 8), (unsigned)(a.batch > 1 ? a.batch : 1),
               (unsigned)nz),
         dim3 (kGemmThreads), 0, s>>> (a, tiles_m, tiles_n, per_xcd, ksplit, ws);
  if (ksplit > 1)
    {
      const size_t total = (size_t)a.M * a.N;
      skinny2_reduce_kernel<<<dim3 ((unsigned)((total + 255) / 256)), dim3 (256), 0, s>>> (
          a, ws, ksplit, a.M);
    }
  return (int)hipGetLastError ();
}
} // namespace

float *
gemm_stream_workspace (hipStream_t s)
{
  return skinny2_workspace (s);
}

size_t
gemm_stream_workspace_bytes ()
{
  return kSk2Workspace;
}

int
gemm_reduce_parts (const GemmArgs &a, const float *ws, int parts, int rows, hipStream_t s)
{
  const size_t total = (size_t)a.M * a.N;
  skinny2_reduce_kernel<<<dim3 ((unsigned)((total + 255) / 256)), dim3 (256), 0, s>>> (a, ws, parts, rows);
  return (int)hipGetLastError ();
}

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
  if (a.batch > 65535)
    return false;
  if (a.wtype == 2) // [K, N] operand: vector loads along N
    return a.nmat == 1 && !a.upgate && (a.N % 8) == 0 && (a.ws % 8) == 0
           && ((uintptr_t)a.wh[0] % 16) == 0 && (a.wbs % 8) == 0
           && (a.xbs % 8) == 0;
  if (a.wtype == 1)
    {
      if ((a.ws % 8) != 0 || (a.wbs % 8) != 0 || (a.xbs % 8) != 0)
        return false;
      for (int t = 0; t < (a.upgate ? 2 : a.nmat); ++t)
        if (((uintptr_t)a.wh[t] % 16) != 0)
          return false;
      return true;
    }
  return false;
}

namespace
{
// the few-row, weight-streaming form: up to 32 rows, one problem, no batch
bool
few_rows_form (const GemmArgs &a)
{
  return a.M <= 32 && a.batch <= 1 && a.wtype != 2 && (a.wtype == 8 || (a.K % 16) == 0);
}

// the half-height tile for few rows, and where full tiles would be too few to
// occupy the compute units (a few hundred token rows)
bool
half_height_tiles (const GemmArgs &a)
{
  if (a.M <= 64)
    return true;
  const long tiles = (long)((a.M + 127) / 128) * ((a.N + (a.upgate ? 63 : 127)) / (a.upgate ? 64 : 128))
                     * (a.batch > 1 ? a.batch : 1) * (a.upgate ? 1 : a.nmat);
  return tiles < kGemmFewTiles;
}
} // namespace

GemmPlan
gemm_plan (const GemmArgs &a)
{
  GemmPlan p = { GEMM_NONE, 0, 1, 0, 0, 0 };
  if (!gemm_mfma_supported (a))
    return p;
  const size_t nm = a.upgate ? 2 : a.nmat;
  const size_t have = a.workspace ? std::min (a.workspace_bytes, kSk2Workspace) : kSk2Workspace;
  // up to 128 token rows against many weight rows: workgroups that run over
  // the whole of K, no partial sums
  if (const int g = gemm_rowsfull_groups (a))
    {
      const int step = gemm_rowsfull_launch_rows (a);
      p.family = GEMM_ROWSFULL, p.groups = g;
      p.tile_rows = a.M <= 32 ? 32 : (a.M <= 64 ? 64 : (a.M <= step ? 96 : step));
      p.launches = (a.M + step - 1) / step;
      return p;
    }
  if (few_rows_form (a))
    {
      // Q8_0: the whole-line forms with slices of 512 if their sums fit the
      // scratch, else (and for fp16 weights) slices of 1024
      if (a.wtype == 8)
        {
          const int S = (a.Kp + kR64Slice - 1) / kR64Slice;
          const size_t need = nm * S * 32 * a.N * sizeof (float);
          if (need <= have)
            {
              p.family = (a.Kp % 256) == 0 ? GEMM_ROWS128 : GEMM_ROWS64;
              p.tile_rows = 32, p.ksplit = S, p.launches = 2, p.workspace_bytes = need;
              return p;
            }
        }
      const int S = a.wtype == 8 ? skinny2_slices<8> (a) : skinny2_slices<1> (a);
      const size_t need = nm * S * 32 * a.N * sizeof (float);
      if (need <= have)
        {
          p.family = GEMM_SLICES, p.tile_rows = 32, p.ksplit = S, p.launches = 2;
          p.workspace_bytes = need;
          return p;
        }
    }
  int wide_rows = 0, wide_ks = 1;
  gemm_wide_choice (a, &wide_rows, &wide_ks);
  if (wide_rows)
    {
      p.family = GEMM_WIDE, p.tile_rows = wide_rows, p.ksplit = wide_ks;
      p.launches = wide_ks > 1 ? 2 : 1;
      p.workspace_bytes = wide_ks > 1 ? (size_t)wide_ks * a.M * a.N * sizeof (float) : 0;
      return p;
    }
  const bool small = half_height_tiles (a);
  p.family = GEMM_TILE, p.tile_rows = small ? 64 : 128;
  if (a.wtype == 8)
    p.ksplit = small ? tile_ksplit<64, 8> (a) : tile_ksplit<128, 8> (a);
  else if (a.wtype == 1)
    p.ksplit = small ? tile_ksplit<64, 1> (a) : tile_ksplit<128, 1> (a);
  p.launches = p.ksplit > 1 ? 2 : 1;
  p.workspace_bytes = p.ksplit > 1 ? nm * p.ksplit * a.M * a.N * sizeof (float) : 0;
  return p;
}

int
gemm_mfma_launch (const GemmArgs &a, hipStream_t s)
{
  const GemmPlan p = gemm_plan (a);
  int err = 0;
  switch (p.family)
    {
    case GEMM_ROWSFULL:
      return gemm_rowsfull_launch (a, s);
    case GEMM_ROWS128:
    case GEMM_ROWS64:
      if (launch_rows64_q8 (a, s, err))
        return err;
      break;
    case GEMM_SLICES:
      if (a.wtype == 8 ? launch_skinny2<8> (a, s, err) : launch_skinny2<1> (a, s, err))
        return err;
      break;
    case GEMM_WIDE:
      return gemm_wide_launch (a, s);
    case GEMM_TILE:
      {
        const bool small = p.tile_rows == 64;
        if (a.wtype == 8)
          return small ? launch_cfg<64, 8> (a, p.ksplit, s) : launch_cfg<128, 8> (a, p.ksplit, s);
        if (a.wtype == 2)
          return small ? launch_cfg<64, 2> (a, p.ksplit, s) : launch_cfg<128, 2> (a, p.ksplit, s);
        return small ? launch_cfg<64, 1> (a, p.ksplit, s) : launch_cfg<128, 1> (a, p.ksplit, s);
      }
    default:
      return (int)hipErrorInvalidValue;
    }
  // (a sliced form that could not get its scratch buffer or raise its LDS limit)
  return err ? err : (int)hipErrorOutOfMemory;
}

size_t
gemm_mfma_workspace_bytes (const GemmArgs &a)
{
  return gemm_plan (a).workspace_bytes;
}

void
gemm_release_workspace (hipStream_t s)
{
  std::lock_guard<std::mutex> lock (g_ws_mu);
  for (auto it = g_ws_table.begin (); it != g_ws_table.end ();)
    if (it->first.second == s)
      {
        (void)hipFree (it->second);
        it = g_ws_table.erase (it);
      }
    else
      ++it;
}

float *
gemm_static_scratch (size_t *bytes)
{
  if (bytes)
    *bytes = kStaticScratchBytes;
  int dev = 0;
  if (hipGetDevice (&dev) != hipSuccess || dev < 0 || dev >= 16)
    return nullptr;
  std::lock_guard<std::mutex> lock (g_ws_mu);
  if (!g_static_scratch[dev])
    {
      // with this device current: the address of ITS copy of the array
      void *p = nullptr;
      if (hipGetSymbolAddress (&p, HIP_SYMBOL (scratch)) != hipSuccess)
        return nullptr;
      g_static_scratch[dev] = (float *)p;
    }
  return g_static_scratch[dev];
}
} // namespace vkl

extern "C" int
vkl_debug_static_scratch (void **ptr, size_t *bytes)
{
  VKL_CHECK_ARG (ptr && bytes);
  *ptr = vkl::gemm_static_scratch (bytes);
  return *ptr ? 0 : (int)hipErrorInvalidSymbol;
}

extern "C" int
vkl_gemm_plan (int M, int N, int K, int wtype, int nmat, int upgate, size_t workspace_bytes,
               vkl_gemm_plan_t *out)
{
  VKL_CHECK_ARG (out && M > 0 && N > 0 && K > 0 && (wtype == 8 || wtype == 1));
  VKL_CHECK_ARG ((nmat == 1 || nmat == 3) && (upgate == 0 || (upgate == 1 && nmat == 1)));
  *out = vkl_gemm_plan_t{ 7, 1, 1, 0, M, 0 };
  if (M < (wtype == 8 ? vkl::kGemmMinRows : vkl::kGemmMinRowsF16))
    return 0;
  // dense, aligned stand-ins for the operands: only their alignment is looked at
  vkl::GemmArgs g = {};
  uint8_t *const aligned = (uint8_t *)4096;
  g.x = (const uint16_t *)aligned, g.xs = (size_t)K;
  g.M = M, g.N = N, g.K = K, g.Kp = (K + 31) / 32 * 32;
  g.wtype = wtype, g.batch = 1, g.nmat = nmat, g.upgate = upgate;
  for (int t = 0; t < 3; ++t)
    {
      g.wq[t] = aligned, g.wd[t] = (const uint16_t *)aligned, g.wh[t] = (const uint16_t *)aligned;
      g.y[t] = (uint16_t *)aligned;
    }
  g.ws = (size_t)K, g.ys = (size_t)N, g.scale = 1.0f;
  if (workspace_bytes)
    g.workspace = (float *)aligned, g.workspace_bytes = workspace_bytes;
  const vkl::GemmPlan p = vkl::gemm_plan (g);
  if (p.family != vkl::GEMM_NONE)
    *out = vkl_gemm_plan_t{ p.family, p.tile_rows, p.ksplit, p.groups, p.launches, p.workspace_bytes };
  return 0;
}

#ifdef VKL_TRACE
extern "C" void
vkl_debug_set_r64_trace (void *buf)
{
  (void)hipMemcpyToSymbol (HIP_SYMBOL (vkl::g_r64_trace), &buf, sizeof (buf));
}
#endif
