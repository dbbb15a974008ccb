// y[M,N] = x[M,K] W[N,K]^T for at most 96 token rows and planar Q8_0 weights
// with many rows (the fused K/Q/V and up/gate products of a short prompt):
// every workgroup runs over the whole of K, so there are no partial sums to
// store and no second launch to add them.
//
// A workgroup owns G groups of 16 weight rows (consecutive groups of the
// concatenated matrices; for the fused up/gate pair G/2 groups of each matrix,
// the same rows in both).  16 rows are one operand of v_mfma_f32_16x16x32_f16:
// A = x (16 tokens x 32 k, once per 16 token rows), B = 16 weight rows of one
// Q8_0 block, so the four sums of a lane all belong to one weight row and take
// one block scale: sum = fma (block sum, d, sum), blocks in order.
//
// K is walked in steps of 256 (8 blocks).  A workgroup is alone on its compute
// unit, so the loads it keeps in flight are all that hides the memory latency
// (2.5-3 us for the weights under load; a compute unit gets about 45 KiB of
// requests served per round trip, so rings deeper than that only queue): the
// step's int8 tiles (16 G x 256 bytes) and scales (16 G x 16 bytes) go
// straight into an LDS ring DW steps deep (global_load_lds_dwordx4, 1 KiB per
// instruction: 8 rows x 128 bytes, stored XOR-swizzled by the choice of which
// chunk a lane fetches, or 64 rows of scales), issued by NL waves that do
// nothing else.  The x tile of a step (32 to 96 rows x 512 bytes, from L2) is as
// large as the weights of three to five groups, so it has a ring of its own, only DX deep, and
// is issued by the KS multiplying waves.  The two kinds of load must come from
// different waves: a wave's loads complete in order, so a wait for a recent x
// tile would also wait for every weight tile requested before it.  Each wave
// counts its own loads (s_waitcnt vmcnt) before the step's one barrier.
//
// Multiplying wave p takes blocks 8 p / KS ... of every step for all G groups
// (one read of an x fragment serves G products); the epilogue adds the KS
// parts in order of p.
#include "vkl_common.h"
#include "vkl_gemm.h"
#include "vkl_gemm_finish.h"

namespace vkl
{
namespace
{
typedef _Float16 half8 __attribute__ ((ext_vector_type (8)));
typedef float f32x4 __attribute__ ((ext_vector_type (4)));
// (vector types, not HIP's structs: LDS reads of a struct type are taken to
// alias the tiles in flight and made to wait for all of them)
typedef uint32_t u32x2 __attribute__ ((ext_vector_type (2)));
#define VKL_LDS __attribute__ ((address_space (3)))

constexpr int kRfStep = 256;                 // k per step
constexpr int kRfXBytes = 32 * kRfStep * 2;  // x tile of a step, per 32 token rows
constexpr int kRfParkLd = 17;                // floats per parked row of 16

template <int G> struct RfGeo
{
  static constexpr int SI = (16 * G + 63) / 64; // scale load instructions per step
  static constexpr int SBASE = G * 4096;        // scales within a weight stage
  static constexpr int WSTAGE = SBASE + SI * 1024;
  static constexpr int WJOBS = 4 * G + SI;      // weight load instructions per step
};
constexpr int kRfXJobs = 16; // x load instructions per step and 32 token rows

template <int G, int KS, int DX, int DW, int TB>
constexpr size_t
rowsfull_lds ()
{
  const size_t ring = (size_t)DX * TB * kRfXBytes + (size_t)DW * RfGeo<G>::WSTAGE,
               park = (size_t)G * KS * 32 * kRfParkLd * 4;
  return ring > park ? ring : park;
}

__device__ __forceinline__ half8
rf_q8_frag (u32x2 r)
{
  h16x2 a, b, c, d;
  i8x4_to_h2x2 (r.x, a, b);
  i8x4_to_h2x2 (r.y, c, d);
  half8 o;
  o[0] = a[0], o[1] = a[1], o[2] = b[0], o[3] = b[1];
  o[4] = c[0], o[5] = c[1], o[6] = d[0], o[7] = d[1];
  return o;
}

template <int N>
__device__ __forceinline__ void
rf_wait_loads ()
{
  // at most N of the wave's loads still in flight, and none of its LDS reads
  static_assert (N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt ((0x0f70 | (N & 15) | ((N >> 4) << 14)) & ~0x0f00);
}

// groups: 16-row groups over all matrices (fused pair: per matrix); gpm: per matrix.
// TB: blocks of 32 token rows (1 to 3).
template <int G, int KS, int NL, int DX, int DW, int TB, bool UPGATE>
__global__ __launch_bounds__ ((KS + NL) * 64) void
gemm_rowsfull_q8_kernel (const GemmArgs a, int groups, int gpm, int vec)
{
  using Geo = RfGeo<G>;
  constexpr int NW = KS + NL, BPW = 8 / KS;
  constexpr int XBYTES = TB * kRfXBytes, RB = 4 * TB; // RB: blocks of 8 token rows
  constexpr int LX = TB * kRfXJobs / KS;                                     // x loads per multiplying wave and step
  constexpr int WJOBS = Geo::WJOBS, LWL = (WJOBS + NL - 1) / NL, REM = WJOBS % NL; // weight loads per loading wave
  constexpr int LJ = LX > LWL ? LX : LWL;
  constexpr int WSTAGE = Geo::WSTAGE, WRING = DX * XBYTES;
  static_assert (KS == 4 || KS == 8, "blocks of a step and x loads divide among the multiplying waves");
  static_assert (DX >= 2 && DW >= 3 && (DX - 2) * LX < 64 && (DW - 2) * LWL < 64, "loads in flight fit the wait counter");
  extern __shared__ __align__ (16) uint8_t rf_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane (threadIdx.x >> 6);
  const bool mul = wave < KS; // a multiplying wave (else a loading wave)
  const int p = wave, ld = wave - KS;
  const int nks = a.K / kRfStep;

  // group gg of this workgroup: matrix, first weight row, and whether it exists
  // (past the end: the last group again, loaded and multiplied but not stored)
  auto group = [&] (int gg, int &mat, int &row0) -> bool {
    if (UPGATE)
      {
        const int pair = blockIdx.x * (G / 2) + (gg >> 1);
        mat = gg & 1;
        row0 = 16 * min (pair, groups - 1);
        return pair < groups;
      }
    const int gi = blockIdx.x * G + gg, gc = min (gi, groups - 1);
    mat = gc / gpm;
    row0 = 16 * (gc - mat * gpm);
    return gi < groups;
  };

  // the wave's load instructions of a step: x job q = p + KS t, or weight job
  // q = ld + NL t
  const uint8_t *src[LJ];
  uint32_t ldo[LJ], inc[LJ];
  const int lr = lane >> 3, chunk = (lane & 7) ^ lr;
#pragma unroll
  for (int t = 0; t < LJ; ++t)
    {
      src[t] = (const uint8_t *)a.x;
      ldo[t] = 0, inc[t] = 0;
      if (mul)
        {
          if (t < LX)
            {
              // x: 64-wide quarter q / RB of the step, token rows 8 (q % RB) ...
              const int q = p + KS * t;
              const int m = min (8 * (q % RB) + lr, a.M - 1);
              src[t] = (const uint8_t *)(a.x + (size_t)m * a.xs + 64 * (q / RB) + 8 * chunk);
              ldo[t] = q * 1024, inc[t] = kRfStep * 2;
            }
        }
      else if (t < LWL)
        {
          const int q = ld + NL * t;
          if (q < 4 * G)
            {
              // int8 plane: group, 128-wide half, rows 8 (jj % 2) ...
              const int gg = q >> 2, jj = q & 3;
              int mat, row0;
              group (gg, mat, row0);
              const uint8_t *w = mat == 0 ? a.wq[0] : (mat == 1 ? a.wq[1] : a.wq[2]);
              const int n = min (row0 + 8 * (jj & 1) + lr, a.N - 1);
              src[t] = w + (size_t)n * a.Kp + 128 * (jj >> 1) + 16 * chunk;
              ldo[t] = q * 1024, inc[t] = kRfStep;
            }
          else
            {
              // scales: lane = row of the workgroup's 16 G, its 8 scales of the step
              const int s = min (q - 4 * G, Geo::SI - 1);
              const int v = min (64 * s + lane, 16 * G - 1);
              int mat, row0;
              group (v >> 4, mat, row0);
              const uint16_t *ds = mat == 0 ? a.wd[0] : (mat == 1 ? a.wd[1] : a.wd[2]);
              const int n = min (row0 + (v & 15), a.N - 1);
              src[t] = (const uint8_t *)(ds + (size_t)n * (a.Kp >> 5));
              ldo[t] = Geo::SBASE + s * 1024, inc[t] = kRfStep / 32 * 2;
            }
        }
    }
  // (the last of a loading wave's LWL is missing for the waves past REM)
  const bool full = REM == 0 || ld < REM;
  auto issue_x = [&] (int tile, int st) {
#pragma unroll
    for (int t = 0; t < LX; ++t)
      __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)(src[t] + (size_t)((uint32_t)tile * inc[t])),
                                        (VKL_LDS void *)(rf_lds + st * XBYTES + ldo[t]), 16, 0, 0);
  };
  auto issue_w = [&] (int tile, int st) {
#pragma unroll
    for (int t = 0; t < LWL; ++t)
      if (t + 1 < LWL || full)
        {
        __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)(src[t] + (size_t)((uint32_t)tile * inc[t])),
                                          (VKL_LDS void *)(rf_lds + WRING + st * WSTAGE + ldo[t]), 16, 0, 0);
        }
  };
  if (mul)
    {
#pragma unroll
      for (int s = 0; s < DX - 1; ++s)
        issue_x (min (s, nks - 1), s);
    }
  else
    {
#pragma unroll
      for (int s = 0; s < DW - 1; ++s)
        issue_w (min (s, nks - 1), s);
    }

  // fragment addresses of the wave's blocks b = p BPW + bb: lane (i, kq) holds
  // token (or weight row) i, k = 32 b + 8 kq ... + 7
  const int fi = lane & 15, kq = lane >> 4;
  uint32_t aoff[BPW], boff[BPW], soff[BPW];
#pragma unroll
  for (int bb = 0; bb < BPW; ++bb)
    {
      const int b = (mul ? p : 0) * BPW + bb;
      aoff[bb] = ((b >> 1) * RB + (fi >> 3)) * 1024 + (fi & 7) * 128 + (((4 * (b & 1) + kq) ^ (fi & 7)) << 4);
      boff[bb] = WRING + ((b >> 2) * 2 + (fi >> 3)) * 1024 + (fi & 7) * 128
                 + (((2 * (b & 3) + (kq >> 1)) ^ (fi & 7)) << 4) + 8 * (kq & 1);
      soff[bb] = WRING + Geo::SBASE + fi * 16 + b * 2;
    }

  f32x4 acc[G][2 * TB]; // [group][block of 16 token rows]
#pragma unroll
  for (int gg = 0; gg < G; ++gg)
#pragma unroll
    for (int tb = 0; tb < 2 * TB; ++tb)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc[gg][tb][e] = 0.f;
  int xst = 0, wst = 0;
  for (int kt = 0; kt < nks; ++kt)
    {
      // this wave's part of tile kt has landed (the barrier covers the others')
      // and every wave has read the last of tile kt - 1: its stages take tiles
      // kt + DX - 1 and kt + DW - 1 (past the end the last tile again, which
      // nothing reads)
      if (mul)
        rf_wait_loads<(DX - 2) * LX> ();
      else if (full)
        rf_wait_loads<(DW - 2) * LWL> ();
      else
        rf_wait_loads<(DW - 2) * (LWL - 1)> ();
      __builtin_amdgcn_s_barrier ();
      __builtin_amdgcn_sched_barrier (0);
      if (!mul)
        issue_w (min (kt + DW - 1, nks - 1), wst == 0 ? DW - 1 : wst - 1);
      else
        {
          issue_x (min (kt + DX - 1, nks - 1), xst == 0 ? DX - 1 : xst - 1);
          const uint32_t xb = xst * XBYTES, wb = wst * WSTAGE;
          // all of the step's fragments first, then the products as they arrive
          half8 af[BPW][2 * TB];
          u32x2 bq[G][BPW];
          uint16_t sc[G][BPW];
#pragma unroll
          for (int bb = 0; bb < BPW; ++bb)
            {
              // (all blocks of 16 token rows, also those past M: they repeat row M - 1)
#pragma unroll
              for (int tb = 0; tb < 2 * TB; ++tb)
                af[bb][tb] = *(const half8 *)(rf_lds + xb + aoff[bb] + tb * 2048);
#pragma unroll
              for (int gg = 0; gg < G; ++gg)
                {
                  bq[gg][bb] = *(const u32x2 *)(rf_lds + wb + boff[bb] + gg * 4096);
                  sc[gg][bb] = *(const uint16_t *)(rf_lds + wb + soff[bb] + gg * 256);
                }
            }
          __builtin_amdgcn_sched_barrier (0);
#pragma unroll
          for (int bb = 0; bb < BPW; ++bb)
#pragma unroll
            for (int gg = 0; gg < G; ++gg)
              {
                const half8 bf = rf_q8_frag (bq[gg][bb]);
                float d = h2f (sc[gg][bb]);
                // (keeps the conversion out of the products: as an fp16 operand
                // it would make them mixed-precision FMAs)
                asm volatile ("" : "+v"(d));
                const f32x4 z = { 0.f, 0.f, 0.f, 0.f };
                f32x4 part[2 * TB];
#pragma unroll
                for (int tb = 0; tb < 2 * TB; ++tb)
                  part[tb] = __builtin_amdgcn_mfma_f32_16x16x32_f16 (af[bb][tb], bf, z, 0, 0, 0);
#pragma unroll
                for (int tb = 0; tb < 2 * TB; ++tb)
#pragma unroll
                  for (int e = 0; e < 4; ++e)
                    acc[gg][tb][e] = __builtin_fmaf (part[tb][e], d, acc[gg][tb][e]);
              }
        }
      __builtin_amdgcn_sched_barrier (0);
      xst = xst == DX - 1 ? 0 : xst + 1;
      wst = wst == DW - 1 ? 0 : wst + 1;
    }

  // Epilogue through LDS: no load may still be writing there and every wave
  // has read its last fragments; then each multiplying wave parks its G blocks
  // of 32 x 16 sums (sum e of lane (j, kq): token 4 kq + e, weight row j) and
  // the workgroup walks the groups' outputs, a lane taking 8 neighbouring
  // columns of one token row.
  __builtin_amdgcn_s_waitcnt (0x0f70 & ~0x0f00);
  __builtin_amdgcn_s_barrier ();
  float *park = (float *)rf_lds;
  constexpr int GO = UPGATE ? G / 2 : G;
#pragma unroll
  for (int half = 0; half < TB; ++half) // 32 token rows at a time
    {
      if (half > 0)
        __syncthreads (); // the walk before is done with the parked sums
      if (mul)
        {
#pragma unroll
          for (int gg = 0; gg < G; ++gg)
            {
              float *pw = park + (p * G + gg) * (32 * kRfParkLd) + (4 * kq) * kRfParkLd + fi;
#pragma unroll
              for (int e = 0; e < 4; ++e)
                {
                  pw[e * kRfParkLd] = acc[gg][2 * half][e];
                  pw[(16 + e) * kRfParkLd] = acc[gg][2 * half + 1][e];
                }
            }
        }
      __syncthreads ();
      for (int u = threadIdx.x; u < GO * 64; u += NW * 64)
        {
          const int go = u >> 6, m = (u >> 1) & 31, c8 = u & 1;
          const int gg = UPGATE ? 2 * go : go;
          int mat, row0;
          if (!group (gg, mat, row0))
            continue;
          float v[8], gt[8];
#pragma unroll
          for (int e = 0; e < 8; ++e)
            v[e] = 0.f, gt[e] = 0.f;
#pragma unroll
          for (int pp = 0; pp < KS; ++pp)
            {
              const float *pr = park + (pp * G + gg) * (32 * kRfParkLd) + m * kRfParkLd + 8 * c8;
#pragma unroll
              for (int e = 0; e < 8; ++e)
                {
                  v[e] += pr[e];
                  if (UPGATE)
                    gt[e] += pr[32 * kRfParkLd + e];
                }
            }
          gemm_finish8<UPGATE> (a, v, gt, 32 * half + m, row0 + 8 * c8, mat, vec, nullptr);
        }
    }
}

// G, KS, NL, DX, DW per number of groups.  Deeper rings do not pay: past some
// 45 KiB of requests in flight per compute unit the memory system only queues
// them (7B K/Q/V at 32 rows: 16.9 us with DX 3 / DW 4, 18.2 us with 4 / 7).
#define RF_CFG1 1, 8, 1, 3, 6, 1
#define RF_CFG2 2, 8, 2, 3, 5, 1
#define RF_CFG3 3, 8, 2, 3, 4, 1
#define RF_CFG4 4, 8, 2, 3, 4, 1
#define RF_CFG6 6, 8, 4, 3, 3, 1
#define RF_CFG8 8, 8, 4, 3, 3, 1
// 33 to 64 token rows: the x tile of a step is 32 KiB
#define RF_CFG1W 1, 8, 1, 3, 6, 2
#define RF_CFG2W 2, 8, 2, 3, 5, 2
#define RF_CFG3W 3, 8, 2, 3, 4, 2
#define RF_CFG4W 4, 8, 2, 3, 3, 2
#define RF_CFG6W 6, 8, 4, 2, 3, 2
// 65 to 96 token rows (single matrices and K/Q/V only): 48 KiB
#define RF_CFG1X 1, 8, 1, 2, 6, 3
#define RF_CFG2X 2, 8, 2, 2, 5, 3
#define RF_CFG3X 3, 8, 2, 2, 4, 3
#define RF_CFG4X 4, 8, 2, 2, 3, 3
// Token rows per launch, and up to how many rows the form is used (two
// launches past the first figure: measured against the tile kernels at 7B,
// K/Q/V 128 rows 43 against 55 us, up/gate 96 rows 62 against 84 us, but 128
// rows 72 against 65 us)
constexpr int kRowsFullPlain = 96, kRowsFullPlainMax = 128;
constexpr int kRowsFullUpgate = 64, kRowsFullUpgateMax = 96;

// Groups per workgroup: a workgroup per compute unit at most (256), as many of
// them busy as the row count allows (0: another form)
int
rowsfull_plan (const GemmArgs &a)
{
  if (a.wtype != 8 || a.M > (a.upgate ? kRowsFullUpgateMax : kRowsFullPlainMax) || a.M < 1 || a.batch > 1 || a.K != a.Kp || (a.K % kRfStep) != 0 || a.K < 3 * kRfStep
      || (a.N % 16) != 0)
    return 0;
  for (int t = 0; t < (a.upgate ? 2 : a.nmat); ++t)
    if (((uintptr_t)a.wq[t] % 16) != 0 || ((uintptr_t)a.wd[t] % 16) != 0)
      return 0;
  if (((uintptr_t)a.x % 16) != 0 || (a.xs % 8) != 0)
    return 0;
  const int gpm = a.N / 16;
  if (a.upgate)
    {
      // rows per matrix and workgroup: 16 G / 2
      const int gr = (gpm + 255) / 256;
      return gr > (a.M > 32 ? 3 : 4) || gpm < 128 * gr ? 0 : 2 * gr;
    }
  const int total = gpm * a.nmat;
  const int gq = (total + 255) / 256;
  if (gq == 1)
    return a.M <= kRowsFullPlain && total >= 200 && a.K <= 4096 ? 1 : 0;
  return gq > 4 || total < 128 * gq ? 0 : gq;
}

template <int G, int KS, int NL, int DX, int DW, int TB, bool UPGATE>
int
rowsfull_run (const GemmArgs &a, int groups, int gpm, int vec, hipStream_t s)
{
  constexpr size_t lds = rowsfull_lds<G, KS, DX, DW, TB> ();
  static_assert (lds <= 160 * 1024, "a workgroup's LDS");
  static LdsLimit limit;
  if (int e = limit.raise ((const void *)gemm_rowsfull_q8_kernel<G, KS, NL, DX, DW, TB, UPGATE>, lds))
    return e;
  constexpr int per = UPGATE ? G / 2 : G;
  const dim3 grid ((unsigned)((groups + per - 1) / per));
  gemm_rowsfull_q8_kernel<G, KS, NL, DX, DW, TB, UPGATE><<<grid, dim3 ((KS + NL) * 64), lds, s>>> (a, groups, gpm, vec);
  return (int)hipGetLastError ();
}
} // namespace

bool
gemm_rowsfull_supported (const GemmArgs &a)
{
  return rowsfull_plan (a) != 0;
}

int
gemm_rowsfull_groups (const GemmArgs &a)
{
  return rowsfull_plan (a);
}

int
gemm_rowsfull_launch_rows (const GemmArgs &a)
{
  return a.upgate ? kRowsFullUpgate : kRowsFullPlain;
}

namespace
{
// one launch: up to 64 token rows for the fused up/gate pair, 96 otherwise
int
rowsfull_launch_rows (const GemmArgs &a, int g, int vec, hipStream_t s)
{
  const int gpm = a.N / 16;
  if (a.upgate && a.M > 32)
    {
      switch (g)
        {
        case 2: return rowsfull_run<RF_CFG2W, true> (a, gpm, gpm, vec, s);
        case 4: return rowsfull_run<RF_CFG4W, true> (a, gpm, gpm, vec, s);
        case 6: return rowsfull_run<RF_CFG6W, true> (a, gpm, gpm, vec, s);
        }
      return (int)hipErrorInvalidValue;
    }
  if (a.upgate)
    {
      switch (g)
        {
        case 2: return rowsfull_run<RF_CFG2, true> (a, gpm, gpm, vec, s);
        case 4: return rowsfull_run<RF_CFG4, true> (a, gpm, gpm, vec, s);
        case 6: return rowsfull_run<RF_CFG6, true> (a, gpm, gpm, vec, s);
        case 8: return rowsfull_run<RF_CFG8, true> (a, gpm, gpm, vec, s);
        }
      return (int)hipErrorInvalidValue;
    }
  const int total = gpm * a.nmat;
  if (a.M > 64)
    switch (g)
      {
      case 1: return rowsfull_run<RF_CFG1X, false> (a, total, gpm, vec, s);
      case 2: return rowsfull_run<RF_CFG2X, false> (a, total, gpm, vec, s);
      case 3: return rowsfull_run<RF_CFG3X, false> (a, total, gpm, vec, s);
      case 4: return rowsfull_run<RF_CFG4X, false> (a, total, gpm, vec, s);
      }
  if (a.M > 32)
    switch (g)
      {
      case 1: return rowsfull_run<RF_CFG1W, false> (a, total, gpm, vec, s);
      case 2: return rowsfull_run<RF_CFG2W, false> (a, total, gpm, vec, s);
      case 3: return rowsfull_run<RF_CFG3W, false> (a, total, gpm, vec, s);
      case 4: return rowsfull_run<RF_CFG4W, false> (a, total, gpm, vec, s);
      }
  switch (g)
    {
    case 1: return rowsfull_run<RF_CFG1, false> (a, total, gpm, vec, s);
    case 2: return rowsfull_run<RF_CFG2, false> (a, total, gpm, vec, s);
    case 3: return rowsfull_run<RF_CFG3, false> (a, total, gpm, vec, s);
    case 4: return rowsfull_run<RF_CFG4, false> (a, total, gpm, vec, s);
    }
  return (int)hipErrorInvalidValue;
}
} // namespace

int
gemm_rowsfull_launch (const GemmArgs &a, hipStream_t s)
{
  const int g = rowsfull_plan (a);
  if (!g)
    return (int)hipErrorInvalidValue;
  int vec = (a.ys % 8) == 0 && (!a.residual || ((uintptr_t)a.residual % 16) == 0)
            && (!a.y32 || ((a.N % 4) == 0 && ((uintptr_t)a.y32 % 16) == 0));
  for (int t = 0; t < (a.upgate ? 1 : a.nmat); ++t)
    vec = vec && ((uintptr_t)a.y[t] % 16) == 0;
  // more rows than one launch holds: a second launch for the rest (the
  // weights are read twice, still faster than the tile kernels up there)
  const int step = a.upgate ? kRowsFullUpgate : kRowsFullPlain;
  for (int m0 = 0; m0 < a.M; m0 += step)
    {
      GemmArgs c = a;
      c.M = a.M - m0 < step ? a.M - m0 : step;
      c.x = a.x + (size_t)m0 * a.xs;
      for (int t = 0; t < 3; ++t)
        if (c.y[t])
          c.y[t] = a.y[t] + (size_t)m0 * a.ys;
      if (c.residual)
        c.residual = a.residual + (size_t)m0 * a.ys;
      if (c.y32)
        c.y32 = a.y32 + (size_t)m0 * a.N;
      const int err = rowsfull_launch_rows (c, g, vec, s);
      if (err)
        return err;
    }
  return 0;
}
} // namespace vkl
