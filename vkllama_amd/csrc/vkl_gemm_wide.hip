// y[M,N] = x[M,K] W[N,K]^T for many token rows (prompt passes of a thousand
// tokens and more), fp16 activations and dense fp16 weights, fp32 accumulation
// on the matrix cores (v_mfma_f32_32x32x16_f16).
//
// One workgroup of four waves per compute unit owns a 256 x 128 output tile;
// each wave a 128 x 64 quarter (4 x 2 accumulators of 32 x 32).  A k-step is 64
// wide, so a tile row is one 128-byte cache line.  The tiles of x and W do not
// pass through registers on their way in: global_load_lds_dwordx4 writes them
// straight into LDS, three k-steps deep (3 x 48 KiB), one 1 KiB instruction
// per 8 tile rows.  Such an instruction writes its 64 x 16 bytes to consecutive
// LDS addresses, so rows cannot be padded against bank conflicts; instead every
// lane fetches the 16-byte chunk (slot ^ f(row)) of its row, which stores the
// row XOR-swizzled, and the fragment reads apply the same f.
//
// The k loop is scheduled by hand (sched_group_barrier): the products of one
// quarter of a k-step are issued alternately with the fragment reads of the
// next quarter and with a share of the loads for the k-step after next, so the
// single wave of a SIMD keeps the matrix core fed.  The barrier that hands over
// the next k-step sits before the last quarter, whose products then overlap
// with the first fragment reads of that step.
//
// Measured on the 7B shapes at 2048 rows: matrix cores busy 63 % of the cycles
// (the tile kernel of vkl_gemm_mfma.hip, which stages through registers:
// 30-39 %).
#include "vkl_common.h"
#include "vkl_gemm.h"

namespace vkl
{
namespace
{
typedef _Float16 half8 __attribute__ ((ext_vector_type (8)));
typedef float float16v __attribute__ ((ext_vector_type (16)));
#define VKL_LDS __attribute__ ((address_space (3)))

constexpr int WBM = 256, WBN = 128, WBK = 64;
constexpr int WSTAGES = 3;
constexpr int WWAVES = 4;                       // 2 x 2
constexpr int WTM = WBM / 2 / 32, WTN = WBN / 2 / 32;
constexpr int WROWB = WBK * 2;                  // bytes of a tile row
constexpr int WSTAGE_BYTES = (WBM + WBN) * WROWB;
constexpr int WGPW = (WBM + WBN) / 8 / WWAVES;  // 1 KiB load instructions per wave and k-step
constexpr int WAG = WBM / 8 / WWAVES;           // of which rows of x
constexpr size_t kWideLds = (size_t)WSTAGES * WSTAGE_BYTES;

// Issue order of one quarter of a k-step: after product Q one fragment read
// (the first NR products) and an even share of the quarter's LQ loads.
template <int Q, int NP, int NR, int LQ> struct WideOrder
{
  static __device__ __forceinline__ void
  run ()
  {
    __builtin_amdgcn_sched_group_barrier (0x008, 1, 0); // one MFMA
    if constexpr (Q < NR)
      __builtin_amdgcn_sched_group_barrier (0x100, 1, 0); // one LDS read
    constexpr int nl = LQ * (Q + 1) / NP - LQ * Q / NP;
    if constexpr (nl > 0)
      __builtin_amdgcn_sched_group_barrier (0x020, nl, 0); // loads
    if constexpr (Q + 1 < NP)
      WideOrder<Q + 1, NP, NR, LQ>::run ();
  }
};

template <int V> struct WideInt
{
  static constexpr int value = V;
};

template <bool UPGATE>
__global__ __launch_bounds__ (WWAVES * 64) void
gemm_wide_f16_kernel (const GemmArgs a, int tiles_m, int tiles_n, int per_xcd, int vec)
{
  extern __shared__ __align__ (16) uint8_t wide_lds[];
  // workgroups go to the XCDs in turn: each XCD gets a contiguous range of
  // tiles, token-row tile fastest, so the weight tiles it shares stay in its L2
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int tile = xcd * per_xcd + j;
  if (j >= per_xcd || tile >= tiles_m * tiles_n)
    return;
  const int tn = tile / tiles_m, tm = tile - tn * tiles_m;
  const int bn_rows = UPGATE ? WBN / 2 : WBN; // weight rows per matrix and tile
  const int m0 = tm * WBM, n0 = tn * bn_rows;
  const int zmat = blockIdx.z;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane (threadIdx.x >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // Load addresses.  Instruction i of a wave covers tile rows 8g .. 8g+7 with
  // g = wave + 4 i (x for i < WAG, then W); lane l fetches row 8g + l/8, and
  // LDS slot l%8 of that row receives chunk (l%8) ^ f(row), f(row) = (row & 7)
  // ^ ((row >> 3) & 1): 8 or 16 consecutive rows then hit different banks at
  // the same chunk.  Rows beyond M or N repeat the last row (never stored).
  const int lr = lane >> 3;
  const int chunk = (lane & 7) ^ lr ^ (wave & 1);
  const uint16_t *src[WGPW];
#pragma unroll
  for (int i = 0; i < WAG; ++i)
    {
      const int m = min (m0 + (wave + WWAVES * i) * 8 + lr, a.M - 1);
      src[i] = a.x + (size_t)m * a.xs + chunk * 8;
    }
#pragma unroll
  for (int i = WAG; i < WGPW; ++i)
    {
      const int v = (wave + WWAVES * (i - WAG)) * 8 + lr; // row of the weight tile
      const int mat = UPGATE ? v >> 6 : zmat;
      const int n = min (UPGATE ? n0 + (v & 63) : n0 + v, a.N - 1);
      const uint16_t *w = mat == 0 ? a.wh[0] : (mat == 1 ? a.wh[1] : a.wh[2]);
      src[i] = w + (size_t)n * a.ws + chunk * 8;
    }

  // fragment reads: lane l holds row l%32 of a 32-row block, k = 16 ks + 8 (l/32) .. +7
  const int fsw = (lane & 7) ^ ((lane >> 3) & 1);
  uint32_t aoff[4], boff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
    {
      const int ko = ((2 * ks + (lane >> 5)) ^ fsw) << 4;
      aoff[ks] = (wm * (WBM / 2) + (lane & 31)) * WROWB + ko;
      boff[ks] = WBM * WROWB + ((UPGATE ? wn * 32 : wn * 64) + (lane & 31)) * WROWB + ko;
    }
  constexpr int BJ = (UPGATE ? 64 : 32) * WROWB; // from a wave's first to its second column block

  float16v acc[WTM][WTN];
#pragma unroll
  for (int i = 0; i < WTM; ++i)
#pragma unroll
    for (int jn = 0; jn < WTN; ++jn)
#pragma unroll
      for (int q = 0; q < 16; ++q)
        acc[i][jn][q] = 0.f;

  const int nk = a.K / WBK;
  auto issue_part = [&] (int kt, int st, int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
      {
        const int g = i < WAG ? wave + WWAVES * i : WBM / 8 + wave + WWAVES * (i - WAG);
        __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)(src[i] + (size_t)kt * WBK),
                                          (VKL_LDS void *)(wide_lds + st * WSTAGE_BYTES + g * 1024), 16, 0, 0);
      }
  };
#pragma unroll
  for (int p = 0; p < WSTAGES - 1; ++p)
    issue_part (p < nk ? p : nk - 1, p, 0, WGPW);

  half8 af[2][WTM], bf[2][WTN];
  // in the order the products need them
  auto read_frags = [&] (int st, int ks, int buf) {
    const uint8_t *sb = wide_lds + st * WSTAGE_BYTES;
    af[buf][0] = *(const half8 *)(sb + aoff[ks]);
#pragma unroll
    for (int jn = 0; jn < WTN; ++jn)
      bf[buf][jn] = *(const half8 *)(sb + boff[ks] + jn * BJ);
#pragma unroll
    for (int i = 1; i < WTM; ++i)
      af[buf][i] = *(const half8 *)(sb + aoff[ks] + i * 32 * WROWB);
  };
  // s_waitcnt immediates: vmcnt = the loads of the newest k-step may stay in
  // flight; the second one also waits for the wave's own LDS reads
  constexpr int VMW = (WSTAGES - 2) * WGPW;
  constexpr int WAITVM = 0x0f70 | (VMW & 15) | ((VMW >> 4) << 14);
  constexpr int LB1 = WGPW / 3, LB2 = 2 * WGPW / 3;
  constexpr int NR = WTM + WTN, NP = WTM * WTN;
  // One k-step.  On entry tile kt is in stage ST and the fragments of its
  // first quarter are on their way into buffer 0.
  auto step = [&] (int kt, auto stc) {
    constexpr int ST = decltype (stc)::value;
    constexpr int SN = (ST + WSTAGES - 1) % WSTAGES, S1 = (ST + 1) % WSTAGES;
    // the loads of tile kt + 2 go to the stage that was multiplied in the step
    // before (every wave has passed that step's barrier); past the end they
    // repeat the last tile into a stage nothing reads
    const int kn = kt + WSTAGES - 1 < nk ? kt + WSTAGES - 1 : nk - 1;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
      {
        if (ks < 3)
          {
            read_frags (ST, ks + 1, (ks + 1) & 1);
            issue_part (kn, SN, ks == 0 ? 0 : ks == 1 ? LB1 : LB2, ks == 0 ? LB1 : ks == 1 ? LB2 : WGPW);
          }
        else
          {
            // tile kt + 1 has landed (this wave's part; the barrier covers the
            // others') and this wave has read the last of tile kt
            __builtin_amdgcn_s_waitcnt (WAITVM & ~0x0f00);
            __builtin_amdgcn_s_barrier ();
            __builtin_amdgcn_sched_barrier (0);
            read_frags (S1, 0, 0);
          }
#pragma unroll
        for (int i = 0; i < WTM; ++i)
#pragma unroll
          for (int jn = 0; jn < WTN; ++jn)
            acc[i][jn] = __builtin_amdgcn_mfma_f32_32x32x16_f16 (af[ks & 1][i], bf[ks & 1][jn], acc[i][jn], 0, 0, 0);
        if (ks == 0)
          WideOrder<0, NP, NR, LB1>::run ();
        else if (ks == 1)
          WideOrder<0, NP, NR, LB2 - LB1>::run ();
        else if (ks == 2)
          WideOrder<0, NP, NR, WGPW - LB2>::run ();
        else
          WideOrder<0, NP, NR, 0>::run ();
        __builtin_amdgcn_sched_barrier (0);
      }
  };
  __builtin_amdgcn_s_waitcnt (WAITVM);
  __builtin_amdgcn_s_barrier ();
  read_frags (0, 0, 0);
  __builtin_amdgcn_sched_barrier (0);
  int kt = 0;
  for (; kt + WSTAGES <= nk; kt += WSTAGES)
    {
      step (kt, WideInt<0> ());
      step (kt + 1, WideInt<1> ());
      step (kt + 2, WideInt<2> ());
    }
  if (kt < nk)
    step (kt, WideInt<0> ());
  if (kt + 1 < nk)
    step (kt + 1, WideInt<1> ());
  __builtin_amdgcn_s_waitcnt (0x0f70); // no load may outlive the workgroup's LDS

  // Epilogue through LDS (the k loop's stages are free now): every wave parks
  // its 128 x 64 fp32 block in a region of its own, then walks it row-wise so
  // that a lane handles 8 neighbouring columns: 16-byte loads and stores, whole
  // cache lines per row, and a short loop instead of 128 unrolled elements.
  // Accumulator register q of lane l is row 8 (q/4) + 4 (l/32) + q%4, column
  // l%32 of its 32 x 32 block.
  __builtin_amdgcn_s_barrier (); // every wave has read its last fragments
  constexpr int LD = 68;         // floats per parked row: 16-byte aligned, rows 4 banks apart
  float *park = (float *)(wide_lds + wave * (128 * LD * 4));
  {
    float *pl = park + (lane >> 5) * 4 * LD + (lane & 31);
#pragma unroll
    for (int i = 0; i < WTM; ++i)
#pragma unroll
      for (int jn = 0; jn < WTN; ++jn)
#pragma unroll
        for (int q = 0; q < 16; ++q)
          pl[(i * 32 + (q >> 2) * 8 + (q & 3)) * LD + jn * 32] = acc[i][jn][q];
  }
  // (a wave reads back only what it wrote itself: no barrier)
  uint16_t *y = a.y[UPGATE ? 0 : zmat];
  constexpr int CPR = UPGATE ? 4 : 8;   // lanes per row
  constexpr int RPI = 64 / CPR;         // rows per iteration
  const int er = lane / CPR, ec = (lane % CPR) * 8;
  const int ncol0 = n0 + (UPGATE ? wn * 32 : wn * 64) + ec;
  const bool plain = a.nmat != 1;       // one of three fused outputs: no scale, activation, residual
  for (int it = 0; it < 128 / RPI; ++it)
    {
      const int row = it * RPI + er;
      const int m = m0 + wm * (WBM / 2) + row;
      const float4 p0 = *(const float4 *)(park + row * LD + ec);
      const float4 p1 = *(const float4 *)(park + row * LD + ec + 4);
      float v[8] = { p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w };
      if (UPGATE)
        {
          const float4 g0 = *(const float4 *)(park + row * LD + 32 + ec);
          const float4 g1 = *(const float4 *)(park + row * LD + 32 + ec + 4);
          const float g[8] = { g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w };
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
        continue;
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
          continue;
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
}

// fewest tiles for which this form is used: below, too many of the 256 compute
// units would idle and the tile kernel with its k-split does better
constexpr int kWideMinTiles = 192;
} // namespace

bool
gemm_wide_supported (const GemmArgs &a)
{
  if (a.wtype != 1 || a.batch > 1 || (a.K % WBK) != 0 || a.M < WBM)
    return false;
  const long tiles = (long)((a.M + WBM - 1) / WBM) * ((a.N + (a.upgate ? 63 : 127)) / (a.upgate ? 64 : 128))
                     * (a.upgate ? 1 : a.nmat);
  return tiles >= kWideMinTiles;
}

int
gemm_wide_launch (const GemmArgs &a, hipStream_t s)
{
  static bool lds_set[16] = {};
  int dev = 0;
  if (hipGetDevice (&dev) != hipSuccess || dev < 0 || dev >= 16)
    return (int)hipErrorInvalidDevice;
  if (!lds_set[dev])
    {
      VKL_HIP (hipFuncSetAttribute ((const void *)gemm_wide_f16_kernel<false>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWideLds));
      VKL_HIP (hipFuncSetAttribute ((const void *)gemm_wide_f16_kernel<true>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWideLds));
      lds_set[dev] = true;
    }
  const int tiles_m = (a.M + WBM - 1) / WBM;
  const int tiles_n = (a.N + (a.upgate ? 63 : 127)) / (a.upgate ? 64 : 128);
  const int per_xcd = (tiles_m * tiles_n + 7) / 8;
  const dim3 grid ((unsigned)(per_xcd * 8), 1, (unsigned)(a.upgate ? 1 : a.nmat));
  // 16-byte accesses to the outputs (and the residual) where their rows allow it
  int vec = (a.ys % 8) == 0 && (!a.residual || ((uintptr_t)a.residual % 16) == 0)
            && (!a.y32 || ((a.N % 4) == 0 && ((uintptr_t)a.y32 % 16) == 0));
  for (int t = 0; t < (a.upgate ? 1 : a.nmat); ++t)
    vec = vec && ((uintptr_t)a.y[t] % 16) == 0;
  if (a.upgate)
    gemm_wide_f16_kernel<true><<<grid, dim3 (WWAVES * 64), kWideLds, s>>> (a, tiles_m, tiles_n, per_xcd, vec);
  else
    gemm_wide_f16_kernel<false><<<grid, dim3 (WWAVES * 64), kWideLds, s>>> (a, tiles_m, tiles_n, per_xcd, vec);
  return (int)hipGetLastError ();
}
} // namespace vkl
