// y[M,N] = x[M,K] W[N,K]^T for many token rows (prompt passes of 128 tokens
// and more), fp16 activations and dense fp16 or planar Q8_0 weights, fp32
// accumulation on the matrix cores (v_mfma_f32_32x32x16_f16).  First the
// kernel for fp16 weights; the one for Q8_0 weights follows it.
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
#include "vkl_gemm_finish.h"

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
constexpr int WTN = WBN / 2 / 32;
constexpr int WROWB = WBK * 2;                  // bytes of a tile row


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

// Epilogue through LDS (the k loop's stages are free by then): every wave parks
// its 128 x 64 fp32 block in a region of its own, then walks it row-wise so
// that a lane handles 8 neighbouring columns: 16-byte loads and stores, whole
// cache lines per row, and a short loop instead of 128 unrolled elements.
// Accumulator register q of lane l is row 8 (q/4) + 4 (l/32) + q%4, column
// l%32 of its 32 x 32 block.
constexpr int kWideParkLd = 68; // floats per parked row: 16-byte aligned, rows 4 banks apart

template <bool UPGATE, int TM>
__device__ __forceinline__ void
wide_epilogue (const GemmArgs &a, const float16v (&acc)[TM][WTN], uint8_t *wide_lds, int wave, int lane,
               int m0, int n0, int zmat, int vec, float *part)
{
  // waves are numbered row block first: wave = 2 wm + wn, TM x 32 rows by 64 columns each
  constexpr int ROWS = TM * 32;
  const int wm = wave >> 1, wn = wave & 1;
  __builtin_amdgcn_s_barrier (); // every wave has read its last fragments
  constexpr int LD = kWideParkLd;
  float *park = (float *)(wide_lds + wave * (ROWS * LD * 4));
  {
    float *pl = park + (lane >> 5) * 4 * LD + (lane & 31);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int jn = 0; jn < WTN; ++jn)
#pragma unroll
        for (int q = 0; q < 16; ++q)
          pl[(i * 32 + (q >> 2) * 8 + (q & 3)) * LD + jn * 32] = acc[i][jn][q];
  }
  // (a wave reads back only what it wrote itself: no barrier)
  constexpr int CPR = UPGATE ? 4 : 8;   // lanes per row
  constexpr int RPI = 64 / CPR;         // rows per iteration
  const int er = lane / CPR, ec = (lane % CPR) * 8;
  const int ncol0 = n0 + (UPGATE ? wn * 32 : wn * 64) + ec;
  for (int it = 0; it < ROWS / RPI; ++it)
    {
      const int row = it * RPI + er;
      const float4 p0 = *(const float4 *)(park + row * LD + ec);
      const float4 p1 = *(const float4 *)(park + row * LD + ec + 4);
      float v[8] = { p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w };
      float g[8] = { 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f };
      if (UPGATE)
        {
          const float4 g0 = *(const float4 *)(park + row * LD + 32 + ec);
          const float4 g1 = *(const float4 *)(park + row * LD + 32 + ec + 4);
          g[0] = g0.x, g[1] = g0.y, g[2] = g0.z, g[3] = g0.w, g[4] = g1.x, g[5] = g1.y, g[6] = g1.z, g[7] = g1.w;
        }
      gemm_finish8<UPGATE> (a, v, g, m0 + wm * ROWS + row, ncol0, zmat, vec, part);
    }
}

// The same for waves in a 2 x 4 grid (TM x 32 rows by 32 columns each; of the
// fused pair the waves 0, 1 of a row block hold up, 2, 3 gate): the whole
// BM x 128 tile is parked, and after a barrier all threads walk it row-wise.
constexpr int kWideTileLd = 132;

template <int BM, bool UPGATE, int TM>
__device__ __forceinline__ void
wide_epilogue_tile (const GemmArgs &a, const float16v (&acc)[TM][1], uint8_t *wide_lds, int wave, int lane,
                    int m0, int n0, int zmat, int vec, float *part)
{
  constexpr int LD = kWideTileLd;
  const int wm = wave >> 2, wn = wave & 3;
  __builtin_amdgcn_s_barrier (); // every wave has read its last fragments
  float *park = (float *)wide_lds;
  {
    float *pl = park + (wm * TM * 32 + (lane >> 5) * 4) * LD + wn * 32 + (lane & 31);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int q = 0; q < 16; ++q)
        pl[(i * 32 + (q >> 2) * 8 + (q & 3)) * LD] = acc[i][0][q];
  }
  __syncthreads ();
  constexpr int LPR = UPGATE ? 8 : 16;        // lanes per row
  constexpr int RPI = 8 * 64 / LPR;           // rows per iteration of the workgroup
  const int er = threadIdx.x / LPR, ec = (threadIdx.x % LPR) * 8;
  for (int it = 0; it < BM / RPI; ++it)
    {
      const int row = it * RPI + er;
      const float4 p0 = *(const float4 *)(park + row * LD + ec);
      const float4 p1 = *(const float4 *)(park + row * LD + ec + 4);
      float v[8] = { p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w };
      float g[8] = { 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f };
      if (UPGATE)
        {
          const float4 g0 = *(const float4 *)(park + row * LD + 64 + ec);
          const float4 g1 = *(const float4 *)(park + row * LD + 64 + ec + 4);
          g[0] = g0.x, g[1] = g0.y, g[2] = g0.z, g[3] = g0.w, g[4] = g1.x, g[5] = g1.y, g[6] = g1.z, g[7] = g1.w;
        }
      gemm_finish8<UPGATE> (a, v, g, m0 + row, n0 + ec, zmat, vec, part);
    }
}

template <int BM>
constexpr size_t
wide_lds_f16 ()
{
  const size_t stages = (size_t)WSTAGES * (BM + WBN) * WROWB, park = (size_t)BM * 2 * kWideParkLd * 4;
  return stages > park ? stages : park;
}

// BM: token rows of a tile, 256 or (where 256-row tiles would be too few to
// occupy the compute units) 128, i.e. 64 x 64 per wave.
template <int BM, bool UPGATE>
__global__ __launch_bounds__ (WWAVES * 64) void
gemm_wide_f16_kernel (const GemmArgs a, int tiles_m, int tiles_n, int per_xcd, int vec, int ksplit, float *ws)
{
  constexpr int TM = BM / 2 / 32;                    // 32-row accumulators per wave
  constexpr int STAGE_BYTES = (BM + WBN) * WROWB;
  constexpr int GPW = (BM + WBN) / 8 / WWAVES;       // 1 KiB load instructions per wave and k-step
  constexpr int AG = BM / 8 / WWAVES;                // of which rows of x
  extern __shared__ __align__ (16) uint8_t wide_lds[];
  // workgroups go to the XCDs in turn: each XCD gets a contiguous range of
  // tiles, token-row tile fastest, so the weight tiles it shares stay in its L2
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int tile = xcd * per_xcd + j;
  // ksplit > 1: the k range is divided among ksplit workgroups per output
  // tile; each writes its fp32 sums to the workspace, a second kernel adds them
  const int plane = tiles_m * tiles_n;
  if (j >= per_xcd || tile >= plane * ksplit)
    return;
  const int ks = tile / plane, t2 = tile - ks * plane;
  const int tn = t2 / tiles_m, tm = t2 - tn * tiles_m;
  const int nk_all = a.K / WBK;
  const int kbase = (int)((long)nk_all * ks / ksplit);
  const int nk = (int)((long)nk_all * (ks + 1) / ksplit) - kbase; // k-steps of this workgroup
  float *part = ksplit > 1 ? ws + (size_t)ks * a.M * a.N : nullptr;
  const int bn_rows = UPGATE ? WBN / 2 : WBN; // weight rows per matrix and tile
  const int m0 = tm * BM, n0 = tn * bn_rows;
  const int zmat = blockIdx.z;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane (threadIdx.x >> 6);
  const int wm = wave >> 1, wn = wave & 1;

  // Load addresses.  Instruction i of a wave covers tile rows 8g .. 8g+7 with
  // g = wave + 4 i (x for i < AG, then W); lane l fetches row 8g + l/8, and
  // LDS slot l%8 of that row receives chunk (l%8) ^ f(row), f(row) = (row & 7)
  // ^ ((row >> 3) & 1): 8 or 16 consecutive rows then hit different banks at
  // the same chunk.  Rows beyond M or N repeat the last row (never stored).
  const int lr = lane >> 3;
  const int chunk = (lane & 7) ^ lr ^ (wave & 1);
  const uint16_t *src[GPW];
#pragma unroll
  for (int i = 0; i < AG; ++i)
    {
      const int m = min (m0 + (wave + WWAVES * i) * 8 + lr, a.M - 1);
      src[i] = a.x + (size_t)m * a.xs + chunk * 8 + (size_t)kbase * WBK;
    }
#pragma unroll
  for (int i = AG; i < GPW; ++i)
    {
      const int v = (wave + WWAVES * (i - AG)) * 8 + lr; // row of the weight tile
      const int mat = UPGATE ? v >> 6 : zmat;
      const int n = min (UPGATE ? n0 + (v & 63) : n0 + v, a.N - 1);
      const uint16_t *w = mat == 0 ? a.wh[0] : (mat == 1 ? a.wh[1] : a.wh[2]);
      src[i] = w + (size_t)n * a.ws + chunk * 8 + (size_t)kbase * WBK;
    }

  // fragment reads: lane l holds row l%32 of a 32-row block, k = 16 ks + 8 (l/32) .. +7
  const int fsw = (lane & 7) ^ ((lane >> 3) & 1);
  uint32_t aoff[4], boff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
    {
      const int ko = ((2 * ks + (lane >> 5)) ^ fsw) << 4;
      aoff[ks] = (wm * (BM / 2) + (lane & 31)) * WROWB + ko;
      boff[ks] = BM * WROWB + ((UPGATE ? wn * 32 : wn * 64) + (lane & 31)) * WROWB + ko;
    }
  constexpr int BJ = (UPGATE ? 64 : 32) * WROWB; // from a wave's first to its second column block

  float16v acc[TM][WTN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int jn = 0; jn < WTN; ++jn)
#pragma unroll
      for (int q = 0; q < 16; ++q)
        acc[i][jn][q] = 0.f;

  auto issue_part = [&] (int kt, int st, int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
      {
        const int g = i < AG ? wave + WWAVES * i : BM / 8 + wave + WWAVES * (i - AG);
        __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)(src[i] + (size_t)kt * WBK),
                                          (VKL_LDS void *)(wide_lds + st * STAGE_BYTES + g * 1024), 16, 0, 0);
      }
  };
#pragma unroll
  for (int p = 0; p < WSTAGES - 1; ++p)
    issue_part (p < nk ? p : nk - 1, p, 0, GPW);

  half8 af[2][TM], bf[2][WTN];
  // in the order the products need them
  auto read_frags = [&] (int st, int ks, int buf) {
    const uint8_t *sb = wide_lds + st * STAGE_BYTES;
    af[buf][0] = *(const half8 *)(sb + aoff[ks]);
#pragma unroll
    for (int jn = 0; jn < WTN; ++jn)
      bf[buf][jn] = *(const half8 *)(sb + boff[ks] + jn * BJ);
#pragma unroll
    for (int i = 1; i < TM; ++i)
      af[buf][i] = *(const half8 *)(sb + aoff[ks] + i * 32 * WROWB);
  };
  // s_waitcnt immediates: vmcnt = the loads of the newest k-step may stay in
  // flight; the second one also waits for the wave's own LDS reads
  constexpr int VMW = (WSTAGES - 2) * GPW;
  constexpr int WAITVM = 0x0f70 | (VMW & 15) | ((VMW >> 4) << 14);
  constexpr int LB1 = GPW / 3, LB2 = 2 * GPW / 3;
  constexpr int NR = TM + WTN, NP = TM * WTN;
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
            issue_part (kn, SN, ks == 0 ? 0 : ks == 1 ? LB1 : LB2, ks == 0 ? LB1 : ks == 1 ? LB2 : GPW);
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
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int jn = 0; jn < WTN; ++jn)
            acc[i][jn] = __builtin_amdgcn_mfma_f32_32x32x16_f16 (af[ks & 1][i], bf[ks & 1][jn], acc[i][jn], 0, 0, 0);
        if (ks == 0)
          WideOrder<0, NP, NR, LB1>::run ();
        else if (ks == 1)
          WideOrder<0, NP, NR, LB2 - LB1>::run ();
        else if (ks == 2)
          WideOrder<0, NP, NR, GPW - LB2>::run ();
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

  wide_epilogue<UPGATE, TM> (a, acc, wide_lds, wave, lane, m0, n0, zmat, vec, part);
}

// ---------------------------------------------------------------------------
// planar Q8_0 weights
// ---------------------------------------------------------------------------
// Same tile, same staging.  The weight tile enters LDS as it lies in memory:
// 128 rows x 64 int8 (8 KiB, 16-byte chunks swizzled by (row >> 1) & 3) plus
// the two fp16 block scales of every row.  A wave converts the int8 fragments
// it reads to fp16 (exact integers) in registers, sums each block of 32 on the
// matrix core from a zero accumulator and applies the block's scale in fp32
// (acc = fma (part, d, acc)): the arithmetic of the tile kernel and of the
// reference shader.  That scaling costs as many vector-ALU cycles as the
// products cost matrix-core cycles, and it wants the block sums in ordinary
// registers: a workgroup is therefore EIGHT waves (two per SIMD, at most 256
// registers each, where the compiler keeps MFMA results out of the
// accumulation registers).  The unit of the schedule is a block (two MFMA
// k-slices): while block b is multiplied, the fragments of block b + 1 are
// read.  (LDS reads must not go through HIP's uint2/uint4 struct types here:
// the compiler takes reads of a struct type to alias the tiles that the
// direct-to-LDS loads still have in flight and waits for all of them.)
constexpr int QWAVES = 8;
// waves along N: 4 (2 x 4 waves, 128 x 32 each) measured 5-12 % faster than 2
// (4 x 2 waves, 64 x 64 each) on the 7B and 13B shapes
constexpr int QGRID = 4;
// Three stages, laid out by kind (x tiles, then quants, then scales).
constexpr int QSTAGES = 3;
constexpr int QB_BYTES = WBN * WBK;
constexpr int QS_BYTES = WBN * 4; // two fp16 scales per row

template <int BM>
constexpr size_t
wide_lds_q8 ()
{
  const size_t stages = (size_t)QSTAGES * (BM * WROWB + QB_BYTES + QS_BYTES), park = (size_t)BM * 2 * kWideParkLd * 4; // (>= BM * kWideTileLd * 4)
  return stages > park ? stages : park;
}

// (a vector type, not HIP's uint2 struct: LDS reads of the struct type are
// taken to alias the tiles in flight and made to wait for all of them)
typedef uint32_t u32x2 __attribute__ ((ext_vector_type (2)));

__device__ __forceinline__ half8
q8_frag (u32x2 r)
{
  h16x2 a, b, c, d;
  i8x4_to_h2x2 (r.x, a, b);
  i8x4_to_h2x2 (r.y, c, d);
  half8 o;
  o[0] = a[0], o[1] = a[1], o[2] = b[0], o[3] = b[1];
  o[4] = c[0], o[5] = c[1], o[6] = d[0], o[7] = d[1];
  return o;
}

// WGN: waves along N, 2 (4 x 2 waves of 64 columns) or 4 (2 x 4 waves of 32
// columns and twice the rows: every weight fragment is converted by two waves
// instead of four).
template <int BM, int WGN, bool UPGATE>
__global__ __launch_bounds__ (QWAVES * 64) void
gemm_wide_q8_kernel (const GemmArgs a, int tiles_m, int tiles_n, int per_xcd, int vec, int ksplit, float *ws)
{
  constexpr int QTM = BM / (QWAVES / WGN) / 32; // 32-row accumulators per wave
  constexpr int QTN = 4 / WGN;                  // 32-column accumulators per wave
  constexpr int QAG = BM / 8 / QWAVES;       // x load instructions per wave and k-step
  constexpr int QA_BYTES = BM * WROWB;
  constexpr int QB_BASE = QSTAGES * QA_BYTES;
  constexpr int QS_BASE = QB_BASE + QSTAGES * QB_BYTES;
  constexpr int QLOADS = QAG + 1 + 1;        // per wave and k-step: x, quants, scales
  extern __shared__ __align__ (16) uint8_t wide_lds[];
  const int xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  const int tile = xcd * per_xcd + j;
  // ksplit > 1: the k range is divided among ksplit workgroups per output
  // tile; each writes its fp32 sums to the workspace, a second kernel adds them
  const int plane = tiles_m * tiles_n;
  if (j >= per_xcd || tile >= plane * ksplit)
    return;
  const int ks = tile / plane, t2 = tile - ks * plane;
  const int tn = t2 / tiles_m, tm = t2 - tn * tiles_m;
  const int nk_all = a.K / WBK;
  const int kbase = (int)((long)nk_all * ks / ksplit);
  const int nk = (int)((long)nk_all * (ks + 1) / ksplit) - kbase; // k-steps of this workgroup
  float *part = ksplit > 1 ? ws + (size_t)ks * a.M * a.N : nullptr;
  const int bn_rows = UPGATE ? WBN / 2 : WBN;
  const int m0 = tm * BM, n0 = tn * bn_rows;
  const int zmat = blockIdx.z;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane (threadIdx.x >> 6);
  const int wm = wave / WGN, wn = wave % WGN;

  // load addresses: x as in the fp16 kernel, instruction i of a wave covering
  // tile rows 8 g .. 8 g + 7 with g = wave + 8 i
  const int lr = lane >> 3;
  const int chunk = (lane & 7) ^ lr ^ (wave & 1);
  const uint8_t *src[QLOADS];
#pragma unroll
  for (int i = 0; i < QAG; ++i)
    {
      const int m = min (m0 + (wave + QWAVES * i) * 8 + lr, a.M - 1);
      src[i] = (const uint8_t *)(a.x + (size_t)m * a.xs + chunk * 8 + (size_t)kbase * WBK);
    }
  // quants: a wave's one instruction covers weight-tile rows 16 wave .. + 15;
  // lane l fetches chunk (l%4) ^ ((row >> 1) & 3) of row 16 wave + l/4
  {
    const int qr = lane >> 2;
    const int v = wave * 16 + qr;
    const int mat = UPGATE ? v >> 6 : zmat;
    const int n = min (UPGATE ? n0 + (v & 63) : n0 + v, a.N - 1);
    const uint8_t *w = mat == 0 ? a.wq[0] : (mat == 1 ? a.wq[1] : a.wq[2]);
    src[QAG] = w + (size_t)n * a.Kp + ((lane & 3) ^ ((qr >> 1) & 3)) * 16 + (size_t)kbase * WBK;
  }
  // scales: the two of a row are one dword; a wave fetches rows 64 (wave & 1)
  // + lane (four waves write each half, all the same values), so that every
  // wave counts the same number of loads
  {
    const int v = (wave & 1) * 64 + lane;
    const int mat = UPGATE ? v >> 6 : zmat;
    const int n = min (UPGATE ? n0 + (v & 63) : n0 + v, a.N - 1);
    const uint16_t *ds = mat == 0 ? a.wd[0] : (mat == 1 ? a.wd[1] : a.wd[2]);
    src[QAG + 1] = (const uint8_t *)(ds + (size_t)n * (a.Kp >> 5) + (size_t)kbase * 2);
  }

  // fragment reads
  const int fsw = (lane & 7) ^ ((lane >> 3) & 1);
  // (rows of the weight tile: for the fused pair 0 .. 63 are up, 64 .. 127 gate)
  const int brow = (WGN == 4 ? wn * 32 : UPGATE ? wn * 32 : wn * 64) + (lane & 31);
  const int qsw = (lane >> 1) & 3;
  uint32_t aoff[4], qoff[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks)
    {
      aoff[ks] = (wm * (QTM * 32) + (lane & 31)) * WROWB + (((2 * ks + (lane >> 5)) ^ fsw) << 4);
      qoff[ks] = QB_BASE + brow * WBK + ((ks ^ qsw) << 4) + (lane >> 5) * 8;
    }
  const uint32_t soff = QS_BASE + brow * 4;
  constexpr int BJR = UPGATE ? 64 : 32; // rows from a wave's first to its second column block

  float16v acc[QTM][QTN];
#pragma unroll
  for (int i = 0; i < QTM; ++i)
#pragma unroll
    for (int jn = 0; jn < QTN; ++jn)
#pragma unroll
      for (int q = 0; q < 16; ++q)
        acc[i][jn][q] = 0.f;

  auto issue = [&] (int kt, int st) {
#pragma unroll
    for (int i = 0; i < QAG; ++i)
      __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)(src[i] + (size_t)kt * WROWB),
                                        (VKL_LDS void *)(wide_lds + st * QA_BYTES + (wave + QWAVES * i) * 1024), 16,
                                        0, 0);
    __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)(src[QAG] + (size_t)kt * WBK),
                                      (VKL_LDS void *)(wide_lds + QB_BASE + st * QB_BYTES + wave * 1024), 16, 0, 0);
    __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)(src[QAG + 1] + (size_t)kt * 4),
                                      (VKL_LDS void *)(wide_lds + QS_BASE + st * QS_BYTES + (wave & 1) * 256), 4,
                                      0, 0);
  };
  issue (0, 0);
  issue (nk > 1 ? 1 : 0, 1);

  half8 af[2][2][QTM];  // [block buffer][k-slice of the block][row block]
  u32x2 bq[2][2][QTN];  // weight fragments as read (int8)
  float d[2][QTN];      // the scales of the tile's two blocks
  auto read_block = [&] (int st, int blk, int buf) {
    const int sa = st * QA_BYTES, sq = st * QB_BYTES;
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2)
      {
        const int ks = 2 * blk + k2;
#pragma unroll
        for (int jn = 0; jn < QTN; ++jn)
          bq[buf][k2][jn] = *(const u32x2 *)(wide_lds + (qoff[ks] + sq) + jn * BJR * WBK);
#pragma unroll
        for (int i = 0; i < QTM; ++i)
          af[buf][k2][i] = *(const half8 *)(wide_lds + (aoff[ks] + sa) + i * 32 * WROWB);
      }
  };
  auto read_scales = [&] (int st) {
#pragma unroll
    for (int jn = 0; jn < QTN; ++jn)
      {
        const uint32_t sc = *(const uint32_t *)(wide_lds + (soff + st * QS_BYTES) + jn * BJR * 4);
        d[0][jn] = h2f ((uint16_t)(sc & 0xffff));
        d[1][jn] = h2f ((uint16_t)(sc >> 16));
        // (keeps the conversion out of the scaling products: as fp16 operands
        // they would become mixed-precision FMAs)
        asm volatile ("" : "+v"(d[0][jn]), "+v"(d[1][jn]));
      }
  };
  // The wave's four 32 x 32 blocks in turn, written so that the two MFMAs of one
  // stand before the sixteen scaling FMAs of the one before; the order within
  // a block is left to the compiler (pinned with scheduling barriers it ran
  // 7 % slower).
  auto multiply = [&] (int buf, const float (&dd)[QTN]) {
    half8 bfc[2][QTN];
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
      for (int jn = 0; jn < QTN; ++jn)
        bfc[k2][jn] = q8_frag (bq[buf][k2][jn]);
    float16v part[2];
#pragma unroll
    for (int p = 0; p <= QTM * QTN; ++p)
      {
        if (p < QTM * QTN)
          {
            const int i = p / QTN, jn = p % QTN;
            float16v z;
#pragma unroll
            for (int e = 0; e < 16; ++e)
              z[e] = 0.f;
            z = __builtin_amdgcn_mfma_f32_32x32x16_f16 (af[buf][0][i], bfc[0][jn], z, 0, 0, 0);
            part[p & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16 (af[buf][1][i], bfc[1][jn], z, 0, 0, 0);
          }
        if (p > 0)
          {
            const int i = (p - 1) / QTN, jn = (p - 1) % QTN;
#pragma unroll
            for (int e = 0; e < 16; ++e)
              acc[i][jn][e] = __builtin_fmaf (part[(p - 1) & 1][e], dd[jn], acc[i][jn][e]);
          }
      }
  };
  // s_waitcnt: the loads of the newest tile may stay in flight; the one in the
  // loop also waits for the wave's own LDS reads
  constexpr int WAITVM = 0x0f70 | (QLOADS & 15) | ((QLOADS >> 4) << 14);
  __builtin_amdgcn_s_waitcnt (WAITVM);
  __builtin_amdgcn_s_barrier ();
  issue (nk > 2 ? 2 : nk - 1, 2);
  read_block (0, 0, 0);
  read_scales (0);
  __builtin_amdgcn_sched_barrier (0);
  // One k-step per turn.  On entry the fragments of block 0 of tile kt (stage
  // st = kt % 3) are in buffer 0, the scales of both its blocks in d, and the
  // loads of tiles kt + 1 and kt + 2 are in flight or done.  (One copy of the
  // step with the stage as a variable: unrolled by the stages, the
  // accumulators wander between sets of registers and the kernel spills.)
  int st = 0;
  for (int kt = 0; kt < nk; ++kt)
    {
      const int s1 = st == QSTAGES - 1 ? 0 : st + 1;
      float d1[QTN];
#pragma unroll
      for (int jn = 0; jn < QTN; ++jn)
        d1[jn] = d[1][jn];
      read_block (st, 1, 1);
      multiply (0, d[0]);
      __builtin_amdgcn_sched_barrier (0);
      // tile kt + 1 has landed (this wave's part; the barrier covers the
      // others') and this wave has read the last of tile kt: its stage takes
      // tile kt + 3 (past the end the last tile again, which nothing reads)
      __builtin_amdgcn_s_waitcnt (WAITVM & ~0x0f00);
      __builtin_amdgcn_s_barrier ();
      __builtin_amdgcn_sched_barrier (0);
      issue (kt + 3 < nk ? kt + 3 : nk - 1, st);
      read_block (s1, 0, 0);
      read_scales (s1);
      multiply (1, d1);
      __builtin_amdgcn_sched_barrier (0);
      st = s1;
    }
  __builtin_amdgcn_s_waitcnt (0x0f70); // no load may outlive the workgroup's LDS
  if constexpr (WGN == 4)
    wide_epilogue_tile<BM, UPGATE, QTM> (a, acc, wide_lds, wave, lane, m0, n0, zmat, vec, part);
  else
    wide_epilogue<UPGATE, QTM> (a, acc, wide_lds, wave, lane, m0, n0, zmat, vec, part);
}

// Which tile height and how many parts of the k range: the pair with the
// lowest estimated time, from a model fitted to measurements on the 7B shapes
// (microseconds: a round of 256-row tiles over the 256 compute units takes
// about 0.95 per k-step + 8, one of 128-row tiles 0.55 per k-step + 6; with Q8_0
// weights 1.35 and 0.90 per k-step, fitted on the 13B shapes at 3968 rows as
// well: every tile converts its weight fragments anew, so short tiles gain
// less there; a reduction launch 5 + its bytes at 2.5 TB/s).
// Below kWideMinGroups workgroups the tile kernel of vkl_gemm_mfma.hip does
// better.
constexpr int kWideMinRows = 128;
// From 65 rows on (where the tile kernel needs a second row of 64-row tiles) in
// one partly empty row of 128-row tiles: fp16 weights, the fused up/gate pair,
// and Q8_0 products with K up to 5120.  Measured at 80-127 rows: fp16 4096^2
// 20-23 -> 16-17 us, 12288 x 4096 41-43 -> 35-39, up/gate 62-67 -> 47-50 (13B
// 89-97 -> 65-70), down even; Q8_0 up/gate 84 -> 66 (13B 108 -> 92), 4096^2
// 27 -> 24.  Not the Q8_0 down product (K = 11008: 39 -> 42 us), and nothing
// below 65 rows (13B Q8_0 up/gate at 64 rows: 83 against 88 us).
constexpr int kWideMinRowsPartial = 65;
constexpr int kWideMinGroups = 88, kWideMinGroupsQ8 = 128;

struct WidePlan
{
  int bm;     // token rows of a tile, 0: this form does not apply
  int ksplit; // parts of the k range
};

long
wide_tiles (const GemmArgs &a, int bm)
{
  return (long)((a.M + bm - 1) / bm) * ((a.N + (a.upgate ? 63 : 127)) / (a.upgate ? 64 : 128))
         * (a.upgate ? 1 : a.nmat);
}

WidePlan
wide_plan (const GemmArgs &a)
{
  WidePlan none = { 0, 1 }, best = none;
  const int min_rows = a.wtype == 1 || a.upgate || a.K <= 5120 ? kWideMinRowsPartial : kWideMinRows;
  if ((a.wtype != 1 && a.wtype != 8) || a.batch > 1 || (a.K % WBK) != 0 || a.M < min_rows)
    return none;
  if (a.wtype == 8)
    {
      // whole k-steps of quants and scale pairs, aligned for 16- and 4-byte loads
      if (a.Kp != a.K)
        return none;
      for (int t = 0; t < (a.upgate ? 2 : a.nmat); ++t)
        if (((uintptr_t)a.wq[t] % 16) != 0 || ((uintptr_t)a.wd[t] % 4) != 0)
          return none;
    }
  const int nk = a.K / WBK;
  const size_t ws_bytes = a.workspace ? a.workspace_bytes : gemm_stream_workspace_bytes ();
  double best_cost = 0;
  for (int bm = 128; bm <= WBM; bm *= 2)
    for (int ks = 1; ks <= 4; ks *= 2)
      {
        // (a single row of 128-row tiles may be partly empty)
        if (a.M < bm && !(bm == 128 && a.M >= min_rows))
          continue;
        // parts only for one matrix with the plain epilogue, of at least 16
        // k-steps each, and as far as the scratch holds them
        if (ks > 1
            && (a.upgate || a.nmat != 1 || nk / ks < 16 || (size_t)ks * a.M * a.N * sizeof (float) > ws_bytes))
          continue;
        const long groups = wide_tiles (a, bm) * ks;
        if (groups < (a.wtype == 8 ? kWideMinGroupsQ8 : kWideMinGroups))
          continue;
        const double per_step = a.wtype == 8 ? (bm == WBM ? 1.35 : 0.90) : (bm == WBM ? 0.95 : 0.55);
        const double round = per_step * nk / ks + (bm == WBM ? 8 : 6);
        const double reduce = ks > 1 ? 5 + (double)ks * a.M * a.N * sizeof (float) / 2.5e6 : 0;
        const double cost = (double)((groups + 255) / 256) * round + reduce;
        if (!best.bm || cost < best_cost)
          best = { bm, ks }, best_cost = cost;
      }
  return best;
}
} // namespace

bool
gemm_wide_supported (const GemmArgs &a)
{
  return wide_plan (a).bm != 0;
}

void
gemm_wide_choice (const GemmArgs &a, int *tile_rows, int *ksplit)
{
  const WidePlan p = wide_plan (a);
  *tile_rows = p.bm, *ksplit = p.bm ? p.ksplit : 1;
}

size_t
gemm_wide_workspace_bytes (const GemmArgs &a)
{
  const WidePlan p = wide_plan (a);
  return p.bm && p.ksplit > 1 ? (size_t)p.ksplit * a.M * a.N * sizeof (float) : 0;
}

int
gemm_wide_launch (const GemmArgs &a, hipStream_t s)
{
  constexpr size_t lds256 = wide_lds_f16<256> (), lds128 = wide_lds_f16<128> ();
  constexpr size_t q256 = wide_lds_q8<256> (), q128 = wide_lds_q8<128> ();
  static LdsLimit limits[8];
  const void *const kernels[8]
      = { (const void *)gemm_wide_f16_kernel<256, false>,       (const void *)gemm_wide_f16_kernel<256, true>,
          (const void *)gemm_wide_f16_kernel<128, false>,       (const void *)gemm_wide_f16_kernel<128, true>,
          (const void *)gemm_wide_q8_kernel<256, QGRID, false>, (const void *)gemm_wide_q8_kernel<256, QGRID, true>,
          (const void *)gemm_wide_q8_kernel<128, QGRID, false>, (const void *)gemm_wide_q8_kernel<128, QGRID, true> };
  const size_t need[8] = { lds256, lds256, lds128, lds128, q256, q256, q128, q128 };
  for (int i = 0; i < 8; ++i)
    if (int e = limits[i].raise (kernels[i], need[i]))
      return e;
  const WidePlan plan = wide_plan (a);
  const int bm = plan.bm;
  int ksplit = plan.ksplit;
  if (!bm)
    return (int)hipErrorInvalidValue;
  float *ws = nullptr;
  if (ksplit > 1 && !(ws = a.workspace ? a.workspace : gemm_stream_workspace (s)))
    ksplit = 1;
  const int tiles_m = (a.M + bm - 1) / bm;
  const int tiles_n = (a.N + (a.upgate ? 63 : 127)) / (a.upgate ? 64 : 128);
  const int per_xcd = (tiles_m * tiles_n * ksplit + 7) / 8;
  const dim3 grid ((unsigned)(per_xcd * 8), 1, (unsigned)(a.upgate ? 1 : a.nmat));
  const dim3 block ((a.wtype == 8 ? QWAVES : WWAVES) * 64);
  // 16-byte accesses to the outputs (and the residual) where their rows allow it
  int vec = (a.ys % 8) == 0 && (!a.residual || ((uintptr_t)a.residual % 16) == 0)
            && (!a.y32 || ((a.N % 4) == 0 && ((uintptr_t)a.y32 % 16) == 0));
  for (int t = 0; t < (a.upgate ? 1 : a.nmat); ++t)
    vec = vec && ((uintptr_t)a.y[t] % 16) == 0;
  if (a.wtype == 8 && bm == 256)
    {
      if (a.upgate)
        gemm_wide_q8_kernel<256, QGRID, true><<<grid, block, q256, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
      else
        gemm_wide_q8_kernel<256, QGRID, false><<<grid, block, q256, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
    }
  else if (a.wtype == 8)
    {
      if (a.upgate)
        gemm_wide_q8_kernel<128, QGRID, true><<<grid, block, q128, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
      else
        gemm_wide_q8_kernel<128, QGRID, false><<<grid, block, q128, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
    }
  else if (bm == 256)
    {
      if (a.upgate)
        gemm_wide_f16_kernel<256, true><<<grid, block, lds256, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
      else
        gemm_wide_f16_kernel<256, false><<<grid, block, lds256, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
    }
  else if (a.upgate)
    gemm_wide_f16_kernel<128, true><<<grid, block, lds128, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
  else
    gemm_wide_f16_kernel<128, false><<<grid, block, lds128, s>>> (a, tiles_m, tiles_n, per_xcd, vec, ksplit, ws);
  if (ksplit > 1)
    return gemm_reduce_parts (a, ws, ksplit, a.M, s);
  return (int)hipGetLastError ();
}
} // namespace vkl
