// The weight pipeline shared by the decode-step translation units: the staged
// activation row (with the RMSNorm folded in), and the register pipeline that
// streams the rows of a projection (Gemv).
#ifndef VKL_DECODE_GEMV_H
#define VKL_DECODE_GEMV_H
#include "vkl_decode_shared.h"

namespace vkl
{
namespace dec
{
namespace
{
// The activation row (K fp16 values, K a multiple of 32, K <= 16384) is
// fetched into registers first: thread t holds the 8-element chunks t,
// t+512, t+1024, t+1536.  Issued before any weight load, these are the oldest
// vector-memory operations of the wave, so they return first (loads return in
// order) while the weight prefetch issued right after them is still in
// flight.
struct XRegs
{
  uint4 v[4];
};

struct NormRegs
{
  uint4 w[4][2]; // 8 fp32 weights per chunk
};

__device__ __forceinline__ void
issue_x (const uint16_t *src, int K, XRegs &x)
{
#pragma unroll
  for (int j = 0; j < 4; ++j)
    {
      const int idx = threadIdx.x + j * kDecThreads;
      x.v[j] = make_uint4 (0, 0, 0, 0);
      if (idx * 8 < K)
        x.v[j] = ldg4 (src + idx * 8);
    }
}

// one row of a planar Q8_0 table: the 8 quants of each chunk land in v[j].x/.y
// and the block scale in v[j].z; dequant_embed turns them into fp16
__device__ __forceinline__ void
issue_embed_q8 (const QMat tab, size_t row, int K, XRegs &x)
{
#pragma unroll
  for (int j = 0; j < 4; ++j)
    {
      const int idx = threadIdx.x + j * kDecThreads;
      x.v[j] = make_uint4 (0, 0, 0, 0);
      if (idx * 8 < K)
        {
          const unsigned long long q
              = ldg ((const unsigned long long *)(tab.q + row * K + idx * 8));
          x.v[j].x = (uint32_t)q, x.v[j].y = (uint32_t)(q >> 32);
          x.v[j].z = ldg (tab.d + row * (K >> 5) + (idx >> 2));
        }
    }
}

// fp16(float(q) * float(d)), the embedding lookup's arithmetic
__device__ __forceinline__ void
dequant_embed (XRegs &x)
{
#pragma unroll
  for (int j = 0; j < 4; ++j)
    {
      const float sc = h2f ((uint16_t)x.v[j].z);
      const uint32_t w[2] = { x.v[j].x, x.v[j].y };
      uint32_t o[4];
#pragma unroll
      for (int i = 0; i < 4; ++i)
        {
          const int8_t b0 = (int8_t)((w[i >> 1] >> (16 * (i & 1))) & 0xff);
          const int8_t b1 = (int8_t)((w[i >> 1] >> (16 * (i & 1) + 8)) & 0xff);
          o[i] = (uint32_t)f2h ((float)b0 * sc)
                 | ((uint32_t)f2h ((float)b1 * sc) << 16);
        }
      x.v[j] = make_uint4 (o[0], o[1], o[2], o[3]);
    }
}

__device__ __forceinline__ void
issue_norm (const float *w, int K, NormRegs &n)
{
#pragma unroll
  for (int j = 0; j < 4; ++j)
    {
      const int idx = threadIdx.x + j * kDecThreads;
      n.w[j][0] = n.w[j][1] = make_uint4 (0, 0, 0, 0);
      if (idx * 8 < K)
        {
          n.w[j][0] = ldg4 (w + idx * 8);
          n.w[j][1] = ldg4 (w + idx * 8 + 4);
        }
    }
}

// Writes the row to LDS as fp16; with `n` it is RMS-normalised on the way:
// y = fp16(x * w * (1 / sqrt(mean(x^2) + eps))).  Ends with a barrier.
template <bool NORM>
__device__ __forceinline__ void
finish_x (const XRegs &x, int K, uint16_t *xl, const NormRegs &n, float eps,
          float *red, unsigned long long *tr = nullptr)
{
  float alpha = 0.f;
#ifdef VKL_TRACE
  if (tr && threadIdx.x == 0)
    {
      // x has arrived once its first word can be read
      asm volatile("" ::"v"(x.v[0].x), "v"(x.v[3].w));
      tr[1] = wall_clock64 ();
    }
#endif
  if (NORM)
    {
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        {
          const bool in = (int)(threadIdx.x + j * kDecThreads) * 8 < K;
          const uint32_t w[4] = { x.v[j].x, x.v[j].y, x.v[j].z, x.v[j].w };
#pragma unroll
          for (int i = 0; i < 4; ++i)
            {
              const float a = in ? h2f ((uint16_t)(w[i] & 0xffff)) : 0.f;
              const float b = in ? h2f ((uint16_t)(w[i] >> 16)) : 0.f;
              s += a * a;
              s += b * b;
            }
        }
      const float total = block_sum (s, red);
#ifdef VKL_TRACE
      if (tr && threadIdx.x == 0)
        tr[3] = wall_clock64 ();
#endif
      alpha = 1.0f / sqrtf (total / (float)K + eps);
    }
#pragma unroll
  for (int j = 0; j < 4; ++j)
    {
      const int idx = threadIdx.x + j * kDecThreads;
      if (idx * 8 >= K)
        continue;
      uint4 o = x.v[j];
      if (NORM)
        {
          const uint32_t w[4] = { x.v[j].x, x.v[j].y, x.v[j].z, x.v[j].w };
          const uint4 g0 = n.w[j][0], g1 = n.w[j][1];
          const uint32_t g[8] = { g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w };
          uint32_t r[4];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            {
              const float a = h2f ((uint16_t)(w[i] & 0xffff));
              const float b = h2f ((uint16_t)(w[i] >> 16));
              r[i] = (uint32_t)f2h (a * __uint_as_float (g[2 * i]) * alpha)
                     | ((uint32_t)f2h (b * __uint_as_float (g[2 * i + 1]) * alpha) << 16);
            }
          o = make_uint4 (r[0], r[1], r[2], r[3]);
        }
      ((uint4 *)xl)[idx] = o;
    }
  __syncthreads ();
}

// ---- the same without a branch -------------------------------------------------
// The helpers above put every load under `if (idx * 8 < K)`.  With branches
// between the first load and the first use of the row the compiler cannot
// count the loads in flight, and the wait for the row becomes a wait for
// everything requested so far: the first weight item, on its way from HBM,
// stands between the row and its normalisation.  Here the number of
// 4096-element chunks of the row is a compile-time constant XCH, every load is
// unconditional from a clamped address, and a thread whose chunk lies past K
// computes and stores a duplicate of the last chunk (same address, same value).
template <int XCH>
__device__ __forceinline__ void
load_row (const uint16_t *src, int K, XRegs &x)
{
#pragma unroll
  for (int j = 0; j < XCH; ++j)
    {
      const int idx = min ((int)threadIdx.x + j * kDecThreads, (K >> 3) - 1);
      x.v[j] = ldg4 (src + idx * 8);
    }
}

template <int XCH>
__device__ __forceinline__ void
load_norm (const float *w, int K, NormRegs &n)
{
#pragma unroll
  for (int j = 0; j < XCH; ++j)
    {
      const int idx = min ((int)threadIdx.x + j * kDecThreads, (K >> 3) - 1);
      n.w[j][0] = ldg4 (w + idx * 8);
      n.w[j][1] = ldg4 (w + idx * 8 + 4);
    }
}

template <bool NORM, int XCH>
__device__ __forceinline__ void
stage_row (const XRegs &x, int K, uint16_t *xl, const NormRegs &n, float eps,
           float *red, unsigned long long *tr = nullptr)
{
  float alpha = 0.f;
#ifdef VKL_TRACE
  if (tr && threadIdx.x == 0)
    {
      asm volatile("" ::"v"(x.v[0].x), "v"(x.v[XCH - 1].w));
      tr[1] = wall_clock64 ();
    }
#endif
  if (NORM)
    {
      float s = 0.f;
#pragma unroll
      for (int j = 0; j < XCH; ++j)
        {
          const bool in = (int)(threadIdx.x + j * kDecThreads) * 8 < K;
          const uint32_t w[4] = { x.v[j].x, x.v[j].y, x.v[j].z, x.v[j].w };
#pragma unroll
          for (int i = 0; i < 4; ++i)
            {
              const float a = in ? h2f ((uint16_t)(w[i] & 0xffff)) : 0.f;
              const float b = in ? h2f ((uint16_t)(w[i] >> 16)) : 0.f;
              s += a * a;
              s += b * b;
            }
        }
      const float total = block_sum (s, red);
#ifdef VKL_TRACE
      if (tr && threadIdx.x == 0)
        tr[3] = wall_clock64 ();
#endif
      alpha = 1.0f / sqrtf (total / (float)K + eps);
    }
#pragma unroll
  for (int j = 0; j < XCH; ++j)
    {
      const int idx = min ((int)threadIdx.x + j * kDecThreads, (K >> 3) - 1);
      uint4 o = x.v[j];
      if (NORM)
        {
          const uint32_t w[4] = { x.v[j].x, x.v[j].y, x.v[j].z, x.v[j].w };
          const uint4 g0 = n.w[j][0], g1 = n.w[j][1];
          const uint32_t g[8] = { g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w };
          uint32_t r[4];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            {
              const float a = h2f ((uint16_t)(w[i] & 0xffff));
              const float b = h2f ((uint16_t)(w[i] >> 16));
              r[i] = (uint32_t)f2h (a * __uint_as_float (g[2 * i]) * alpha)
                     | ((uint32_t)f2h (b * __uint_as_float (g[2 * i + 1]) * alpha) << 16);
            }
          o = make_uint4 (r[0], r[1], r[2], r[3]);
        }
      ((uint4 *)xl)[idx] = o;
    }
  __syncthreads ();
}

// ---------------------------------------------------------------------------
// projections
// ---------------------------------------------------------------------------
struct Epilogue
{
  uint16_t *y[3];           // outputs (MODE 1 uses three)
  const uint16_t *residual; // MODE 0: y = fp16(fp16(v) + residual) if set
  float *y32;               // MODE 0: widened copy if set
  float *amax_val;          // MODE 0: per-workgroup arg-max partials if set
  uint32_t *amax_idx;
  bool through;             // results are stored through to memory: other
                            // workgroups of this launch read them
};

__device__ __forceinline__ void
st_h (const Epilogue &e, uint16_t *p, uint16_t v)
{
  if (e.through)
    __hip_atomic_store (p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  else
    stg (p, v);
}

__device__ __forceinline__ void
st_h2 (const Epilogue &e, uint32_t *p, uint32_t v)
{
  if (e.through)
    st_coherent_u32 (p, v);
  else
    stg (p, v);
}

// How the units of a product are dealt to the workgroups.  Plain: workgroup
// g of G takes the g-th of G contiguous shares.  Owned: the workgroups that
// run on one XCD share an L2; the output row is cut into 128-byte lines (`upl`
// units each), XCD `slot` takes the slot-th of eight contiguous runs of whole
// lines and deals its units to its `n` workgroups (this one is number `idx`
// among them), so that every line of the output is written through ONE L2
// only.  A row handed over inside a launch can then be read with ordinary
// loads once its writers have counted in: an L2 either never saw a line (and
// fetches it from memory, where the written-through values are) or saw every
// write to it.
struct Deal
{
  int own; // 0: plain
  int slot, idx, n;
};

__device__ __forceinline__ void
dealt_units (const Deal dl, int U, int upl, int wg, int G, int &lo, int &hi)
{
  if (!dl.own)
    {
      lo = (int)((unsigned)U * (unsigned)wg / (unsigned)G);
      hi = (int)((unsigned)U * (unsigned)(wg + 1) / (unsigned)G);
      return;
    }
  const int k = dl.slot;
  const int nl = (U + upl - 1) / upl;
  const int a = min (U, upl * (nl * k / 8)), b = min (U, upl * (nl * (k + 1) / 8));
  lo = hi = 0;
  if (dl.idx < 0 || dl.idx >= dl.n)
    return;
  lo = a + (int)((unsigned)(b - a) * (unsigned)dl.idx / (unsigned)dl.n);
  hi = a + (int)((unsigned)(b - a) * (unsigned)(dl.idx + 1) / (unsigned)dl.n);
}

// The pipeline's registers: two item buffers shared by every projection phase
// (each item is 8 dwordx4 weight loads and 8 scales per lane), and the small
// state of the phase in progress.  Keeping ONE pair of buffers for all phases
// matters in the persistent kernel, where a phase's first items are issued
// while the previous phase is still being finished.
// weight matrix view: planar Q8_0 (quants + scales) or dense fp16 (bytes)
template <int WT>
__device__ __forceinline__ QMat
wmat (const void *w, int N, int K)
{
  if (WT == 8)
    return qmat (w, N, K);
  return QMat{ (const uint8_t *)w, (const uint16_t *)w };
}

struct PipeState
{
  // MODE 1 reaches its second and third matrix through byte offsets from the
  // first: selecting among pointers held here by a runtime index would force
  // the whole pipeline state out of registers into scratch
  QMat m0;
  long long dq1, dq2, dd1, dd2;
  int mode, N, Kp, nb, nch;
  int lane, wave, wg;
  int u_lo, nit, primed;
  int U; // units of the whole product
  float best_v;
  uint32_t best_i;
  const uint16_t *residual; // mode 0: fetched with each item, see issue ()
};

// mode 0: y = x W^T (+ residual); a unit is 2 consecutive rows of m0
// mode 1: three matrices with three outputs; a unit is 2 rows of one of them
// mode 2: y = silu(x Wgate^T) * (x Wup^T); a unit is row r of m0 (up) and
//         row r of m1 (gate)
// One copy of the code serves all three (the mode only steers the cheap row
// addressing and the lane-0 epilogue).
// WT: 8 = planar Q8_0 weights, 1 = dense fp16 weights.  For fp16 a row is
// addressed as 2*K bytes, so the 16-byte loads of an item are laid out exactly
// as for the int8 plane; only the scale load and the dot product differ.
// NT: the weights are read with the non-temporal hint (a stream read once)
// RU: rows per unit, 2, or 1 (mode 0 only): a product with long rows and few
// of them then has a unit for every wave and both of its items in flight
// from the start.  An item is always 8 loads of 16 bytes per lane: RU rows x
// 8 / RU k-steps of 1024.
template <int WT = 8, bool NT = false, int RU = 2> struct Gemv
{
  static constexpr int R = RU;     // rows per unit
  static constexpr int S = 8 / RU; // k-steps of 1024 per item
  static constexpr int CHUNK = S * VKL_WAVE * 16;

  static __device__ __forceinline__ void
  rows_of (const PipeState &ps, int u, const uint8_t *(&q)[R],
           const uint16_t *(&d)[R])
  {
    const int Kp = ps.Kp, nb = ps.nb;
    if (R == 1)
      q[0] = ps.m0.q + (size_t)u * Kp, d[0] = ps.m0.d + (size_t)u * nb;
    else if (ps.mode == 0)
      {
        const int r0 = 2 * u;
        const int r1 = min (r0 + 1, ps.N - 1);
        q[0] = ps.m0.q + (size_t)r0 * Kp, d[0] = ps.m0.d + (size_t)r0 * nb;
        q[R - 1] = ps.m0.q + (size_t)r1 * Kp, d[R - 1] = ps.m0.d + (size_t)r1 * nb;
      }
    else if (ps.mode == 1)
      {
        const int half = ps.N >> 1;
        const int mat = u / half, r0 = 2 * (u - mat * half);
        const long long oq = (mat == 1 ? ps.dq1 : 0) + (mat == 2 ? ps.dq2 : 0);
        const long long od = (mat == 1 ? ps.dd1 : 0) + (mat == 2 ? ps.dd2 : 0);
        q[0] = ps.m0.q + oq + (size_t)r0 * Kp;
        d[0] = (const uint16_t *)((const uint8_t *)ps.m0.d + od) + (size_t)r0 * nb;
        q[R - 1] = q[0] + Kp, d[R - 1] = d[0] + nb;
      }
    else
      {
        q[0] = ps.m0.q + (size_t)u * Kp, d[0] = ps.m0.d + (size_t)u * nb;
        q[R - 1] = ps.m0.q + ps.dq1 + (size_t)u * Kp;
        d[R - 1] = (const uint16_t *)((const uint8_t *)ps.m0.d + ps.dd1) + (size_t)u * nb;
      }
  }

  // the range of units of this workgroup / wave; issues the first `depth`
  // (0..2) items
  static __device__ __forceinline__ void
  begin (PipeState &ps, PipeBuf &A, PipeBuf &B, int mode, const QMat a,
         const QMat b, const QMat c, int N, int K, int wg, int G, int depth,
         const uint16_t *residual = nullptr, bool always = false,
         const Deal dl = Deal{ 0, 0, 0, 0 })
  {
    ps.mode = mode;
    ps.residual = residual;
    ps.m0 = a;
    ps.dq1 = b.q - a.q, ps.dq2 = c.q - a.q;
    ps.dd1 = (const uint8_t *)b.d - (const uint8_t *)a.d;
    ps.dd2 = (const uint8_t *)c.d - (const uint8_t *)a.d;
    ps.N = N;
    if (WT == 8)
      ps.Kp = ((K + 31) >> 5) << 5, ps.nb = ps.Kp >> 5;
    else
      ps.Kp = K * 2, ps.nb = 0; // row bytes
    ps.nch = (ps.Kp + CHUNK - 1) / CHUNK;
    ps.lane = threadIdx.x & 63, ps.wave = threadIdx.x >> 6, ps.wg = wg;
    const int U = mode == 0 ? (N + R - 1) / R : (mode == 1 ? 3 * (N >> 1) : N);
    int lo, hi;
    // (64 fp16 results per line: 32 two-row units of mode 0, 64 units
    // otherwise; owned dealing serves mode 0 and the pair units of mode 2)
    dealt_units (dl, U, mode == 0 && R == 2 ? 32 : 64, wg, G, lo, hi);
    ps.u_lo = lo + ps.wave;
    ps.U = U;
    const int nunits
        = ps.u_lo < hi ? (hi - ps.u_lo + kDecWaves - 1) / kDecWaves : 0;
    ps.nit = nunits * ps.nch;
    ps.best_v = -INFINITY, ps.best_i = 0xffffffffu;
    ps.primed = 0;
    if (always)
      {
        // the first item without a condition around its loads: the waits
        // that follow in the caller can then be counted exactly
        if (depth >= 1)
          {
            issue (ps, A, 0);
            ps.primed = 1;
          }
        if (depth >= 2)
          {
            issue (ps, B, 1);
            ps.primed = 2;
          }
      }
    else
      prime (ps, A, B, depth);
  }

  // issues the first `depth` (<= 2) items if they are not in flight yet
  static __device__ __forceinline__ void
  prime (PipeState &ps, PipeBuf &A, PipeBuf &B, int depth)
  {
    if (ps.primed < 1 && depth >= 1 && ps.nit > 0)
      {
        issue (ps, A, 0);
        ps.primed = 1;
      }
    if (ps.primed < 2 && depth >= 2 && ps.nit > 1)
      {
        issue (ps, B, 1);
        ps.primed = 2;
      }
  }

  static __device__ __forceinline__ void
  issue (const PipeState &ps, PipeBuf &b, int it)
  {
    const int ui = it / ps.nch, c = it - ui * ps.nch;
    // (a wave without units still requests the last unit's first item when
    // begin () is told to issue unconditionally; it is never consumed)
    const int u = min (ps.u_lo + ui * kDecWaves, ps.U - 1);
    const uint8_t *q[R];
    const uint16_t *d[R];
    rows_of (ps, u, q, d);
    // Every load below is unconditional, from a clamped (always valid)
    // address; what lies outside the row is ignored when the item is
    // consumed.  A branch around a load would keep the compiler from counting
    // the loads in flight, and the wait for one item would then wait for
    // the next one as well.
    //
    // The residual pair of the unit travels with the item, so the epilogue
    // does not start a dependent trip to memory at the end of the row.
    const uint16_t *rp = ps.residual ? ps.residual : (const uint16_t *)ps.m0.q;
    if (R == 1)
      b.res = ldg (rp + u);
    else
      b.res = ldg ((const uint32_t *)(rp + (2 * u + 1 < ps.N ? 2 * u : 0)));
    // an item past the wave's last (requested all the same when begin ()
    // issues unconditionally) reads one and the same KiB for every load, so
    // that it adds nothing to the traffic
    const bool none = it >= ps.nit;
    if (none)
      {
#pragma unroll
        for (int r = 0; r < R; ++r)
          q[r] = ps.m0.q, d[r] = ps.m0.d;
      }
#pragma unroll
    for (int s = 0; s < S; ++s)
      {
        const int kk = c * CHUNK + s * (VKL_WAVE * 16) + ps.lane * 16;
        const int kc = none ? ps.lane * 16 : (kk < ps.Kp ? kk : 0);
#pragma unroll
        for (int r = 0; r < R; ++r)
          {
            b.w[r * S + s] = NT ? ldg4_stream (q[r] + kc) : ldg4 (q[r] + kc);
            if (WT == 8)
              b.d[r * S + s] = ldg (d[r] + (kc >> 5));
          }
      }
  }

  static __device__ __forceinline__ void
  consume (PipeState &ps, float (&acc)[R], const PipeBuf &b, int it,
           const uint16_t *xl, const Epilogue &e)
  {
    const int ui = it / ps.nch, c = it - ui * ps.nch;
    if (c == 0)
      {
#pragma unroll
        for (int r = 0; r < R; ++r)
          acc[r] = 0.f;
      }
#pragma unroll
    for (int s = 0; s < S; ++s)
      {
        const int kk = c * CHUNK + s * (VKL_WAVE * 16) + ps.lane * 16;
        if (WT != 8)
          {
            if (kk < ps.Kp) // kk counts bytes of the fp16 row
              {
                const uint4 xv = *(const uint4 *)(xl + (kk >> 1));
#pragma unroll
                for (int r = 0; r < R; ++r)
                  acc[r] = dot8_f16 (b.w[r * S + s], xv, acc[r]);
              }
          }
        else if (kk < ps.Kp)
          {
            const uint4 *xp = (const uint4 *)(xl + kk);
            const uint4 x0 = xp[0], x1 = xp[1];
            const h16x2 xv[8]
                = { __builtin_bit_cast (h16x2, x0.x), __builtin_bit_cast (h16x2, x0.y),
                    __builtin_bit_cast (h16x2, x0.z), __builtin_bit_cast (h16x2, x0.w),
                    __builtin_bit_cast (h16x2, x1.x), __builtin_bit_cast (h16x2, x1.y),
                    __builtin_bit_cast (h16x2, x1.z), __builtin_bit_cast (h16x2, x1.w) };
#pragma unroll
            for (int r = 0; r < R; ++r)
              acc[r] += dot16_q8 (b.w[r * S + s], xv, 0.f) * h2f (b.d[r * S + s]);
          }
      }
    if (c == ps.nch - 1)
      finish (ps, acc, ps.u_lo + ui * kDecWaves, e, b.res);
  }

  static __device__ __forceinline__ void
  finish (PipeState &ps, const float (&acc)[R], int u, const Epilogue &e,
          uint32_t res)
  {
    float v[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
      v[r] = wave_sum (acc[r]);
    if (ps.lane != 0)
      return;
    const int N = ps.N;
    if (R == 1)
      {
        // one row per unit (mode 0, launch-per-phase kernels only)
        uint16_t h = f2h (v[0]);
        if (e.residual)
          h = f2h (h2f (h) + h2f (ps.residual ? (uint16_t)(res & 0xffff) : ldg (e.residual + u)));
        st_h (e, e.y[0] + u, h);
        if (e.y32)
          stg (e.y32 + u, h2f (h));
        if (e.amax_val && better (h2f (h), (uint32_t)u, ps.best_v, ps.best_i))
          ps.best_v = h2f (h), ps.best_i = (uint32_t)u;
        return;
      }
    if (ps.mode == 1)
      {
        const int half = N >> 1;
        const int mat = u / half, r0 = 2 * (u - mat * half);
        // the three outputs are N elements apart
        uint16_t *y = e.y[0] + (size_t)mat * N;
        st_h2 (e, (uint32_t *)(y + r0), (uint32_t)f2h (v[0]) | ((uint32_t)f2h (v[R - 1]) << 16));
        return;
      }
    if (ps.mode == 2)
      {
        st_h (e, e.y[0] + u, f2h (silu (v[R - 1]) * v[0]));
        return;
      }
    const int r0 = 2 * u;
    const bool two = r0 + 1 < N;
    uint16_t h0 = f2h (v[0]), h1 = f2h (v[R - 1]);
    if (e.residual)
      {
        // prefetched with the item unless the phase was begun without it
        const uint32_t rr
            = !two ? (uint32_t)ldg (e.residual + r0)
                   : (ps.residual ? res
                                  : ldg ((const uint32_t *)(e.residual + r0)));
        h0 = f2h (h2f (h0) + h2f ((uint16_t)(rr & 0xffff)));
        h1 = f2h (h2f (h1) + h2f ((uint16_t)(rr >> 16)));
      }
    if (two)
      st_h2 (e, (uint32_t *)(e.y[0] + r0), (uint32_t)h0 | ((uint32_t)h1 << 16));
    else
      st_h (e, e.y[0] + r0, h0);
    if (e.y32)
      {
        stg (e.y32 + r0, h2f (h0));
        if (two)
          stg (e.y32 + r0 + 1, h2f (h1));
      }
    if (e.amax_val)
      {
        if (better (h2f (h0), (uint32_t)r0, ps.best_v, ps.best_i))
          ps.best_v = h2f (h0), ps.best_i = (uint32_t)r0;
        if (two && better (h2f (h1), (uint32_t)r0 + 1, ps.best_v, ps.best_i))
          ps.best_v = h2f (h1), ps.best_i = (uint32_t)r0 + 1;
      }
  }

  // All items through ONE buffer (the other one may hold an item of the next
  // phase): the first item is in flight in A (begin with depth 1), later
  // items are requested when A is free.  For phases whose waves have one
  // item, seldom two.
  static __device__ __forceinline__ void
  run_single (PipeState &ps, PipeBuf &A, const uint16_t *xl, const Epilogue &e)
  {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
      acc[r] = 0.f;
    const int nit = ps.nit;
    for (int it = 0; it < nit; ++it)
      {
        consume (ps, acc, A, it, xl, e);
        if (it + 1 < nit)
          issue (ps, A, it + 1);
      }
  }

  // all items; xl must be staged.  `red` = 2*kDecWaves LDS words.
  static __device__ __forceinline__ void
  run (PipeState &ps, PipeBuf &A, PipeBuf &B, const uint16_t *xl,
       const Epilogue &e, float *red)
  {
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
      acc[r] = 0.f;
    prime (ps, A, B, 1);
    const int nit = ps.nit;
    for (int it = 0; it < nit; it += 2)
      {
        if (it + 1 < nit && !(it == 0 && ps.primed == 2))
          issue (ps, B, it + 1);
        consume (ps, acc, A, it, xl, e);
        if (it + 1 < nit)
          {
            if (it + 2 < nit)
              issue (ps, A, it + 2);
            consume (ps, acc, B, it + 1, xl, e);
          }
      }
    if (e.amax_val)
      {
        // lane 0 of each wave holds that wave's best; combine in LDS
        float *bv = red;
        uint32_t *bi = (uint32_t *)(red + kDecWaves);
        __syncthreads ();
        if (ps.lane == 0)
          {
            bv[ps.wave] = ps.best_v;
            bi[ps.wave] = ps.best_i;
          }
        __syncthreads ();
        if (threadIdx.x == 0)
          {
            float v = bv[0];
            uint32_t i = bi[0];
            for (int w = 1; w < kDecWaves; ++w)
              if (better (bv[w], bi[w], v, i))
                v = bv[w], i = bi[w];
            // (written through: the launch's last workgroup may read them)
            st_coherent_u32 ((uint32_t *)(e.amax_val + ps.wg), __float_as_uint (v));
            st_coherent_u32 (e.amax_idx + ps.wg, i);
          }
      }
  }
};
} // namespace
} // namespace dec
} // namespace vkl
#endif
