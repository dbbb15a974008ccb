// The decode step as ONE persistent launch per token (Q8_0 weights).
//
// All G workgroups are resident (one per compute unit, 512 threads).  Wave 0
// of a workgroup hands activations over; waves 1..7 stream weights and never
// touch global memory otherwise:
//
//   wave 0 (control)                         waves 1..7 (workers)
//   ----------------                         --------------------
//   norm weights -> LDS                      (weight items of this and later
//   wait for the producers of the row         phases are in flight)
//   row -> LDS (coherent, LDS-direct)
//   ------------------------------ barrier ------------------------------
//   all threads: RMSNorm of the row inside LDS (norm phases)
//   ------------------------------ barrier ------------------------------
//   (idle)                                   consume this phase's items from
//                                            registers, request later items
//                                            (also of later PHASES), results
//                                            -> LDS
//   ------------------------------ barrier ------------------------------
//   results (+ residual) -> memory with
//   write-through stores, arrival
//
// A worker's items form one sequence over all phases of the token, consumed
// in groups of four from four register buffers; the group after the one being
// consumed is always in flight.  Weights do not depend on activations, so this
// look-ahead runs across phase boundaries: while a workgroup waits for the
// grid to arrive and for its row, HBM keeps streaming the next phase's
// weights.  Arrivals are counted per slot (workgroup index mod 8, which is the
// XCD a workgroup runs on; one counter for all workgroups serialises every
// atomic on one address: 3.7 us for 256 arrivals against 1.5 us); the last
// arriver of a slot publishes the epoch in the slot's flag and a waiter polls
// the eight flags.  Activations cross workgroups through write-through stores
// and loads that bypass the per-XCD L2 (sc0 sc1).  Every wait is bounded: a
// wait that gives up sets the error word of the scratch buffer, which
// vkl_decode_status reports, and the launch runs to its end without waiting.
#include "vkl_decode_shared.h"
#include <algorithm>

namespace vkl
{
namespace dec
{
namespace
{
constexpr int kPWorkers = kDecWaves - 1;
constexpr int kSyncErr = 1;    // word index: a wait gave up
constexpr int kSyncCnt = 64;   // + 32 * slot: arrivals of the slot
constexpr int kSyncFlag = 512; // + 32 * slot: last epoch the slot completed
constexpr int kSyncSlots = 8;
constexpr int kSyncWords = kSyncFlag + 32 * kSyncSlots;
constexpr int kSpinLimit = 1 << 20;
constexpr int kOutvBytes = 1024; // a workgroup's results of one phase, fp16
constexpr int kGeoBytes = 64;    // units [lo, hi) of the workgroup per kind of phase

// kinds of phase in the flat sequence [5 per layer] + output layer
enum Kind
{
  K_KQV = 0,
  K_ATTN,
  K_WO,
  K_UPGATE,
  K_DOWN,
  K_HEAD
};

// One phase of the token as the workers see it; the table of all phases is
// written in front of every launch and read with scalar loads.  A unit is two
// rows: rows 2u and 2u + 1 of a matrix, or row u of the up matrix and row u of
// the gate matrix.
// fields of vkl_layer_weights as 64-bit words (the layer table is read with
// scalar loads, one field at a time)
constexpr int kLwAttnNorm = offsetof (vkl_layer_weights, attn_norm) / 8;
constexpr int kLwFfnNorm = offsetof (vkl_layer_weights, ffn_norm) / 8;
constexpr int kLwKcache = offsetof (vkl_layer_weights, kcache) / 8;
constexpr int kLwVcache = offsetof (vkl_layer_weights, vcache) / 8;

struct PhaseRec
{
  // int8 plane and scale plane of the first matrix; K/Q/V has three matrices,
  // the second and third at these byte offsets from the first (selecting among
  // pointers by a run-time index would move the record out of registers)
  const uint8_t *Q0, *D0;
  long long qm1, qm2, dm1, dm2;
  long long dq1r, dd1r; // from a unit's first row to its second, bytes
  int qs, ds;           // from a unit's first row to the next unit's, bytes
  int upm;              // units per matrix
  int Kp, nch;          // padded row length, chunks of 4096 per row
  int silu;             // the unit's result is silu(row 1) * row 0
  int kind, N;
  int pad[8];
};
static_assert (offsetof (PhaseRec, qs) == 64 && sizeof (PhaseRec) == 128, "PhaseRec is read as 32 words");

typedef uint32_t pu32x4 __attribute__ ((ext_vector_type (4)));
typedef uint32_t pu32x8 __attribute__ ((ext_vector_type (8)));
typedef uint32_t pu32x16 __attribute__ ((ext_vector_type (16)));

__device__ __forceinline__ PhaseRec
load_phase (const uint8_t *ptab, int ph)
{
  // through the constant address space: scalar loads, tracked by the scalar
  // counter (a vector load would queue behind the weight loads in flight);
  // field by field, so that the record lives in scalar registers
  typedef const __attribute__ ((address_space (4))) unsigned long long *cptr;
  typedef const __attribute__ ((address_space (4))) int *iptr;
  cptr t = (cptr) (ptab + (size_t)ph * sizeof (PhaseRec));
  iptr w = (iptr) (ptab + (size_t)ph * sizeof (PhaseRec));
  PhaseRec r;
  r.Q0 = (const uint8_t *)t[0], r.D0 = (const uint8_t *)t[1];
  r.qm1 = (long long)t[2], r.qm2 = (long long)t[3];
  r.dm1 = (long long)t[4], r.dm2 = (long long)t[5];
  r.dq1r = (long long)t[6], r.dd1r = (long long)t[7];
  r.qs = w[16], r.ds = w[17], r.upm = w[18], r.Kp = w[19], r.nch = w[20];
  r.silu = w[21], r.kind = w[22], r.N = w[23];
  return r;
}

__device__ __forceinline__ int
phase_kind (int ph, int L)
{
  return ph < 5 * L ? ph % 5 : K_HEAD;
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t
buf_rsrc (const void *p, uint32_t bytes)
{
  return __builtin_amdgcn_make_buffer_rsrc ((void *)p, 0, (int)bytes, 0x00020000);
}

// cache policy of a buffer access: sc0 | sc1 = coherent across the GPU
constexpr int kAuxCoherent = 17;

__device__ __forceinline__ void
st_coherent_u16 (uint16_t *p, uint16_t v)
{
  __hip_atomic_store (p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct PSync
{
  uint32_t *words;
  uint32_t slot;     // of this workgroup
  uint32_t cum;      // arrivals of the slot that complete the current epoch
  uint32_t per_proj; // arrivals of the slot in a projection epoch
  uint32_t per_attn; // ... in an attention epoch
  uint32_t n_attn;   // workgroups that run attention heads
  bool dead;         // a wait gave up: no more waiting in this launch
};

__device__ __forceinline__ PSync
psync_init (const Params &p, int wg, int G, int n_attn)
{
  PSync gs;
  gs.words = p.s.sync;
  gs.slot = (uint32_t)wg & (kSyncSlots - 1);
  gs.cum = 0;
  gs.per_proj = (uint32_t)(G + kSyncSlots - 1 - (int)gs.slot) / kSyncSlots;
  gs.per_attn = (uint32_t)(n_attn + kSyncSlots - 1 - (int)gs.slot) / kSyncSlots;
  gs.n_attn = (uint32_t)n_attn;
  gs.dead = false;
  return gs;
}

// this workgroup has finished the epoch (wave 0; its stores are complete)
__device__ __forceinline__ void
psync_arrive (const PSync &g, uint32_t epoch)
{
  if ((threadIdx.x & 63) == 0)
    {
      const uint32_t old = __hip_atomic_fetch_add (
          g.words + kSyncCnt + 32 * g.slot, 1u, __ATOMIC_RELAXED,
          __HIP_MEMORY_SCOPE_AGENT);
      if (old + 1u == g.cum)
        st_coherent_u32 (g.words + kSyncFlag + 32 * g.slot, epoch);
    }
}

// wave 0: until every slot with arrivals in `epoch` has completed it
__device__ __forceinline__ void
psync_wait (PSync &g, uint32_t epoch, bool attn_epoch)
{
  if (g.dead)
    return;
  const uint32_t s = threadIdx.x & (kSyncSlots - 1);
  // slots without a workgroup in an attention epoch never publish it
  const bool need = !attn_epoch || s < g.n_attn;
  bool ok = false;
  for (int spin = 0; spin < kSpinLimit; ++spin)
    {
      const uint32_t v = ld_coherent_u32 (g.words + kSyncFlag + 32 * s);
      const bool good = !need || (int32_t)(v - epoch) >= 0;
      if (__builtin_amdgcn_ballot_w64 (!good) == 0)
        {
          ok = true;
          break;
        }
      __builtin_amdgcn_s_sleep (1);
    }
  if (!ok)
    {
      g.dead = true;
      if ((threadIdx.x & 63) == 0)
        st_coherent_u32 (g.words + kSyncErr, 1u);
    }
}

// LDS carve-up
struct PLds
{
  uint16_t *xl;   // staged row
  float *red;     // reduction words
  uint8_t *nl;    // fp32 norm weights of the phase
  uint16_t *outv; // the workgroup's results of the phase
  int *geo;       // [6][2]: units [lo, hi) of the workgroup per kind
  int *flags;     // [0] last phase whose row is staged, [1] units finished so far
};

__host__ __device__ inline size_t
kib (size_t v)
{
  return (v + 1023) & ~(size_t)1023;
}

// the staged row: whole chunks of 4096 values (a worker multiplies whole
// chunks; beyond K the row is zero)
__host__ __device__ inline size_t
row_bytes (size_t kmax)
{
  return ((kmax + 4095) & ~(size_t)4095) * 2;
}

// bytes below the geometry words: the staging layout (row in whole KiB
// requests, reduction words, norm weights, results) or the attention of a
// head, which works in the same memory
__host__ __device__ inline size_t
persist_geo_offset (int dim, int ffn, int maxlen, int hd)
{
  const size_t kmax = (size_t)(dim > ffn ? dim : ffn);
  const size_t stage = row_bytes (kmax) + 256 + kib ((size_t)dim * 4) + kOutvBytes;
  const size_t rpb = kDecThreads / (hd / 8);
  const size_t attn = 1024 + (size_t)((maxlen + 3) & ~3) * 4 + rpb * hd * 4 + 256;
  return ((stage > attn ? stage : attn) + 63) & ~(size_t)63;
}

__host__ __device__ inline size_t
persist_lds_bytes (int dim, int ffn, int maxlen, int hd)
{
  return persist_geo_offset (dim, ffn, maxlen, hd) + kGeoBytes;
}

__device__ __forceinline__ PLds
persist_lds (uint8_t *lds, const vkl_decode_model &m)
{
  const int kmax = m.dim > m.ffn ? m.dim : m.ffn;
  PLds l;
  l.xl = (uint16_t *)lds;
  l.red = (float *)(lds + row_bytes (kmax));
  l.nl = (uint8_t *)l.red + 256;
  l.outv = (uint16_t *)(l.nl + kib ((size_t)m.dim * 4));
  l.geo = (int *)(lds + persist_geo_offset (m.dim, m.ffn, m.maxlen, m.head_dim));
  l.flags = l.geo + 12;
  return l;
}

// units of a phase of each kind
__device__ __forceinline__ int
kind_units (const vkl_decode_model &m, int kind)
{
  switch (kind)
    {
    case K_KQV:
      return 3 * (m.dim >> 1);
    case K_ATTN:
      return 0;
    case K_UPGATE:
      return m.ffn;
    case K_HEAD:
      return (m.vocab + 1) >> 1;
    default:
      return m.dim >> 1;
    }
}

__device__ __forceinline__ int
uniform (int v)
{
  return __builtin_amdgcn_readfirstlane (v);
}

// the workgroup's units go round the workers
__device__ __forceinline__ int
worker_stride (int wv)
{
  return kPWorkers;
}

// units of worker wv among the workgroup's [lo, hi): wv, wv + stride, ...
__device__ __forceinline__ int
worker_units (int lo, int hi, int wv)
{
  const int n = hi - lo - wv, st = worker_stride (wv);
  return n > 0 ? (n + st - 1) / st : 0;
}

// The registers of one item: 8 x 16 weights and their 8 block scales per lane.
// A scale is fetched as the aligned 32-bit word that holds it and picked out
// when the item is consumed: values known to be 16 bits wide get packed in
// pairs by the compiler at the end of the loop body, and that packing waits
// for every load in flight.
struct PBuf
{
  uint4 w[8];
  uint32_t d[8];
};

// Requests chunk c (4096 values of K) of unit u: 8 weight loads and 8 scale
// loads per lane, all unconditional from clamped addresses so that the
// compiler counts the loads in flight exactly.  `none`: nothing to request in
// this slot; the same cached KiB is read instead, which adds no traffic.
template <bool NT>
__device__ __forceinline__ void
pissue (PBuf &b, const PhaseRec &r, int u, int c, bool none, int lane)
{
  const int mat = (u >= r.upm ? 1 : 0) + (u >= 2 * r.upm ? 1 : 0);
  const int lu = u - mat * r.upm;
  const uint8_t *q0 = r.Q0 + (mat == 1 ? r.qm1 : 0) + (mat == 2 ? r.qm2 : 0) + (long long)lu * r.qs;
  const uint8_t *d0 = r.D0 + (mat == 1 ? r.dm1 : 0) + (mat == 2 ? r.dm2 : 0) + (long long)lu * r.ds;
  const uint8_t *q1 = q0 + r.dq1r, *d1 = d0 + r.dd1r;
  if (none)
    q0 = q1 = r.Q0, d0 = d1 = r.D0;
  // a scale is fetched as the aligned 32-bit word that holds it: scalar base
  // rounded down, the remainder added to the lane's offset
  const int p0 = (int)((uintptr_t)d0 & 3), p1 = (int)((uintptr_t)d1 & 3);
  const uint8_t *d0a = d0 - p0, *d1a = d1 - p1;
#pragma unroll
  for (int k = 0; k < 4; ++k)
    {
      // (unsigned: the offsets extend to 64 bits without a sign, so a load takes
      // its scalar base and this one register)
      const uint32_t kk = (uint32_t)(c * 4096 + k * 1024 + lane * 16);
      const uint32_t kc = none ? (uint32_t)lane * 16u : (kk < (uint32_t)r.Kp ? kk : 0u);
      b.w[k] = NT ? ldg4_stream (q0 + kc) : ldg4 (q0 + kc);
      b.d[k] = ldg ((const uint32_t *)(d0a + (((kc >> 5) * 2u + (uint32_t)p0) & ~3u)));
      b.w[4 + k] = NT ? ldg4_stream (q1 + kc) : ldg4 (q1 + kc);
      b.d[4 + k] = ldg ((const uint32_t *)(d1a + (((kc >> 5) * 2u + (uint32_t)p1) & ~3u)));
    }
}

// the arithmetic of Gemv::consume / finish for Q8_0 two-row units; lane 0
// leaves the unit's fp16 results in the workgroup's LDS result array
__device__ __forceinline__ void
pconsume (const PBuf &b, int nch, int silu_out, int oi, int c, int sh0, int sh1,
          float (&acc)[2], const uint16_t *xl, uint16_t *outv, int *done, int lane)
{
  // sh0 / sh1: where in its 32-bit word the lane's block scale sits, for the
  // unit's two rows (the same for every 1024-wide step: 1024 / 32 is even).
  // The staged row is zero beyond K up to a multiple of 4096, and what was
  // fetched for those positions is real data: the products vanish.
  if (c == 0)
    acc[0] = acc[1] = 0.f;
#pragma unroll
  for (int k = 0; k < 4; ++k)
    {
      const int kk = c * 4096 + k * 1024 + lane * 16;
        {
          const uint4 *xp = (const uint4 *)(xl + kk);
          const uint4 x0 = xp[0], x1 = xp[1];
          const h16x2 xv[8]
              = { __builtin_bit_cast (h16x2, x0.x), __builtin_bit_cast (h16x2, x0.y),
                  __builtin_bit_cast (h16x2, x0.z), __builtin_bit_cast (h16x2, x0.w),
                  __builtin_bit_cast (h16x2, x1.x), __builtin_bit_cast (h16x2, x1.y),
                  __builtin_bit_cast (h16x2, x1.z), __builtin_bit_cast (h16x2, x1.w) };
          acc[0] += dot16_q8 (b.w[k], xv, 0.f) * h2f ((uint16_t)(b.d[k] >> sh0));
          acc[1] += dot16_q8 (b.w[4 + k], xv, 0.f) * h2f ((uint16_t)(b.d[4 + k] >> sh1));
        }
    }
  if (c == nch - 1)
    {
      const float v0 = wave_sum (acc[0]), v1 = wave_sum (acc[1]);
      if (lane == 0)
        {
          if (silu_out)
            outv[oi] = f2h (silu (v1) * v0);
          else
            ((uint32_t *)outv)[oi] = (uint32_t)f2h (v0) | ((uint32_t)f2h (v1) << 16);
          // the result is in LDS before the count says so (LDS operations of a
          // wave complete in order)
          asm volatile("" ::: "memory");
          __hip_atomic_fetch_add (done, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
}

// wave 0: `bytes` from global memory straight into LDS, 1 KiB per request
// (lane l delivers 16 bytes at offset 16 l of the request's KiB); what lies
// past `bytes` arrives as zeros
template <bool COHERENT>
__device__ __forceinline__ void
copy_to_lds (const void *src, uint32_t bytes, uint8_t *dst, int lane)
{
  const __amdgpu_buffer_rsrc_t r = buf_rsrc (src, bytes);
  typedef __attribute__ ((address_space (3))) void *lds_ptr;
  const int n = (int)((bytes + 1023) >> 10);
  for (int i = 0; i < n; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds (r, (lds_ptr)(dst + i * 1024), 16, lane * 16,
                                              i * 1024, 0, COHERENT ? kAuxCoherent : 0);
}

#ifdef VKL_TRACE
#define VKL_PTR(ph, slot)                                                     \
  if ((threadIdx.x & 63) == 0 && p.trace)                                     \
    p.trace[((size_t)(ph)*1024 + blockIdx.x) * 8 + (slot)] = wall_clock64 ();
#define VKL_PTW(ph, slot)                                                     \
  if (wv == 0)                                                                \
    {                                                                         \
      VKL_PTR (ph, slot)                                                      \
    }
#else
#define VKL_PTR(ph, slot)
#define VKL_PTW(ph, slot)
#endif

// Words in LDS through which wave 0 and the workers of a workgroup meet (no
// workgroup barrier: a worker that is still requesting weights holds nobody
// up).  Accesses are relaxed atomics of workgroup scope; LDS operations of a
// wave complete in order, so data written before a word is visible with it.
__device__ __forceinline__ int
lds_peek (const int *w)
{
  const int v = __hip_atomic_load (w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  asm volatile("" ::: "memory");
  return v;
}

__device__ __forceinline__ void
lds_post (int *w, int v)
{
  asm volatile("" ::: "memory");
  __hip_atomic_store (w, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// wave 0: RMSNorm of the row inside LDS, every sum in the order in which the
// 512 threads of stage_row form it: lane l stands for threads l, l + 64, ...
__device__ __forceinline__ void
norm_row_wave (uint16_t *xl, const uint8_t *nl, int K, float eps, int lane)
{
  // sq[v]: the sum thread v * 64 + lane of stage_row forms over its chunks
  float sq[kDecWaves];
#pragma unroll
  for (int v = 0; v < kDecWaves; ++v)
    sq[v] = 0.f;
#pragma unroll 1
  for (int j = 0; j < 4; ++j)
    {
      if (j * kDecThreads * 8 >= K)
        break;
      uint4 x[kDecWaves];
#pragma unroll
      for (int v = 0; v < kDecWaves; ++v)
        {
          const int idx = v * 64 + lane + j * kDecThreads;
          x[v] = ((const uint4 *)xl)[idx * 8 < K ? idx : 0];
        }
#pragma unroll
      for (int v = 0; v < kDecWaves; ++v)
        {
          const int idx = v * 64 + lane + j * kDecThreads;
          const uint32_t w[4] = { x[v].x, x[v].y, x[v].z, x[v].w };
          float s = sq[v];
#pragma unroll
          for (int i = 0; i < 4; ++i)
            {
              const float a = h2f ((uint16_t)(w[i] & 0xffff));
              const float b = h2f ((uint16_t)(w[i] >> 16));
              s += a * a;
              s += b * b;
            }
          sq[v] = idx * 8 < K ? s : sq[v];
        }
    }
  // block_sum: the waves' sums added in wave order
  float total = 0.f;
#pragma unroll
  for (int v = 0; v < kDecWaves; ++v)
    total += wave_sum (sq[v]);
  const float alpha = 1.0f / sqrtf (total / (float)K + eps);
#pragma unroll 1
  for (int j = 0; j < 4; ++j)
    {
#pragma unroll
      for (int v = 0; v < kDecWaves; ++v)
        {
          const int idx = v * 64 + lane + j * kDecThreads;
          if (idx * 8 < K)
            {
              const uint4 x = ((const uint4 *)xl)[idx];
              const uint32_t w[4] = { x.x, x.y, x.z, x.w };
              const uint4 g0 = ((const uint4 *)nl)[2 * idx], g1 = ((const uint4 *)nl)[2 * idx + 1];
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
              ((uint4 *)xl)[idx] = make_uint4 (r[0], r[1], r[2], r[3]);
            }
        }
    }
}

// wave 0 of a workgroup
template <int HD>
__device__ __forceinline__ void
persistent_control (const Params &p, int G, uint8_t *lds)
{
  const vkl_decode_model &m = p.m;
  const int wg = (int)blockIdx.x;
  const int dim = m.dim, ffn = m.ffn, L = m.n_layers;
  const int lane = threadIdx.x & 63;
  const PLds l = persist_lds (lds, m);
  const int nph = 5 * L + 1;
  const int n_attn = m.n_heads < G ? m.n_heads : G;
  const bool attn_wg = wg < n_attn;
  PSync gs = psync_init (p, wg, G, n_attn);
  int units_done = 0; // units the workers have finished once the current phase is complete

  for (int ph = 0; ph < nph; ++ph)
    {
      const int layer = ph < 5 * L ? ph / 5 : L - 1;
      const int kind = phase_kind (ph, L);
      const uint32_t epoch = (uint32_t)ph + 1u;
      const vkl_layer_weights *lw = m.layers + layer;
      typedef const __attribute__ ((address_space (4))) unsigned long long *cptr;
      cptr lwp = (cptr)lw; // read with scalar loads
      if (kind == K_ATTN)
        {
          gs.cum += gs.per_attn;
          if (attn_wg)
            {
              vkl_layer_weights w = {};
              w.kcache = (void *)lwp[kLwKcache], w.vcache = (void *)lwp[kLwVcache];
              VKL_PTR (ph, 0)
              psync_wait (gs, epoch - 1u, false);
              VKL_PTR (ph, 1)
              __syncthreads (); // the workers have nothing in flight and join
              for (int h = wg; h < m.n_heads; h += G)
                attention_head<HD, true> (p, w, h, lds);
              // this wave's stores are complete
              __builtin_amdgcn_s_waitcnt (0x0f70);
              __syncthreads ();
              VKL_PTR (ph, 4)
              psync_arrive (gs, epoch);
              VKL_PTR (ph, 5)
            }
          continue;
        }
      const int lo = uniform (l.geo[2 * kind]), hi = uniform (l.geo[2 * kind + 1]);
      const int nu = hi - lo; // units of the workgroup
      const int K = kind == K_DOWN ? ffn : dim;
      const bool norm = kind == K_KQV || kind == K_UPGATE || kind == K_HEAD;
      const bool resid = kind == K_WO || kind == K_DOWN;
      gs.cum += gs.per_proj;
      units_done += nu;
      uint32_t res = 0; // residual pair of lane l's unit
      VKL_PTR (ph, 0)
      if (norm)
        {
          const float *nwp = kind == K_KQV ? (const float *)lwp[kLwAttnNorm]
                             : (kind == K_UPGATE ? (const float *)lwp[kLwFfnNorm] : m.output_norm);
          copy_to_lds<false> (nwp, (uint32_t)dim * 4, l.nl, lane);
        }
      if (ph == 0)
        {
          // the token's embedding row: fp16(float(q) * float(d)); workgroup 0
          // also makes it the residual stream
          uint32_t tok = ldg (step_tok (p));
          if (tok >= (uint32_t)m.vocab)
            tok = 0;
          const QMat tab = qmat (m.tok_embd, m.vocab, dim);
          const __amdgpu_buffer_rsrc_t rx = buf_rsrc (p.s.x, (uint32_t)dim * 2);
#pragma unroll 1
          for (int c0 = 0; c0 < (dim >> 3); c0 += 256)
            {
              unsigned long long qv[4];
              uint16_t dv[4];
#pragma unroll
              for (int v = 0; v < 4; ++v)
                {
                  const int ch = min (c0 + v * 64 + lane, (dim >> 3) - 1);
                  qv[v] = ldg ((const unsigned long long *)(tab.q + (size_t)tok * dim + ch * 8));
                  dv[v] = ldg (tab.d + (size_t)tok * (dim >> 5) + (ch >> 2));
                }
#pragma unroll
              for (int v = 0; v < 4; ++v)
                {
                  const int ch = min (c0 + v * 64 + lane, (dim >> 3) - 1);
                  const float sc = h2f (dv[v]);
                  const uint32_t w[2] = { (uint32_t)qv[v], (uint32_t)(qv[v] >> 32) };
                  uint32_t o[4];
#pragma unroll
                  for (int i = 0; i < 4; ++i)
                    {
                      const int8_t b0 = (int8_t)((w[i >> 1] >> (16 * (i & 1))) & 0xff);
                      const int8_t b1 = (int8_t)((w[i >> 1] >> (16 * (i & 1) + 8)) & 0xff);
                      o[i] = (uint32_t)f2h ((float)b0 * sc) | ((uint32_t)f2h ((float)b1 * sc) << 16);
                    }
                  ((uint4 *)l.xl)[ch] = make_uint4 (o[0], o[1], o[2], o[3]);
                  if (wg == 0)
                    {
                      const pu32x4 ov = { o[0], o[1], o[2], o[3] };
                      __builtin_amdgcn_raw_buffer_store_b128 (ov, rx, ch * 16, 0, kAuxCoherent);
                    }
                }
            }
        }
      else
        {
          psync_wait (gs, epoch - 1u, phase_kind (ph - 1, L) == K_ATTN);
          VKL_PTR (ph, 1)
          const uint16_t *src = kind == K_WO ? p.s.att : (kind == K_DOWN ? p.s.t : p.s.x);
          copy_to_lds<true> (src, (uint32_t)K * 2, (uint8_t *)l.xl, lane);
        }
      // zeros from the end of the row to the end of its last chunk of 4096
      for (size_t o = (size_t)K * 2 + (size_t)lane * 16; o < row_bytes ((size_t)K); o += 1024)
        *(uint4 *)((uint8_t *)l.xl + o) = make_uint4 (0, 0, 0, 0);
      if (resid) // x[2 lo .. 2 hi): written two or more phases ago
        res = ld_coherent_u32 ((const uint32_t *)p.s.x + lo + (lane < nu ? lane : 0));
      // the row (and the norm weights) are in LDS
      __builtin_amdgcn_s_waitcnt (0x0f70);
      VKL_PTR (ph, 2)
      if (norm)
        norm_row_wave (l.xl, l.nl, K, kind == K_HEAD ? m.final_eps : m.eps, lane);
      // the workers may consume the phase's items
      __builtin_amdgcn_s_waitcnt (0xc07f); // lgkmcnt(0)
      lds_post (l.flags + 0, ph);
      VKL_PTR (ph, 3)
      // until every unit of the phase has been finished
      for (int spin = 0; lds_peek (l.flags + 1) < units_done && spin < (1 << 24); ++spin)
        __builtin_amdgcn_s_sleep (1);
      VKL_PTR (ph, 4)
      if (kind == K_UPGATE)
        {
          if (lane < nu)
            st_coherent_u16 (p.s.t + lo + lane, l.outv[lane]);
        }
      else if (kind == K_HEAD)
        {
          float bv = -INFINITY;
          uint32_t bi = 0xffffffffu;
          for (int i = lane; i < 2 * nu; i += 64)
            {
              const int r = 2 * lo + i;
              if (r < m.vocab)
                {
                  const uint16_t h = l.outv[i];
                  stg (p.s.logits16 + r, h);
                  stg (p.logits32 + r, h2f (h));
                  if (better (h2f (h), (uint32_t)r, bv, bi))
                    bv = h2f (h), bi = (uint32_t)r;
                }
            }
#pragma unroll
          for (int o = 32; o > 0; o >>= 1)
            {
              const float ov = __shfl_xor (bv, o, 64);
              const uint32_t oi = __shfl_xor (bi, o, 64);
              if (better (ov, oi, bv, bi))
                bv = ov, bi = oi;
            }
          if (lane == 0)
            {
              st_coherent_u32 ((uint32_t *)(p.s.amax_val + wg), __float_as_uint (bv));
              st_coherent_u32 (p.s.amax_idx + wg, bi);
            }
        }
      else if (lane < nu)
        {
          uint32_t v = ((const uint32_t *)l.outv)[lane];
          if (resid)
            {
              const uint16_t h0 = f2h (h2f ((uint16_t)(v & 0xffff)) + h2f ((uint16_t)(res & 0xffff)));
              const uint16_t h1 = f2h (h2f ((uint16_t)(v >> 16)) + h2f ((uint16_t)(res >> 16)));
              v = (uint32_t)h0 | ((uint32_t)h1 << 16);
            }
          uint16_t *dst = kind == K_KQV ? p.s.kqv : p.s.x;
          st_coherent_u32 ((uint32_t *)dst + lo + lane, v);
        }
      __builtin_amdgcn_s_waitcnt (0x0f70);
      psync_arrive (gs, epoch);
      VKL_PTR (ph, 5)
    }
  if ((p.next_tok || p.loop) && wg == 0)
    {
      psync_wait (gs, (uint32_t)nph, false);
      __syncthreads ();
      final_argmax<true> (p, G, lds);
    }
}

// which item a register buffer holds
struct Slot
{
  int ph; // phase, < 0: none
  int oi; // the unit's index among the workgroup's units
  int c;  // chunk of the row
};

// waves 1..7 of a workgroup
template <int HD, bool NT>
__device__ __forceinline__ void
persistent_worker (const Params &p, int G, uint8_t *lds, int wv)
{
  const vkl_decode_model &m = p.m;
  const int wg = (int)blockIdx.x;
  const int dim = m.dim, ffn = m.ffn, L = m.n_layers;
  const int lane = threadIdx.x & 63;
  const PLds l = persist_lds (lds, m);
  const uint8_t *ptab = p.s.ptab;
  const int nph = 5 * L + 1;
  const int n_attn = m.n_heads < G ? m.n_heads : G;
  const bool attn_wg = wg < n_attn;

  PBuf A, B, C, D;
  Slot sa = { -1, 0, 0 }, sb = sa, sc = sa, sd = sa;
  // request position: phase, its record, the worker's unit index and chunk
  PhaseRec ir = load_phase (ptab, 0);
  int iph = -1, inu = 0, iui = 0, ic = 0;
  bool held = false; // an attention workgroup does not look ahead past its attention phase
  // consumption: the phase whose row this wave has seen staged
  int cur = -1, cKp = 0, cnch = 1, csilu = 0, clo = 0;
  const int lanepar = (lane >> 1) & 1; // the lane's 16 values are the upper half of their block's pair
  float acc[2] = { 0.f, 0.f };

  for (;;)
    {
      // ---- move the request position to a phase with items of this worker
      while (!held && iph < nph && iui >= inu)
        {
          ++iph;
          if (iph >= nph)
            break;
          const int k = phase_kind (iph, L);
          if (k == K_ATTN)
            {
              held = attn_wg;
              continue;
            }
          inu = worker_units (uniform (l.geo[2 * k]), uniform (l.geo[2 * k + 1]), wv);
          iui = 0, ic = 0;
          if (inu > 0)
            ir = load_phase (ptab, iph);
        }
      const bool empty = sa.ph < 0 && sb.ph < 0 && sc.ph < 0 && sd.ph < 0;
      if (empty && iph >= nph)
        break;
      if (empty && held)
        {
          // the attention phase iph of this workgroup: all eight waves
          typedef const __attribute__ ((address_space (4))) unsigned long long *cptr;
          cptr lwp = (cptr)(m.layers + iph / 5);
          vkl_layer_weights w = {};
          w.kcache = (void *)lwp[kLwKcache], w.vcache = (void *)lwp[kLwVcache];
          __syncthreads (); // wave 0 has seen the K/Q/V phase complete
          for (int h = wg; h < m.n_heads; h += G)
            attention_head<HD, true> (p, w, h, lds);
          // this wave's stores are complete
          __builtin_amdgcn_s_waitcnt (0x0f70);
          __syncthreads ();
          // nothing is in the buffers (saying so frees their registers for the
          // attention code); the look-ahead restarts behind the attention phase
          A = PBuf{};
          B = PBuf{};
          C = PBuf{};
          D = PBuf{};
          held = false;
          inu = 0, iui = 0;
          continue;
        }
      // ---- a round: each buffer's item is consumed, the next item requested
#define VKL_PSTEP(X, sx)                                                      \
  if (sx.ph >= 0)                                                             \
    {                                                                         \
      if (sx.ph != cur)                                                       \
        {                                                                     \
          cur = sx.ph;                                                        \
          while (lds_peek (l.flags + 0) < cur)                                \
            __builtin_amdgcn_s_sleep (1);                                     \
          const int ck = phase_kind (cur, L);                                 \
          cKp = (((ck == K_DOWN ? ffn : dim) + 31) >> 5) << 5;                \
          cnch = (cKp + 4095) / 4096;                                         \
          csilu = ck == K_UPGATE;                                             \
          clo = uniform (l.geo[2 * ck]);                                      \
          VKL_PTW (cur, 6)                                                    \
        }                                                                     \
      {                                                                       \
        /* scale rows are nb 16-bit words long: with nb odd every other */   \
        /* row starts in the upper half of a 32-bit word */                  \
        const int nbodd = (cKp >> 5) & 1;                                     \
        const int par0 = csilu ? ((clo + sx.oi) & nbodd) : 0;                 \
        const int par1 = csilu ? par0 : nbodd;                                \
        pconsume (X, cnch, csilu, sx.oi, sx.c, 16 * (lanepar ^ par0),         \
                  16 * (lanepar ^ par1), acc, l.xl, l.outv, l.flags + 1,      \
                  lane);                                                      \
      }                                                                       \
      VKL_PTW (cur, 7)                                                        \
    }                                                                         \
  /* the buffer's registers are free: the scheduler must not start the */   \
  /* next request before the last use of the item consumed */              \
  __builtin_amdgcn_sched_barrier (0);                                         \
  {                                                                           \
    const bool none = held || iph >= nph || iui >= inu;                       \
    const int oi = wv + iui * worker_stride (wv);                             \
    pissue<NT> (X, ir, uniform (l.geo[2 * ir.kind]) + oi, ic, none, lane);    \
    sx.ph = none ? -1 : iph, sx.oi = oi, sx.c = ic;                           \
    if (!none && ++ic == ir.nch)                                              \
      ic = 0, ++iui;                                                          \
  }                                                                           \
  __builtin_amdgcn_sched_barrier (0);
      VKL_PSTEP (A, sa)
      VKL_PSTEP (B, sb)
      VKL_PSTEP (C, sc)
      VKL_PSTEP (D, sd)
#undef VKL_PSTEP
    }
  if ((p.next_tok || p.loop) && wg == 0)
    {
      __syncthreads ();
      final_argmax<true> (p, G, lds);
    }
}

template <int HD, bool NT>
__global__ __launch_bounds__ (kDecThreads) void
decode_persistent_kernel (const Params p, int G)
{
  extern __shared__ __align__ (16) uint8_t lds[];
  const int wave = __builtin_amdgcn_readfirstlane ((int)(threadIdx.x >> 6));
  {
    // the workgroup's units of each kind of phase, and the words through which
    // its waves meet
    const PLds l = persist_lds (lds, p.m);
    if (threadIdx.x < 6)
      {
        const unsigned U = (unsigned)kind_units (p.m, (int)threadIdx.x);
        l.geo[2 * threadIdx.x] = (int)(U * blockIdx.x / (unsigned)G);
        l.geo[2 * threadIdx.x + 1] = (int)(U * (blockIdx.x + 1) / (unsigned)G);
      }
    if (threadIdx.x == 0)
      l.flags[0] = -1, l.flags[1] = 0;
    __syncthreads ();
  }
  if (wave == 0)
    persistent_control<HD> (p, G, lds);
  else
    persistent_worker<HD, NT> (p, G, lds, wave - 1);
}

// In front of every launch: the arrival counters and flags restart from zero
// (a fill kernel rather than a memset node, so that a caller may capture the
// step in a graph; the error word is left alone, vkl_decode_status reads and
// clears it) and the table of phases is written.
__global__ void
persistent_setup_kernel (const Params p)
{
  const vkl_decode_model &m = p.m;
  for (int i = threadIdx.x; i < kSyncWords; i += blockDim.x)
    if (i != kSyncErr && (i < 16 || i >= 32)) // words 16.. hold the replayed loop's state
      st_coherent_u32 (p.s.sync + i, 0u);
  const int L = m.n_layers, dim = m.dim, ffn = m.ffn;
  for (int ph = threadIdx.x; ph < 5 * L + 1; ph += blockDim.x)
    {
      const int kind = ph < 5 * L ? ph % 5 : K_HEAD;
      const vkl_layer_weights &lw = m.layers[ph < 5 * L ? ph / 5 : L - 1];
      PhaseRec r = {};
      int N = dim, K = dim;
      QMat a, b, c;
      r.kind = kind;
      if (kind == K_KQV)
        a = qmat (lw.wk, dim, dim), b = qmat (lw.wq, dim, dim), c = qmat (lw.wv, dim, dim);
      else if (kind == K_UPGATE)
        N = ffn, a = c = qmat (lw.w_up, ffn, dim), b = qmat (lw.w_gate, ffn, dim);
      else if (kind == K_DOWN)
        K = ffn, a = b = c = qmat (lw.w_down, dim, ffn);
      else if (kind == K_HEAD)
        N = m.vocab, a = b = c = qmat (m.output, m.vocab, dim);
      else
        a = b = c = qmat (lw.wo, dim, dim);
      r.N = N;
      r.Kp = ((K + 31) >> 5) << 5;
      r.nch = (r.Kp + 4095) / 4096;
      const int nb = r.Kp >> 5;
      r.Q0 = a.q, r.D0 = (const uint8_t *)a.d;
      r.upm = 0x3fffffff;
      if (kind == K_UPGATE)
        {
          // unit u: row u of up, row u of gate
          r.silu = 1;
          r.qs = r.Kp, r.ds = nb * 2;
          r.dq1r = b.q - a.q;
          r.dd1r = (const uint8_t *)b.d - (const uint8_t *)a.d;
        }
      else
        {
          // unit u: rows 2u and 2u + 1 (N is even)
          r.qs = 2 * r.Kp, r.ds = 4 * nb;
          r.dq1r = r.Kp, r.dd1r = nb * 2;
          if (kind == K_KQV)
            {
              r.upm = dim >> 1;
              r.qm1 = b.q - a.q, r.qm2 = c.q - a.q;
              r.dm1 = (const uint8_t *)b.d - (const uint8_t *)a.d;
              r.dm2 = (const uint8_t *)c.d - (const uint8_t *)a.d;
            }
        }
      ((PhaseRec *)p.s.ptab)[ph] = r;
    }
}

template <int HD, bool NT>
int
launch_persistent_as (const Params &p, int n_cu, size_t lds, hipStream_t s)
{
  // per device: the kernel's LDS limit is raised, one workgroup fits a compute unit
  static size_t lds_set[16] = {};
  static int resident[16] = {};
  int dev = 0;
  VKL_HIP (hipGetDevice (&dev));
  VKL_CHECK_ARG (dev >= 0 && dev < 16);
  const void *fn = (const void *)decode_persistent_kernel<HD, NT>;
  if (lds > lds_set[dev])
    {
      VKL_HIP (hipFuncSetAttribute (fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      lds_set[dev] = lds;
      resident[dev] = 0;
    }
  if (resident[dev] == 0)
    {
      int per_cu = 0;
      VKL_HIP (hipOccupancyMaxActiveBlocksPerMultiprocessor (&per_cu, fn, kDecThreads, lds));
      resident[dev] = per_cu < 1 ? -1 : 1;
    }
  // every workgroup waits for all the others: the whole grid must be resident
  if (resident[dev] < 1)
    return (int)hipErrorLaunchOutOfResources;
  const int G = n_cu;
  // a workgroup's results of one phase pass through kOutvBytes of LDS, and one
  // lane of wave 0 writes each unit's results out
  const int umax = std::max (std::max (p.m.vocab / 2 + 1, 3 * (p.m.dim / 2)), p.m.ffn);
  VKL_CHECK_ARG ((size_t)(umax / G + 2) * 4 <= (size_t)kOutvBytes);
  VKL_CHECK_ARG (std::max (3 * (p.m.dim / 2), p.m.ffn) / G + 2 <= 64);
  VKL_CHECK_ARG ((p.m.vocab % 2) == 0 && (p.m.dim % 2) == 0);
  persistent_setup_kernel<<<dim3 (1), dim3 (256), 0, s>>> (p);
  decode_persistent_kernel<HD, NT><<<dim3 ((unsigned)G), dim3 (kDecThreads), lds, s>>> (p, G);
  return vkl_launch_status ();
}
} // namespace

int
launch_persistent (const Params &p, int n_cu, hipStream_t s)
{
  const size_t lds = persist_lds_bytes (p.m.dim, p.m.ffn, p.m.maxlen, p.m.head_dim);
  VKL_CHECK_ARG (lds <= 160 * 1024);
  if (p.m.head_dim == 128)
    return p.stream_once ? launch_persistent_as<128, true> (p, n_cu, lds, s)
                         : launch_persistent_as<128, false> (p, n_cu, lds, s);
  return p.stream_once ? launch_persistent_as<64, true> (p, n_cu, lds, s)
                       : launch_persistent_as<64, false> (p, n_cu, lds, s);
}
} // namespace dec
} // namespace vkl
