// One layer of the decode step as ONE launch.
//
// The launch-per-phase kernels stream at about 6 TB/s while they run, but
// every kernel boundary costs 2.5-3.5 us in which the memory is idle (the end
// of one kernel's tail, the launch gap, the way to the next kernel's first
// bytes): five boundaries on a layer of some 50 us.  Here the G workgroups
// (512 threads, two per compute unit, all resident at once) stay for the five
// phases of a layer and keep the shape of the launch-per-phase kernels: every
// wave computes, a workgroup normalises its own copy of the row with all of
// its threads, two weight items per wave are in flight.  What changes is the
// hand-over between phases:
//
//   results -> memory (stores written through, acknowledged)
//   barrier, ONE arrival per workgroup at the counter of the XCD it runs
//   on; the XCD's last arriver raises the XCD's flag
//   NEXT phase: both weight items of every wave are requested first, so that
//   the memory keeps streaming during everything that follows
//   wave 0 polls the eight flags (bounded); barrier
//   the row is read with ordinary loads, normalised, staged in LDS
//
// Ordinary loads of a row that was written inside the same launch are safe
// because (a) caches are invalidated between launches and no buffer is read
// before it is written inside one launch (the residual stream after the Wo
// projection has a buffer of its own, xm), so no cache holds an older copy of
// a line, and (b) the results are dealt so that every 128-byte line of a row
// is written by workgroups of ONE XCD (see Deal): an L2 has either seen all
// writes to a line or none.  Nothing is assumed about which XCD a workgroup
// lands on: it reads the XCD's number from the hardware register and takes a
// ticket at the XCD's counter, and (XCD, ticket) decide its role and share.
//
// Attention runs on n_heads workgroups (the first to have taken a ticket on
// each XCD), one head each, while the others already hold their Wo weights;
// the heads count in at one counter and the last one raises a flag per XCD.
//
// Flags carry the number of the launch (a word in the sync area that
// workgroup 0 advances at the end of every launch), counters are zeroed by
// their last arriver: nothing has to be cleared between launches.  Every wait
// is bounded; a workgroup whose wait gave up marks the error word that
// vkl_decode_status reports, keeps counting in (so that nobody else waits for
// it in vain) and drops its results into a sink instead of storing them.  The
// error word names the first cause: 0x100 | stage for a wait that gave
// up, 0x200 | xcd for an XCD that was dealt more than its share of workgroups.
#include "vkl_decode_gemv.h"
#include "vkl_decode_shared.h"
#include <algorithm>

namespace vkl
{
namespace dec
{
namespace
{
// words of the layer-sync area (Scratch::lsync); every counter and flag on a
// 128-byte line of its own
constexpr int kLsLaunch = 0;              // launches completed so far
constexpr int kLsCnt = 32;                // + (stage * 8 + slot) * 32
constexpr int kLsTicket = kLsCnt + 4 * 8 * 32; // + slot * 32: workgroups of the XCD that have started
// (the flags, (stage * 8 + slot) * 32 words into vkl_decode_model::flags, are
// polled through the scalar memory path and live in memory no cache holds)
static_assert ((kLsTicket + 8 * 32) * 4 <= kLayerSyncBytes, "layer-sync area too small");
constexpr int kSyncErr = 1; // word of Scratch::sync: a wait gave up
constexpr int kLayerSpinLimit = 1 << 14;
// The last wave of a workgroup is its courier.  A wave's loads return in
// order, so a poll or a row read issued behind two weight items would wait
// for those 16 KiB to arrive from a memory that has 60 MB of requests queued.
// The courier therefore requests no weights ahead: it counts the workgroup
// in, polls, brings the row into LDS, and only then streams its own (the
// workgroup's last) units while the other waves are at their later items.
constexpr int kCourier = kDecWaves - 1;
// Weight items a worker requests before the wait for the previous phase.  The
// memory path of a compute unit serves requests in order, also across waves:
// the courier's polls and the row queue behind whatever the 14 workers of the
// compute unit have requested, so the look-ahead is what the wait can hide
// (one item: 116 KiB per compute unit, some 4 us at the rate a compute unit
// is served), not everything the registers can hold.
#ifndef VKL_LAYER_AHEAD
#define VKL_LAYER_AHEAD 2
#endif
constexpr int kAhead = VKL_LAYER_AHEAD;
// The first up/gate item of a wave is requested when the attention output has
// arrived (0) or already together with the Wo item, while the heads are being
// computed (1).  The early request fills the memory's idle time, but the
// heads share compute units with workgroups that request, and a compute
// unit's memory path is served in order: their polls and cache rows queue
// behind those items.
#ifndef VKL_LAYER_UP_EARLY
#define VKL_LAYER_UP_EARLY 1
#endif
#define VKL_LDS __attribute__ ((address_space (3)))

enum Stage
{
  ST_KQV = 0,
  ST_ATT,
  ST_WO,
  ST_UP
};

// the error word keeps the FIRST cause reported since the host last looked
__device__ __forceinline__ void
report (uint32_t *err, uint32_t code)
{
  uint32_t expected = 0u;
  __hip_atomic_compare_exchange_strong (err, &expected, code, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                        __HIP_MEMORY_SCOPE_AGENT);
}

// counts the workgroup in at `cnt` once its stores have been acknowledged;
// the last of `n` arrivals zeroes the counter and raises `nflags` flags
__device__ __forceinline__ void
arrive (uint32_t *cnt, uint32_t n, uint32_t *flag, int nflags, uint32_t mark, bool silent)
{
  __builtin_amdgcn_s_waitcnt (0x0f70); // vmcnt(0)
  __syncthreads ();
  // (the courier counts in: the other waves go on to request the next phase's
  // weights instead of waiting for the counter's answer; they wait for the
  // second barrier so that the atomic enters the compute unit's memory path,
  // which is served in order, ahead of those requests)
  uint32_t old = 0;
  const bool courier = __builtin_amdgcn_readfirstlane ((int)(threadIdx.x >> 6)) == kCourier;
  const int lane = (int)threadIdx.x & 63;
  if (courier && lane == 0)
    old = __hip_atomic_fetch_add (cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __builtin_amdgcn_s_barrier ();
  if (courier)
    {
      old = (uint32_t)__builtin_amdgcn_readfirstlane ((int)old);
      if (old + 1u == n)
        {
          if (lane == 0)
            st_coherent_u32 (cnt, 0u);
          if (lane < nflags && !silent)
            st_coherent_u32 (flag + 32 * lane, mark);
        }
    }
}

// The courier polls `nflags` flags (1 or 8, 32 words apart) until all carry
// `mark` (bounded), then brings the row of K fp16 values straight into LDS
// (every lane 16 bytes per load, a load fills 1 KiB of consecutive LDS; the
// tail of the last KiB repeats the row's last 16 bytes and lands in unused
// LDS behind the row).  Ends with a barrier.  False: the wait gave up (the
// error word is set, the row is not there).
template <bool COURIER>
__device__ __forceinline__ bool
courier_fetch (bool poll, const uint32_t *flag, int nflags, uint32_t mark, int limit,
               uint32_t *err, uint32_t *lds_word, uint32_t code, const uint16_t *src, int K,
               uint8_t *xl, const float *norm_w = nullptr, int norm_n = 0, uint8_t *norm_lds = nullptr,
               unsigned long long *tr = nullptr)
{
  if (COURIER)
    {
      const int lane = (int)threadIdx.x & 63;
      // (norm weights do not depend on anybody: they travel while this wave polls)
      if (norm_w)
        for (int i = 0; i < (norm_n * 4 + 1023) >> 10; ++i)
          {
            const int off = min (i * 1024 + lane * 16, norm_n * 4 - 16);
            __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)((const uint8_t *)norm_w + off),
                                              (VKL_LDS void *)(norm_lds + i * 1024), 16, 0, 0);
          }
      bool ok = !poll;
      if (poll)
        {
          for (int spin = 0; spin < limit; ++spin)
            {
              if (flags_equal_scalar (flag, nflags, mark))
                {
                  ok = true;
                  break;
                }
              __builtin_amdgcn_s_sleep (1);
            }
        }
#ifdef VKL_TRACE
      if (tr && lane == 0)
        tr[0] = wall_clock64 ();
#endif
      if (ok)
        {
          const int bytes = K * 2, n = (bytes + 1023) >> 10;
          for (int i = 0; i < n; ++i)
            {
              const int off = min (i * 1024 + lane * 16, bytes - 16);
              __builtin_amdgcn_global_load_lds ((const VKL_GLOBAL void *)((const uint8_t *)src + off),
                                                (VKL_LDS void *)(xl + i * 1024), 16, 0, 0);
            }
        }
      __builtin_amdgcn_s_waitcnt (0x0f70); // vmcnt(0)
#ifdef VKL_TRACE
      if (tr && lane == 0)
        tr[1] = wall_clock64 ();
#endif
      if (lane == 0)
        {
          *lds_word = ok ? 1u : 0u;
          if (!ok)
            report (err, code);
        }
    }
  __syncthreads ();
  return *lds_word != 0u;
}

// the plain wait of the head workgroups (they hold no weights)
__device__ __forceinline__ bool
wait_flags (const uint32_t *flag, int nflags, uint32_t mark, int limit, uint32_t *err,
            uint32_t *lds_word, uint32_t code)
{
  if (threadIdx.x < 64)
    {
      bool ok = false;
      for (int spin = 0; spin < limit; ++spin)
        {
          if (flags_equal_scalar (flag, nflags, mark))
            {
              ok = true;
              break;
            }
          __builtin_amdgcn_s_sleep (1);
        }
      if (threadIdx.x == 0)
        {
          *lds_word = ok ? 1u : 0u;
          if (!ok)
            report (err, code);
        }
    }
  __syncthreads ();
  return *lds_word != 0u;
}

// norm weights as the courier left them in LDS
template <int XCH>
__device__ __forceinline__ void
norm_from_lds (const uint8_t *nl, int K, NormRegs &n)
{
#pragma unroll
  for (int j = 0; j < XCH; ++j)
    {
      const int idx = min ((int)threadIdx.x + j * kDecThreads, (K >> 3) - 1);
      n.w[j][0] = ((const uint4 *)nl)[2 * idx];
      n.w[j][1] = ((const uint4 *)nl)[2 * idx + 1];
    }
}

// the row as the courier left it in LDS, into the registers stage_row expects
template <int XCH>
__device__ __forceinline__ void
row_from_lds (const uint16_t *xl, int K, XRegs &x)
{
#pragma unroll
  for (int j = 0; j < XCH; ++j)
    {
      const int idx = min ((int)threadIdx.x + j * kDecThreads, (K >> 3) - 1);
      x.v[j] = ((const uint4 *)xl)[idx];
    }
}

struct LayerCtx
{
  uint32_t *ls, *err, *word, *flags;
  uint32_t mark;
  int limit, n_slot, slot, idx, nh, wg, G, layer;
  bool silent;
};

__device__ __forceinline__ uint32_t *
cnt_of (const LayerCtx &c, int stage, int k)
{
  return c.ls + kLsCnt + (stage * 8 + k) * 32;
}

__device__ __forceinline__ uint32_t *
flag_of (const LayerCtx &c, int stage, int k)
{
  return c.flags + (stage * 8 + k) * 32;
}

#ifdef VKL_TRACE
#define VKL_TL(slot_)                                                          \
  if (threadIdx.x == 0 && p.trace)                                             \
    p.trace[((size_t)layer * 1024 + wg) * 16 + (slot_)] = wall_clock64 ();
#else
#define VKL_TL(slot_)
#endif

// A layer from the attention on, for the workers (COURIER false) or for the
// courier of the workgroup: the same barriers in the same order in both.
//
// The two item buffers are handed from phase to phase so that the memory has
// work during the attention and no wave waits for a third up/gate item with
// nothing else to do: the Wo projection takes two-row units (a wave then has
// one item, rarely two) and runs them through buffer A alone; buffer B
// receives the wave's FIRST up/gate item together with the Wo item, i.e.
// while the heads are computed and the memory would otherwise idle; A takes
// the second up/gate item as soon as the Wo product has left it.  When the
// residual row arrives both are there, and the third item travels while the
// second is multiplied.
template <int WT, int XD, int XF, bool NT, bool COURIER>
__device__ __forceinline__ void
layer_tail (const Params &p, const vkl_layer_weights &lw, const LayerCtx &c, uint8_t *lds)
{
  typedef Gemv<WT, NT, 2> GV2;    // up/gate: two-row units
  typedef Gemv<WT, false, 2> GVO; // Wo: two-row units, plain loads (short phase)
  typedef Gemv<WT, NT, 1> GVD;    // down
  const vkl_decode_model &m = p.m;
  const int dim = m.dim, ffn = m.ffn, wg = c.wg, G = c.G, slot = c.slot, idx = c.idx;
  const int layer = c.layer;
  (void)layer;
  uint16_t *xl = (uint16_t *)lds;
  bool live = true; // false once a wait of this workgroup gave up
  Epilogue e = {};
  XRegs x;
  NormRegs nw;
  PipeState ps, pu; // pu: the up/gate product, begun during the Wo phase
  PipeBuf A, B;
  const QMat up = wmat<WT> (lw.w_up, ffn, dim), gate = wmat<WT> (lw.w_gate, ffn, dim);
  const Deal deal_up = Deal{ 1, slot, idx, c.n_slot };
  // where the norm weights of the up/gate phase are parked (behind the staged
  // row and the reduction words)
  uint8_t *norm_lds = lds + lds_norm_offset (dim, ffn);
  // heads h = slot, slot + 8, ... run on the first workgroups of XCD `slot`
  const int n_heads_here = (c.nh - slot + 7) >> 3;
  if (idx < n_heads_here)
    {
      // ---- one head of the attention ---------------------------------------
      // (the cached K and V rows are requested before the wait for this
      // token's q, k and v: they do not depend on it)
      auto wait_kqv = [&] () {
        live = wait_flags (flag_of (c, ST_KQV, 0), 8, c.mark, c.limit, c.err, c.word, 0x100u | ST_KQV);
        VKL_TL (4)
        return live;
      };
      if (m.head_dim == 128)
        attention_head<128, true, true> (p, lw, idx * 8 + slot, lds, nullptr, wait_kqv);
      else
        attention_head<64, true, true> (p, lw, idx * 8 + slot, lds, nullptr, wait_kqv);
      VKL_TL (5)
      arrive (cnt_of (c, ST_ATT, 0), (uint32_t)c.nh, flag_of (c, ST_ATT, 0), 8, c.mark, c.silent);
      arrive (cnt_of (c, ST_WO, slot), (uint32_t)c.n_slot, flag_of (c, ST_WO, slot), 1, c.mark, false);
      VKL_TL (6)
      if (!COURIER)
        GV2::begin (pu, B, A, 2, up, gate, up, ffn, dim, wg, G, 2, nullptr, true, deal_up);
    }
  else
    {
      // ---- Wo + residual -> xm ---------------------------------------------
      const QMat w = wmat<WT> (lw.wo, dim, dim);
      const Deal dl = Deal{ 1, slot, idx - n_heads_here, c.n_slot - n_heads_here };
      if (!COURIER)
        {
          GVO::begin (ps, A, B, 0, w, w, w, dim, dim, wg, G, 1, p.s.x, true, dl);
          if (VKL_LAYER_UP_EARLY)
            GV2::begin (pu, B, A, 2, up, gate, up, ffn, dim, wg, G, 1, nullptr, true, deal_up);
        }
      live = courier_fetch<COURIER> (true, flag_of (c, ST_ATT, slot), 1, c.mark, c.limit,
                                     c.err, c.word, 0x100u | ST_ATT, p.s.att, dim, lds, lw.ffn_norm,
                                     dim, norm_lds);
      if (COURIER)
        GVO::begin (ps, A, B, 0, w, w, w, dim, dim, wg, G, 1, p.s.x, true, dl);
      else if (!VKL_LAYER_UP_EARLY)
        GV2::begin (pu, B, A, 2, up, gate, up, ffn, dim, wg, G, 1, nullptr, true, deal_up);
      VKL_TL (4)
      e = Epilogue{};
      e.y[0] = live ? p.s.xm : p.s.sink, e.residual = p.s.x;
      e.through = true;
      GVO::run_single (ps, A, xl, e);
      VKL_TL (5)
      arrive (cnt_of (c, ST_WO, slot), (uint32_t)c.n_slot, flag_of (c, ST_WO, slot), 1, c.mark, false);
      VKL_TL (6)
      // (after the arrival: it waits for everything the wave has in flight)
      if (!COURIER)
        GV2::issue (pu, A, 1), pu.primed = 2;
    }

  // ---- RMSNorm + up/gate with SiLU -> t -------------------------------------
  {
    float *red = (float *)(lds + (size_t)dim * 2);
    // (a head's workgroup had its LDS in use until now: it fetches the norm weights here)
    const bool head = idx < n_heads_here;
    live = courier_fetch<COURIER> (true, flag_of (c, ST_WO, 0), 8, c.mark, c.limit, c.err, c.word,
                                   0x100u | ST_WO, p.s.xm, dim, lds, head ? lw.ffn_norm : nullptr, dim,
                                   norm_lds)
           && live;
    VKL_TL (7)
    norm_from_lds<XD> (norm_lds, dim, nw);
    row_from_lds<XD> (xl, dim, x);
    stage_row<true, XD> (x, dim, xl, nw, m.eps, red, nullptr);
    VKL_TL (8)
    // (the courier's requests come after the barriers of the staging: a wave
    // that waits for room in the memory path would hold up the other seven)
    if (COURIER)
      GV2::begin (pu, B, A, 2, up, gate, up, ffn, dim, wg, G, 2, nullptr, true, deal_up);
    e = Epilogue{};
    e.y[0] = live ? p.s.t : p.s.sink;
    e.through = true;
    GV2::run (pu, B, A, xl, e, red);
    VKL_TL (9)
    arrive (cnt_of (c, ST_UP, slot), (uint32_t)c.n_slot, flag_of (c, ST_UP, slot), 1, c.mark, false);
    VKL_TL (10)
  }

  // ---- down + residual -> x ---------------------------------------------------
  {
    const QMat w = wmat<WT> (lw.w_down, dim, ffn);
    float *red = (float *)(lds + (size_t)ffn * 2);
    if (!COURIER)
      GVD::begin (ps, A, B, 0, w, w, w, dim, ffn, wg, G, kAhead, p.s.xm, true);
    live = courier_fetch<COURIER> (true, flag_of (c, ST_UP, 0), 8, c.mark, c.limit, c.err, c.word,
                                   0x100u | ST_UP, p.s.t, ffn, lds)
           && live;
    if (COURIER)
      GVD::begin (ps, A, B, 0, w, w, w, dim, ffn, wg, G, 2, p.s.xm, true);
    else if (kAhead < 2)
      GVD::issue (ps, B, 1), ps.primed = 2;
    VKL_TL (11)
    e = Epilogue{};
    e.y[0] = live ? p.s.x : p.s.sink, e.residual = p.s.xm;
    GVD::run (ps, A, B, xl, e, red);
    VKL_TL (13)
  }
}

// XD / XF: 4096-element chunks of a row of dim / ffn values
template <int WT, int XD, int XF, bool NT>
__global__ __launch_bounds__ (kDecThreads) __attribute__ ((amdgpu_waves_per_eu (4, 4))) void
decode_layer_kernel (const Params p, const vkl_layer_weights lw, int layer, int G,
                     size_t lds_word_at)
{
  extern __shared__ __align__ (16) uint8_t lds[];
  typedef Gemv<WT, NT, 2> GV2; // K/Q/V: two-row units
  const vkl_decode_model &m = p.m;
  const int dim = m.dim, nh = m.n_heads;
  const int wg = (int)blockIdx.x;
  uint32_t *ls = p.s.lsync;
  uint32_t *err = p.s.sync + kSyncErr;
  uint32_t *word = (uint32_t *)(lds + lds_word_at); // [0] wait result, [1] XCD, [2] ticket
  uint16_t *xl = (uint16_t *)lds;
  const bool silent = m.wait_test != 0;
  // the number of this launch; flags raised in it carry it
  const uint32_t mark = ld_coherent_u32 (ls + kLsLaunch) + 1u;
  // once a wait has given up the step is lost anyway: the launches that
  // follow until the host has looked do not wait at all
  const int limit
      = ld_coherent_u32 (err) != 0u ? 1 : (m.wait_polls > 0 ? m.wait_polls : kLayerSpinLimit);
  // Where this workgroup runs, and its number among the workgroups of that
  // XCD in order of arrival: nothing is assumed about how the dispatcher
  // deals workgroups to XCDs except that each gets G / 8 of them (if not, a
  // counter below never fills up and the bounded waits report it).
  const int n_slot = G >> 3;
  uint32_t xcc = 0, ticket = 0;
  if (threadIdx.x == 0)
    {
      xcc = __builtin_amdgcn_s_getreg (20 | (0 << 6) | (3 << 11)) & 7u;
      ticket = __hip_atomic_fetch_add (ls + kLsTicket + 32 * xcc, 1u, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
    }
  VKL_TL (0)
  Epilogue e = {};
  XRegs x;
  NormRegs nw;
  PipeState ps;
  PipeBuf A, B;
  // (a scalar: branches on it are wave-uniform)
  const bool courier = __builtin_amdgcn_readfirstlane ((int)(threadIdx.x >> 6)) == kCourier;
  int slot = 0, idx = 0;
  // (after a barrier that follows the store below)
  auto place = [&] () {
    slot = __builtin_amdgcn_readfirstlane ((int)word[1]);
    idx = __builtin_amdgcn_readfirstlane ((int)word[2]);
    if (idx >= n_slot && threadIdx.x == 0)
      report (err, 0x200u | (uint32_t)slot);
  };

  {
    // ---- RMSNorm + K/Q/V -------------------------------------------------
    const QMat wk = wmat<WT> (lw.wk, dim, dim), wq = wmat<WT> (lw.wq, dim, dim),
               wv = wmat<WT> (lw.wv, dim, dim);
    float *red = (float *)(lds + (size_t)dim * 2);
    load_row<XD> (p.s.x, dim, x);
    load_norm<XD> (lw.attn_norm, dim, nw);
    __builtin_amdgcn_sched_barrier (0);
    GV2::begin (ps, A, B, 1, wk, wq, wv, dim, dim, wg, G, 1, nullptr, true);
    if (threadIdx.x == 0)
      word[1] = xcc, word[2] = ticket;
    stage_row<true, XD> (x, dim, xl, nw, m.eps, red, nullptr);
    VKL_TL (1)
    place ();
    e = Epilogue{};
    e.y[0] = p.s.kqv, e.y[1] = p.s.kqv + dim, e.y[2] = p.s.kqv + 2 * dim;
    e.through = true;
    GV2::run (ps, A, B, xl, e, red);
    VKL_TL (2)
    arrive (ls + kLsCnt + (ST_KQV * 8 + slot) * 32, (uint32_t)n_slot,
            (uint32_t *)m.flags + (ST_KQV * 8 + slot) * 32, 1, mark, false);
    VKL_TL (3)
  }
#ifdef VKL_TRACE
  if (threadIdx.x == 0 && p.trace)
    {
      p.trace[((size_t)layer * 1024 + wg) * 16 + 12] = __builtin_amdgcn_s_getreg (4 | (0 << 6) | (31 << 11));
      p.trace[((size_t)layer * 1024 + wg) * 16 + 14] = (unsigned)idx | (unsigned)slot << 16;
    }
#endif
  const LayerCtx c = { ls, err, word, (uint32_t *)m.flags, mark, limit, n_slot, slot, idx, nh, wg, G, layer, silent };
  // the courier's path is a copy of the workers' (the branch is wave-uniform):
  // in one copy, with the courier's weight requests under a condition, the
  // item buffers of the two roles collide and spill
  if (courier)
    layer_tail<WT, XD, XF, NT, true> (p, lw, c, lds);
  else
    layer_tail<WT, XD, XF, NT, false> (p, lw, c, lds);
  // (every workgroup has read the launch number and taken its ticket before
  // its first arrival, and this one has seen all of them arrive)
  if (wg == 0 && threadIdx.x < 9)
    st_coherent_u32 (threadIdx.x == 8 ? ls + kLsLaunch : ls + kLsTicket + 32 * (int)threadIdx.x,
                     threadIdx.x == 8 ? mark : 0u);
}

// the token's embedding row as the start of the residual stream
template <int WT>
__global__ __launch_bounds__ (kDecThreads) void
embed_row_kernel (const Params p)
{
  embed_row<WT> (p, ldg (step_tok (p)), (int)blockIdx.x, (int)gridDim.x);
}

template <int WT, int XD, int XF, bool NT>
int
launch_layer_t (const Params &p, const vkl_layer_weights &lw, int layer, int G,
                hipStream_t s)
{
  const size_t at = (lds_bytes_needed (p.m.dim, p.m.ffn, p.m.maxlen, p.m.head_dim) + 15) & ~(size_t)15;
  const size_t lds = at + 16;
  static LdsLimit limit;
  if (int e = limit.raise ((const void *)decode_layer_kernel<WT, XD, XF, NT>, lds))
    return e;
  decode_layer_kernel<WT, XD, XF, NT>
      <<<dim3 ((unsigned)G), dim3 (kDecThreads), lds, s>>> (p, lw, layer, G, at);
  return 0;
}

template <int WT, int XD, int XF>
int
launch_layer_x (const Params &p, const vkl_layer_weights &lw, int layer, int G,
                hipStream_t s)
{
  return p.stream_once ? launch_layer_t<WT, XD, XF, true> (p, lw, layer, G, s)
                       : launch_layer_t<WT, XD, XF, false> (p, lw, layer, G, s);
}

template <int WT>
int
launch_layer_wt (const Params &p, const vkl_layer_weights &lw, int layer, int G,
                 hipStream_t s)
{
  const int xd = (p.m.dim + 4095) / 4096, xf = (p.m.ffn + 4095) / 4096;
  if (xd == 1 && xf == 1)
    return launch_layer_x<WT, 1, 1> (p, lw, layer, G, s);
  if (xd == 1 && xf <= 3)
    return launch_layer_x<WT, 1, 3> (p, lw, layer, G, s);
  return launch_layer_x<WT, 2, 4> (p, lw, layer, G, s);
}
} // namespace

bool
layer_launch_supported (const vkl_decode_model &m, int G)
{
  // rows of up to two (dim) and four (ffn) chunks of 4096; every slot needs
  // workgroups beside the heads; two workgroups per compute unit must fit
  return m.flags != nullptr && m.dim <= 8192 && m.ffn <= 16384 && (m.dim % 8) == 0 && (m.ffn % 8) == 0
         && G >= m.n_heads + 8 && (G % 8) == 0
         && 2 * (lds_bytes_needed (m.dim, m.ffn, m.maxlen, m.head_dim) + 32) <= 160 * 1024;
}

int
launch_layer (const Params &p, const vkl_layer_weights &lw, int layer, int G,
              hipStream_t s)
{
  return p.m.wtype == 8 ? launch_layer_wt<8> (p, lw, layer, G, s)
                        : launch_layer_wt<1> (p, lw, layer, G, s);
}

int
launch_embed_row (const Params &p, hipStream_t s)
{
  const int grid = std::max (1, std::min (8, p.m.dim / (kDecThreads * 8)));
  if (p.m.wtype == 8)
    embed_row_kernel<8><<<dim3 ((unsigned)grid), dim3 (kDecThreads), 0, s>>> (p);
  else
    embed_row_kernel<1><<<dim3 ((unsigned)grid), dim3 (kDecThreads), 0, s>>> (p);
  return 0;
}
} // namespace dec
} // namespace vkl
