// Fused one-token decode step for Llama-2-shaped models with Q8_0 weights.
//
// Work decomposition: a grid of G workgroups of 512 threads (8 waves), two
// per compute unit (one per compute unit in the persistent mode).  In a
// projection phase the output rows are grouped into units: 2 rows (K/Q/V,
// the output layer), an up row and the gate row that pairs with it (the
// fused up/gate product), or 1 row (Wo and down, whose rows are few and long:
// every wave then has a unit).  Workgroup g owns a contiguous range of units,
// so it streams one contiguous span of each int8 plane, and wave w of the
// group takes every 8th unit.  Lane l of a wave handles the 16 quants at
// k = step*1024 + 16*l of a row (one dwordx4 load = half a Q8_0 block).
//
// A wave's work is a sequence of items (one unit x one K chunk, 8 dwordx4
// loads per lane) that runs through a two-deep register pipeline: the loads of
// item i+1 are in flight while item i is multiplied, and the first item of a
// phase is issued BEFORE the activation vector is staged (its weights do not
// depend on the activations), which takes the activation latency off the
// critical path.  The activation vector sits in LDS as fp16, with the RMSNorm
// folded into the staging where a phase starts with one.  Attention runs one
// workgroup per head with the first cache rows prefetched the same way.
//
// Every phase is HBM-bound: 34 bytes per 32 weights are read exactly once, the
// activations (a few KiB) come from L2.
#include "../../include/vkl_decode.h"
#include "vkl_decode_shared.h"
#include "vkl_decode_gemv.h"
#include <algorithm>
#include <stdio.h>
#include <stdlib.h>
#include <vector>

namespace vkl
{
using namespace dec;
namespace
{
// contexts from this length on run the split form of the attention phase
inline int
attn_split_min (const vkl_decode_model &m)
{
  return m.attn_split_min == 0 ? kAttnSplitMinLen : std::max (m.attn_split_min, 2);
}
// words of the sync area for the fused attention + Wo launch: a counter of the
// heads whose attention output is in memory, and eight flags (one per
// workgroup index mod 8, i.e. per XCD) that the last head sets and the
// projection's workgroups poll (polling the counter itself from every
// workgroup held up the heads' atomics); all zeroed by the layer's K/Q/V phase
// (each on a cache line of its own, clear of the words the persistent mode uses)
constexpr int kSyncAttnDone = 32;
constexpr int kSyncHeadDone = 64; // workgroups of the lm_head launch whose arg-max partials are in memory
constexpr int kAttnFlagGroup = 4;  // group of vkl_decode_model::flags, + 32 * slot
constexpr int kFuseSpinLimit = 1 << 13; // some 10 ms; a head takes microseconds

// the lm_head launch ends with the arg-max (not when a sampler follows it)
__host__ __device__ __forceinline__ bool
head_picks_token (const Params &p)
{
  return (p.next_tok || p.loop) && !p.sample;
}

__device__ __forceinline__ void
reset_attn_done (const Params &p, int wg)
{
  if (wg == 0 && threadIdx.x < 9)
    {
      if (threadIdx.x == 8)
        st_coherent_u32 (p.s.sync + kSyncAttnDone, 0u);
      else if (p.m.flags)
        st_coherent_u32 ((uint32_t *)p.m.flags + kAttnFlagGroup * kFlagGroupWords + 32 * (int)threadIdx.x, 0u);
    }
}


// ---------------------------------------------------------------------------
// phases
// ---------------------------------------------------------------------------
enum Phase
{
  PH_KQV = 0,
  PH_ATTN,
  PH_WO,
  PH_UPGATE,
  PH_DOWN,
  PH_HEAD,
  PH_ARGMAX,
  PH_GEMV, // a stand-alone y = W x (+ residual) on the down projection's path
  PH_LAYER // a whole layer in one launch (vkl_decode_layer.hip)
};

// ---------------------------------------------------------------------------
// one phase of the step in its general form
// ---------------------------------------------------------------------------
// Used for the phases that do not have (or need) the branch-free form below:
// the K/Q/V projection of layer 0 (which embeds the token), attention with
// one workgroup per head, the final arg-max, and every phase of a model
// whose rows exceed what the direct kernels stage.  Every projection phase
// runs in this order: activation loads, norm-weight loads, first weight item
// (all issued back to back), then the activation is normalised / written to
// LDS, then the weight pipeline runs.
template <int WT = 8>
__device__ __forceinline__ void
run_phase (const Params &p, const vkl_layer_weights &lw, int layer, int phase,
           int wg, int G, uint8_t *lds)
{
  typedef Gemv<WT> GV;
  const vkl_decode_model &m = p.m;
  const int dim = m.dim, ffn = m.ffn;
  uint16_t *xl = (uint16_t *)lds;
  const int kstage = phase == PH_DOWN || phase == PH_GEMV ? ffn : dim;
  float *red = (float *)(lds + (size_t)kstage * 2); // 2*kDecWaves words
  Epilogue e = {};
  XRegs x;
  NormRegs nw;
  PipeState ps;
  PipeBuf A, B;
  VKL_TR (0);
  switch (phase)
    {
    case PH_KQV:
      {
        const QMat wk = wmat<WT> (lw.wk, dim, dim), wq = wmat<WT> (lw.wq, dim, dim),
                   wv = wmat<WT> (lw.wv, dim, dim);
        if (layer == 0)
          {
            uint32_t tok = ldg (step_tok (p));
            if (tok >= (uint32_t)m.vocab)
              tok = 0;
            if (WT == 8)
              issue_embed_q8 (wmat<WT> (m.tok_embd, m.vocab, dim), tok, dim, x);
            else
              issue_x ((const uint16_t *)m.tok_embd + (size_t)tok * dim, dim, x);
          }
        else
          issue_x (p.s.x, dim, x);
        issue_norm (lw.attn_norm, dim, nw);
        GV::begin (ps, A, B, 1, wk, wq, wv, dim, dim, wg, G, 1);
        if (layer == 0)
          {
            if (WT == 8)
              dequant_embed (x);
            if (wg == 0) // the residual stream starts as the embedding row
              {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                  {
                    const int idx = threadIdx.x + j * kDecThreads;
                    if (idx * 8 < dim)
                      {
                        uint32_t *dst = (uint32_t *)p.s.x + idx * 4;
                        stg (dst, x.v[j].x);
                        stg (dst + 1, x.v[j].y);
                        stg (dst + 2, x.v[j].z);
                        stg (dst + 3, x.v[j].w);
                      }
                  }
              }
          }
        finish_x<true> (x, dim, xl, nw, m.eps, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.kqv, e.y[1] = p.s.kqv + dim, e.y[2] = p.s.kqv + 2 * dim;
        GV::run (ps, A, B, xl, e, red);
        reset_attn_done (p, wg);
        break;
      }
    case PH_ATTN:
      {
        for (int h = wg; h < m.n_heads; h += G)
          {
            if (m.head_dim == 128)
              attention_head<128, false> (p, lw, h, lds, VKL_TRP);
            else
              attention_head<64, false> (p, lw, h, lds, VKL_TRP);
          }
        break;
      }
    case PH_WO:
      {
        const QMat w = wmat<WT> (lw.wo, dim, dim);
        issue_x (p.s.att, dim, x);
        GV::begin (ps, A, B, 0, w, w, w, dim, dim, wg, G, 1, p.s.x);
        finish_x<false> (x, dim, xl, nw, 0.f, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.x, e.residual = p.s.x;
        GV::run (ps, A, B, xl, e, red);
        break;
      }
    case PH_UPGATE:
      {
        const QMat up = wmat<WT> (lw.w_up, ffn, dim), gate = wmat<WT> (lw.w_gate, ffn, dim);
        issue_x (p.s.x, dim, x);
        issue_norm (lw.ffn_norm, dim, nw);
        GV::begin (ps, A, B, 2, up, gate, up, ffn, dim, wg, G, 1);
        finish_x<true> (x, dim, xl, nw, m.eps, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.t;
        GV::run (ps, A, B, xl, e, red);
        break;
      }
    case PH_DOWN:
      {
        const QMat w = wmat<WT> (lw.w_down, dim, ffn);
        issue_x (p.s.t, ffn, x);
        GV::begin (ps, A, B, 0, w, w, w, dim, ffn, wg, G, 1, p.s.x);
        finish_x<false> (x, ffn, xl, nw, 0.f, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.x, e.residual = p.s.x;
        GV::run (ps, A, B, xl, e, red);
        break;
      }
    case PH_GEMV:
      {
        // y[dim] = W[dim, ffn] x[ffn] (+ residual) for a caller's operands:
        // x in s.t, y in s.x, W in w_down
        const QMat w = wmat<WT> (lw.w_down, dim, ffn);
        issue_x (p.s.t, ffn, x);
        GV::begin (ps, A, B, 0, w, w, w, dim, ffn, wg, G, 1, p.gemv_res);
        finish_x<false> (x, ffn, xl, nw, 0.f, red, VKL_TRP);
        e.y[0] = p.s.x, e.residual = p.gemv_res;
        GV::run (ps, A, B, xl, e, red);
        break;
      }
    case PH_HEAD:
      {
        const QMat w = wmat<WT> (m.output, m.vocab, dim);
        issue_x (p.s.x, dim, x);
        issue_norm (m.output_norm, dim, nw);
        GV::begin (ps, A, B, 0, w, w, w, m.vocab, dim, wg, G, 1);
        finish_x<true> (x, dim, xl, nw, m.final_eps, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.logits16, e.y32 = p.logits32;
        e.amax_val = p.s.amax_val, e.amax_idx = p.s.amax_idx;
        GV::run (ps, A, B, xl, e, red);
        break;
      }
    default: // (PH_ARGMAX: the lm_head launch picks the token itself)
      break;
    }
  VKL_TR (4);
}

// ---------------------------------------------------------------------------
// the projection phases of the launch-per-phase mode, without a branch between
// the first load and the staged row (see load_row): row, norm weights, first
// weight item, then normalisation and staging, then the weight pipeline.
// Layer 0's K/Q/V phase, which starts from the embedding table, keeps the
// general form above.
// ---------------------------------------------------------------------------
template <int PHASE, int WT, int XCH, bool NT>
__device__ __forceinline__ void
run_phase_direct (const Params &p, const vkl_layer_weights &lw, int layer,
                  int wg, int G, uint8_t *lds)
{
  // NT: the weights stream past once per token and do not fit the caches.
  // Read with the non-temporal hint they arrive about a tenth faster in the
  // long phases (the short Wo phase measured slower with it and keeps plain
  // loads).  Weights that fit the caches must not carry the hint: it would
  // keep them from staying there for the next token.
  // Wo, down and the stand-alone product have few rows (two-row units would
  // leave half of the waves without work): one row per unit there
  typedef Gemv<WT, NT && PHASE != PH_WO,
               PHASE == PH_DOWN || PHASE == PH_GEMV || PHASE == PH_WO ? 1 : 2>
      GV;
  constexpr int phase = PHASE;
  const vkl_decode_model &m = p.m;
  const int dim = m.dim, ffn = m.ffn;
  uint16_t *xl = (uint16_t *)lds;
  const int kstage = phase == PH_DOWN || phase == PH_GEMV ? ffn : dim;
  float *red = (float *)(lds + (size_t)kstage * 2); // 2*kDecWaves words
  Epilogue e = {};
  XRegs x;
  NormRegs nw;
  PipeState ps;
  PipeBuf A, B;
  VKL_TR (0);
  switch (phase)
    {
    case PH_KQV:
      {
        const QMat wk = wmat<WT> (lw.wk, dim, dim), wq = wmat<WT> (lw.wq, dim, dim),
                   wv = wmat<WT> (lw.wv, dim, dim);
        load_row<XCH> (p.s.x, dim, x);
        load_norm<XCH> (lw.attn_norm, dim, nw);
        // keep the scheduler from moving the row / norm loads behind the weight
        // loads: waiting for them would then wait for the weights as well
        __builtin_amdgcn_sched_barrier (0);
        GV::begin (ps, A, B, 1, wk, wq, wv, dim, dim, wg, G, 1, nullptr, true);
        stage_row<true, XCH> (x, dim, xl, nw, m.eps, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.kqv, e.y[1] = p.s.kqv + dim, e.y[2] = p.s.kqv + 2 * dim;
        reset_attn_done (p, wg);
        break;
      }
    case PH_WO:
      {
        const QMat w = wmat<WT> (lw.wo, dim, dim);
        load_row<XCH> (p.s.att, dim, x);
        // keep the scheduler from moving the row / norm loads behind the weight
        // loads: waiting for them would then wait for the weights as well
        __builtin_amdgcn_sched_barrier (0);
        GV::begin (ps, A, B, 0, w, w, w, dim, dim, wg, G, 1, p.s.x, true);
        stage_row<false, XCH> (x, dim, xl, nw, 0.f, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.x, e.residual = p.s.x;
        break;
      }
    case PH_UPGATE:
      {
        const QMat up = wmat<WT> (lw.w_up, ffn, dim), gate = wmat<WT> (lw.w_gate, ffn, dim);
        load_row<XCH> (p.s.x, dim, x);
        load_norm<XCH> (lw.ffn_norm, dim, nw);
        // keep the scheduler from moving the row / norm loads behind the weight
        // loads: waiting for them would then wait for the weights as well
        __builtin_amdgcn_sched_barrier (0);
        GV::begin (ps, A, B, 2, up, gate, up, ffn, dim, wg, G, 1, nullptr, true);
        stage_row<true, XCH> (x, dim, xl, nw, m.eps, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.t;
        break;
      }
    case PH_DOWN:
    case PH_GEMV:
      {
        const uint16_t *res = phase == PH_DOWN ? p.s.x : p.gemv_res;
        const QMat w = wmat<WT> (lw.w_down, dim, ffn);
        load_row<XCH> (p.s.t, ffn, x);
        // keep the scheduler from moving the row / norm loads behind the weight
        // loads: waiting for them would then wait for the weights as well
        __builtin_amdgcn_sched_barrier (0);
        GV::begin (ps, A, B, 0, w, w, w, dim, ffn, wg, G, 1, res, true);
        stage_row<false, XCH> (x, ffn, xl, nw, 0.f, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.x, e.residual = res;
        break;
      }
    default: // PH_HEAD
      {
        const QMat w = wmat<WT> (m.output, m.vocab, dim);
        load_row<XCH> (p.s.x, dim, x);
        load_norm<XCH> (m.output_norm, dim, nw);
        // keep the scheduler from moving the row / norm loads behind the weight
        // loads: waiting for them would then wait for the weights as well
        __builtin_amdgcn_sched_barrier (0);
        GV::begin (ps, A, B, 0, w, w, w, m.vocab, dim, wg, G, 1, nullptr, true);
        stage_row<true, XCH> (x, dim, xl, nw, m.final_eps, red, VKL_TRP);
        VKL_TR (2);
        e.y[0] = p.s.logits16, e.y32 = p.logits32;
        e.amax_val = p.s.amax_val, e.amax_idx = p.s.amax_idx;
        break;
      }
    }
  GV::run (ps, A, B, xl, e, red);
  VKL_TR (4);
  if (PHASE == PH_HEAD && head_picks_token (p))
    {
      // The launch's last workgroup picks the token (no wait: every workgroup
      // counts in once its partials are in memory and only the last one goes
      // on), hands it to the next step and, in a replayed loop, starts the
      // next step's residual stream with the token's embedding row.
      __builtin_amdgcn_s_waitcnt (0x0f70); // vmcnt(0)
      __syncthreads ();
      uint32_t *last = (uint32_t *)red;
      if (threadIdx.x == 0)
        {
          uint32_t *done = p.s.sync + kSyncHeadDone;
          const uint32_t old
              = __hip_atomic_fetch_add (done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          *last = old + 1u == (uint32_t)G ? 1u : 0u;
          if (old + 1u == (uint32_t)G)
            st_coherent_u32 (done, 0u);
        }
      __syncthreads ();
      if (*last == 0u)
        return;
      __syncthreads ();
      const uint32_t id = final_argmax<true> (p, G, lds);
      if (p.loop)
        embed_row<WT> (p, id, 0, 1);
    }
}

template <int PHASE, int WT, int XCH, bool NT>
__global__ __launch_bounds__ (kDecThreads) void
decode_phase_direct_kernel (const Params p, const vkl_layer_weights lw, int layer,
                            int G)
{
  extern __shared__ __align__ (16) uint8_t lds[];
  run_phase_direct<PHASE, WT, XCH, NT> (p, lw, layer, (int)blockIdx.x, G, lds);
}

// ---------------------------------------------------------------------------
// short contexts: attention and the Wo projection in one launch
// ---------------------------------------------------------------------------
// The attention phase moves little data (a head's cache rows) but takes
// 4-6 us of dependent steps on n_heads compute units, and the Wo projection
// after it spends half of its 5 us waiting for its first weights.  In one
// launch the first n_heads workgroups compute a head each while the G others
// already have their Wo weights on the way; those then wait until every head
// has counted itself in (the last one sets the flags they poll; the K/Q/V
// phase of the layer has zeroed counter and flags), read the attention row
// and multiply.  The row can be read with ordinary loads: no cache of this
// launch has seen its lines before the wait (caches are invalidated between
// launches), and the heads' stores went through to memory before they counted.  The head workgroups have the lowest indices, so
// they are resident before any waiter; the wait is bounded all the same, and
// one that gives up sets the error word that vkl_decode_status reports.
// Results are those of the two separate launches bit for bit.
template <int WT, int XCH>
__global__ __launch_bounds__ (kDecThreads) void
decode_attn_wo_kernel (const Params p, const vkl_layer_weights lw, int layer, int G)
{
  extern __shared__ __align__ (16) uint8_t lds[];
  const vkl_decode_model &m = p.m;
  const int nh = m.n_heads, dim = m.dim;
  uint32_t *done = p.s.sync + kSyncAttnDone;
  if ((int)blockIdx.x < nh)
    {
      if (m.head_dim == 128)
        attention_head<128, true> (p, lw, (int)blockIdx.x, lds, nullptr);
      else
        attention_head<64, true> (p, lw, (int)blockIdx.x, lds, nullptr);
      // count in once the head's output is in memory
      __builtin_amdgcn_s_waitcnt (0x0f70);
      __syncthreads ();
      if (threadIdx.x < 64)
        {
          uint32_t old = 0;
          if (threadIdx.x == 0)
            old = __hip_atomic_fetch_add (done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          old = (uint32_t)__builtin_amdgcn_readfirstlane ((int)old);
          // (wait_test: a test of the bounded wait; the flags then stay unset)
          if (old + 1u == (uint32_t)nh && threadIdx.x < 8 && !m.wait_test)
            st_coherent_u32 ((uint32_t *)m.flags + kAttnFlagGroup * kFlagGroupWords + 32 * (int)threadIdx.x, 1u);
        }
      return;
    }
  const int wg = (int)blockIdx.x - nh;
  typedef Gemv<WT, false, 1> GV;
  uint16_t *xl = (uint16_t *)lds;
  float *red = (float *)(lds + (size_t)dim * 2);
  Epilogue e = {};
  XRegs x;
  NormRegs nw;
  PipeState ps;
  PipeBuf A, B;
  const QMat w = wmat<WT> (lw.wo, dim, dim);
  // (both items of a wave: with one or two rows per wave that is all of them)
  GV::begin (ps, A, B, 0, w, w, w, dim, dim, wg, G, 2, p.s.x, true);
  uint32_t *seen = (uint32_t *)red + 2 * kDecWaves;
  if (threadIdx.x < 64)
    {
      // (through the scalar memory path: a poll does not queue behind the two
      // weight items this wave and its neighbours have just requested)
      const uint32_t *flag
          = (const uint32_t *)m.flags + kAttnFlagGroup * kFlagGroupWords + 32 * ((int)blockIdx.x & 7);
      bool ok = false;
      const int limit = m.wait_polls > 0 ? m.wait_polls : kFuseSpinLimit;
      for (int spin = 0; spin < limit; ++spin)
        {
          if (flags_equal_scalar (flag, 1, 1u))
            {
              ok = true;
              break;
            }
          __builtin_amdgcn_s_sleep (4);
        }
      if (threadIdx.x == 0)
        {
          *seen = ok ? 1u : 0u;
          if (!ok)
            st_coherent_u32 (p.s.sync + 1, 1u);
        }
    }
  __syncthreads ();
  // a workgroup whose wait gave up must not touch the residual stream: the
  // attention row it would multiply is not complete
  if (*seen == 0u)
    return;
  load_row<XCH> (p.s.att, dim, x);
  stage_row<false, XCH> (x, dim, xl, nw, 0.f, red, nullptr);
  e.y[0] = p.s.x, e.residual = p.s.x;
  GV::run (ps, A, B, xl, e, red);
}

// ---------------------------------------------------------------------------
// long contexts: attention split over chunks of the context
// ---------------------------------------------------------------------------
// One workgroup per head walks the cache row by row, which at several thousand
// positions is a long chain of dependent sweeps on 32..40 compute units.  For
// long contexts the head's rows are split into C chunks, one workgroup each
// (grid C x heads), in one launch.
constexpr int kAttnThreads = 256;

// Every (chunk, head) workgroup scores
// its rows, takes the chunk's own maximum m_c, weights its V rows with
// exp(s - m_c) in fp32 and publishes m_c, sum_c = sum exp(s - m_c) and the
// weighted rows; the workgroup that arrives last at the head's counter
// rescales the parts by exp(m_c - M) / S and rounds the head's output to fp16.
// The K rows of a chunk are requested at the start, its V rows as soon as the
// scores are formed (requested together with K they arrived no earlier and
// the kernel ran 1.6 us longer at 40 heads x 4000 positions).  Scores are
// fp16 values as in the one-workgroup form; the probabilities are not rounded
// to fp16 one by one (that needs M and S before the V pass), which moves an
// output value by at most its last fp16 digit.
// Parts cross compute units without a kernel boundary: they are written and
// read with coherent accesses, and a workgroup counts itself in only after
// its stores have completed.  The last arriver zeroes the counter again.
template <int HD>
__global__ __launch_bounds__ (kAttnThreads) void
attn_chunk_kernel (const Params p, const vkl_layer_weights lw, int C)
{
  constexpr int LPR = HD / 8;             // lanes per cache row
  constexpr int RPS = kAttnThreads / LPR; // rows per sweep
  constexpr int UN = kAttnSweeps;         // sweeps in flight
#ifdef VKL_TRACE
#define VKL_TRC(slot)                                                         \
  if (threadIdx.x == 0 && p.trace)                                            \
    p.trace[((size_t)(blockIdx.y * 32 + blockIdx.x)) * 8 + (slot)] = wall_clock64 ();
#else
#define VKL_TRC(slot)
#endif
  VKL_TRC (0)
  extern __shared__ __align__ (16) uint8_t lds[];
  uint16_t *qk = (uint16_t *)lds;           // [3*HD]: rotated q, rotated k, v
  float *red = (float *)(lds + 1024);       // [16]
  float *part = (float *)(lds + 1024 + 64); // [RPS][HD]
  float *sc = part + RPS * HD;              // [rows of the chunk]
  const int head = blockIdx.y, c = blockIdx.x;
  const int maxlen = p.m.maxlen, dim = p.m.dim;
  const int pos = (int)step_pos (p), L = pos + 1;
  const int R = (L + C - 1) / C;
  const int l0 = c * R, l1 = min (L, l0 + R);
  const int tid = threadIdx.x, sub = tid % LPR, grp = tid / LPR;
  uint32_t *pmax = (uint32_t *)p.s.part_max + head * kAttnChunks;
  uint32_t *psum = (uint32_t *)p.s.part_sum + head * kAttnChunks;
  uint32_t *pout = (uint32_t *)p.s.part_out + (size_t)head * kAttnChunks * HD;
  if (l0 >= L)
    {
      // an empty chunk reports -inf / 0 and drops out of the sums
      if (tid == 0)
        {
          st_coherent_u32 (pmax + c, __float_as_uint (-INFINITY));
          st_coherent_u32 (psum + c, 0u);
        }
      if (tid < HD)
        st_coherent_u32 (pout + c * HD + tid, 0u);
    }
  else
    {
      const bool has_new = pos >= l0 && pos < l1;
      uint16_t *kc = (uint16_t *)lw.kcache + (size_t)head * maxlen * HD;
      uint16_t *vc = (uint16_t *)lw.vcache + (size_t)head * maxlen * HD;
      // The token's q, k and v pairs and the rotation factors are requested
      // first, the K rows right behind them (unconditional loads from clamped
      // addresses: rows past the chunk repeat its last cached row and count
      // with weight 0).  The row of the new position is not read from
      // the cache (this kernel writes it): it is taken from LDS.
      const bool is_q = tid < HD / 2, is_k = !is_q && tid < HD;
      const bool is_v = tid >= HD && tid < HD + HD / 2;
      const int pi = is_q ? tid : (is_k ? tid - HD / 2 : (is_v ? tid - HD : 0));
      const uint16_t *src = p.s.kqv + (is_k ? 0 : (is_v ? 2 * dim : dim)) + head * HD;
      const uint32_t inw = ldg ((const uint32_t *)src + pi);
      const float cs = ldg (p.m.freqc + (size_t)pos * (HD / 2) + pi);
      const float sn = ldg (p.m.freqs + (size_t)pos * (HD / 2) + pi);
      __builtin_amdgcn_sched_barrier (0);
      const int lc1 = has_new ? pos : l1; // cached rows of the chunk: [l0, lc1)
      const int lastrow = max (lc1 - 1, 0);
      uint4 kv[UN], vv[UN];
#pragma unroll
      for (int j = 0; j < UN; ++j)
        kv[j] = ldg4 (kc + (size_t)min (l0 + j * RPS + grp, lastrow) * HD + sub * 8);
      __builtin_amdgcn_sched_barrier (0);

      const float ra = h2f ((uint16_t)(inw & 0xffff)), rb = h2f ((uint16_t)(inw >> 16));
      const uint32_t rot = (uint32_t)f2h (ra * cs - rb * sn)
                           | ((uint32_t)f2h (ra * sn + rb * cs) << 16);
      if (is_q || is_k)
        ((uint32_t *)qk)[(is_k ? HD / 2 : 0) + pi] = rot;
      if (is_v)
        ((uint32_t *)qk)[HD + pi] = inw;
      __syncthreads ();

      const float scale = 1.0f / sqrtf ((float)HD);
      const uint4 qv = ((const uint4 *)qk)[sub];
      float mx = -INFINITY;
      auto score_row = [&] (int l, int lim, const uint4 kr) {
        const float sv = row_sum<LPR> (dot8_f16 (qv, kr, 0.f));
        if (l < lim && sub == 0)
          {
            const float r = h2f (f2h (sv * scale + 0.f));
            sc[l - l0] = r;
            mx = fmaxf (mx, r);
          }
      };
      for (int lb = l0; lb < lc1; lb += UN * RPS)
        {
          if (lb > l0)
            {
#pragma unroll
              for (int j = 0; j < UN; ++j)
                kv[j] = ldg4 (kc + (size_t)min (lb + j * RPS + grp, lastrow) * HD + sub * 8);
            }
#pragma unroll
          for (int j = 0; j < UN; ++j)
            if (lb + j * RPS < lc1) // uniform over the workgroup
              score_row (lb + j * RPS + grp, lc1, kv[j]);
        }
      if (has_new) // uniform over the workgroup: every row group forms it, group 0 records it
        score_row (grp == 0 ? pos : l1, l1, ((const uint4 *)(qk + HD))[sub]);
      __builtin_amdgcn_sched_barrier (0);
#pragma unroll
      for (int j = 0; j < UN; ++j)
        vv[j] = ldg4 (vc + (size_t)min (l0 + j * RPS + grp, lastrow) * HD + sub * 8);
      __builtin_amdgcn_sched_barrier (0);
      mx = wave_max (mx);
      if ((tid & 63) == 0)
        red[tid >> 6] = mx;
      __syncthreads ();
      VKL_TRC (1)
      mx = fmaxf (fmaxf (red[0], red[1]), fmaxf (red[2], red[3]));
      float sum = 0.f;
      for (int l = l0 + tid; l < l1; l += kAttnThreads)
        {
          const float e = expf (sc[l - l0] - mx);
          sc[l - l0] = e;
          sum += e;
        }
      sum = wave_sum (sum);
      if ((tid & 63) == 0)
        red[4 + (tid >> 6)] = sum;
      __syncthreads ();
      VKL_TRC (2)

      float acc[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        acc[j] = 0.f;
      auto add_row = [&] (float pl, const uint4 vr) {
        const uint32_t w[4] = { vr.x, vr.y, vr.z, vr.w };
#pragma unroll
        for (int i = 0; i < 4; ++i)
          {
            acc[2 * i] = __builtin_fmaf (pl, h2f ((uint16_t)(w[i] & 0xffff)), acc[2 * i]);
            acc[2 * i + 1] = __builtin_fmaf (pl, h2f ((uint16_t)(w[i] >> 16)), acc[2 * i + 1]);
          }
      };
      for (int lb = l0; lb < lc1; lb += UN * RPS)
        {
          if (lb > l0)
            {
#pragma unroll
              for (int j = 0; j < UN; ++j)
                vv[j] = ldg4 (vc + (size_t)min (lb + j * RPS + grp, lastrow) * HD + sub * 8);
            }
#pragma unroll
          for (int j = 0; j < UN; ++j)
            {
              const int l = lb + j * RPS + grp;
              if (lb + j * RPS >= lc1) // uniform over the workgroup
                continue;
              add_row (l < lc1 ? sc[min (l, lastrow) - l0] : 0.f, vv[j]);
            }
        }
      if (has_new && grp == 0)
        add_row (sc[pos - l0], ((const uint4 *)(qk + 2 * HD))[sub]);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        part[grp * HD + sub * 8 + j] = acc[j];
      __syncthreads ();
      VKL_TRC (3)
      if (tid < HD)
        {
          float o = 0.f;
          for (int g = 0; g < RPS; ++g)
            o += part[g * HD + tid];
          st_coherent_u32 (pout + c * HD + tid, __float_as_uint (o));
        }
      if (tid == 0)
        {
          st_coherent_u32 (pmax + c, __float_as_uint (mx));
          st_coherent_u32 (psum + c, __float_as_uint (red[4] + red[5] + red[6] + red[7]));
        }
      // the new K and V rows of the cache
      if (has_new && is_k)
        stg ((uint32_t *)(kc + (size_t)pos * HD) + pi, rot);
      if (has_new && is_v)
        stg ((uint32_t *)(vc + (size_t)pos * HD) + pi, inw);
    }
  // count in once this workgroup's parts are in memory
  __builtin_amdgcn_s_waitcnt (0x0f70);
  __syncthreads ();
  VKL_TRC (4)
  uint32_t *flag = (uint32_t *)red + 8;
  if (tid == 0)
    {
      const uint32_t old = __hip_atomic_fetch_add (p.s.attn_cnt + head, 1u, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
      const bool last = old + 1u == (uint32_t)C;
      if (last)
        st_coherent_u32 (p.s.attn_cnt + head, 0u);
      *flag = last ? 1u : 0u;
    }
  __syncthreads ();
  VKL_TRC (5)
  if (*flag == 0u)
    return;
  // the head's last workgroup: M = max m_c, S = sum sum_c exp(m_c - M), and
  // the parts added in chunk order (all loads requested at once)
  const int ci = tid & 31; // kAttnChunks <= 32
  const float mi = __uint_as_float (ld_coherent_u32 (pmax + min (ci, C - 1)));
  const float si = __uint_as_float (ld_coherent_u32 (psum + min (ci, C - 1)));
  float pv[kAttnChunks];
#pragma unroll
  for (int i = 0; i < kAttnChunks; ++i)
    pv[i] = __uint_as_float (ld_coherent_u32 (pout + min (i, C - 1) * HD + (tid & (HD - 1))));
  float M = row_max<16> (ci < C ? mi : -INFINITY);
  M = fmaxf (lane_value (M, 0), lane_value (M, 16));
#ifdef VKL_TRACE
  asm volatile("" ::"v"(pv[kAttnChunks - 1]));
#endif
  VKL_TRC (6)
  // lane i holds chunk i's weight; S and the output add the chunks in index order
  const float wi = (ci < C && mi > -INFINITY) ? expf (mi - M) : 0.f;
  const float swi = wi * si;
  float S = 0.f, o = 0.f;
#pragma unroll
  for (int i = 0; i < kAttnChunks; ++i)
    {
      S += lane_value (swi, i);
      o += lane_value (wi, i) * pv[i];
    }
  if (tid < HD)
    stg (p.s.att + head * HD + tid, f2h (o / S));
  VKL_TRC (7)
}

template <int PHASE, int WT>
__global__ __launch_bounds__ (kDecThreads) void
decode_phase_kernel (const Params p, const vkl_layer_weights lw, int layer,
                     int G)
{
  extern __shared__ __align__ (16) uint8_t lds[];
  run_phase<WT> (p, lw, layer, PHASE, (int)blockIdx.x, G, lds);
}

int
check_model (const vkl_decode_model *m)
{
  VKL_CHECK_ARG (m != nullptr);
  VKL_CHECK_ARG (m->wtype == 8 || m->wtype == 1);
  VKL_CHECK_ARG (m->dim > 0 && m->n_layers > 0 && m->n_heads > 0);
  VKL_CHECK_ARG (m->head_dim == 64 || m->head_dim == 128);
  VKL_CHECK_ARG (m->n_heads * m->head_dim == m->dim);
  VKL_CHECK_ARG ((m->dim % 32) == 0 && (m->ffn % 32) == 0 && m->ffn > 0);
  VKL_CHECK_ARG (m->dim <= 16384 && m->ffn <= 16384);
  VKL_CHECK_ARG (m->vocab > 0 && (m->vocab % 2) == 0 && m->maxlen > 0);
  VKL_CHECK_ARG (m->layers && m->layers_h && m->tok_embd && m->output
                 && m->output_norm);
  VKL_CHECK_ARG (m->freqc && m->freqs && m->scratch);
  VKL_CHECK_ARG (lds_bytes_needed (m->dim, m->ffn, m->maxlen, m->head_dim)
                 <= 160 * 1024);
  return 0;
}

// phase timing: event pairs recorded around launches, read back after the
// step's stream synchronisation
struct PhaseTimer
{
  bool on = false;
  std::vector<hipEvent_t> pool; // start/stop pairs
  std::vector<int> kind;        // phase kind of pair i of the current step
  double ms[VKL_DECODE_PHASES] = {};
  uint64_t n[VKL_DECODE_PHASES] = {};
};
PhaseTimer g_timer;

int
timer_mark (int kind, bool stop, hipStream_t s)
{
  PhaseTimer &t = g_timer;
  if (!t.on)
    return 0;
  const size_t i = stop ? t.kind.size () - 1 : t.kind.size ();
  if (!stop)
    {
      t.kind.push_back (kind);
      while (t.pool.size () < 2 * t.kind.size ())
        {
          hipEvent_t e;
          VKL_HIP (hipEventCreate (&e));
          t.pool.push_back (e);
        }
    }
  VKL_HIP (hipEventRecord (t.pool[2 * i + (stop ? 1 : 0)], s));
  return 0;
}

int
timer_collect (hipStream_t s)
{
  PhaseTimer &t = g_timer;
  if (!t.on)
    return 0;
  VKL_HIP (hipStreamSynchronize (s));
  for (size_t i = 0; i < t.kind.size (); ++i)
    {
      float ms = 0.f;
      VKL_HIP (hipEventElapsedTime (&ms, t.pool[2 * i], t.pool[2 * i + 1]));
      t.ms[t.kind[i]] += ms;
      t.n[t.kind[i]] += 1;
    }
  t.kind.clear ();
  return 0;
}

template <int PHASE, int WT>
int launch_direct (const Params &p, const vkl_layer_weights &lw, int layer,
                   int grid, int G, size_t lds, hipStream_t s);

template <int PHASE, int WT>
int
launch_phase_wt (const Params &p, const vkl_layer_weights &lw, int layer,
                 int grid, int G, size_t lds, hipStream_t s)
{
  if (PHASE == PH_WO || PHASE == PH_UPGATE || PHASE == PH_DOWN || PHASE == PH_HEAD
      || PHASE == PH_GEMV || (PHASE == PH_KQV && layer > 0))
    return launch_direct<PHASE, WT> (p, lw, layer, grid, G, lds, s);
  static LdsLimit limit;
  if (int e = limit.raise ((const void *)decode_phase_kernel<PHASE, WT>, lds))
    return e;
  decode_phase_kernel<PHASE, WT>
      <<<dim3 ((unsigned)grid), dim3 (kDecThreads), lds, s>>> (p, lw, layer,
                                                                 G);
  return 0;
}

// the branch-free form of a projection phase; XCH = 4096-element chunks of
// the staged row
template <int PHASE, int WT, int XCH, bool NT>
int
launch_direct_nt (const Params &p, const vkl_layer_weights &lw, int layer,
                  int grid, int G, size_t lds, hipStream_t s)
{
  static LdsLimit limit;
  if (int e = limit.raise ((const void *)decode_phase_direct_kernel<PHASE, WT, XCH, NT>, lds))
    return e;
  decode_phase_direct_kernel<PHASE, WT, XCH, NT>
      <<<dim3 ((unsigned)grid), dim3 (kDecThreads), lds, s>>> (p, lw, layer, G);
  return 0;
}

template <int PHASE, int WT, int XCH>
int
launch_direct_xch (const Params &p, const vkl_layer_weights &lw, int layer,
                   int grid, int G, size_t lds, hipStream_t s)
{
  return p.stream_once
             ? launch_direct_nt<PHASE, WT, XCH, true> (p, lw, layer, grid, G, lds, s)
             : launch_direct_nt<PHASE, WT, XCH, false> (p, lw, layer, grid, G, lds, s);
}

template <int PHASE, int WT>
int
launch_direct (const Params &p, const vkl_layer_weights &lw, int layer,
               int grid, int G, size_t lds, hipStream_t s)
{
  const int kstage = PHASE == PH_DOWN || PHASE == PH_GEMV ? p.m.ffn : p.m.dim;
  switch ((kstage + 4095) / 4096)
    {
    case 1:
      return launch_direct_xch<PHASE, WT, 1> (p, lw, layer, grid, G, lds, s);
    case 2:
      return launch_direct_xch<PHASE, WT, 2> (p, lw, layer, grid, G, lds, s);
    case 3:
      return launch_direct_xch<PHASE, WT, 3> (p, lw, layer, grid, G, lds, s);
    default:
      return launch_direct_xch<PHASE, WT, 4> (p, lw, layer, grid, G, lds, s);
    }
}

// bytes of weights one decode step reads
size_t
step_weight_bytes (const vkl_decode_model &m)
{
  const double per = m.wtype == 8 ? 34.0 / 32.0 : 2.0;
  const double layer = 4.0 * m.dim * m.dim + 3.0 * (double)m.dim * m.ffn;
  return (size_t)((m.n_layers * layer + (double)m.vocab * m.dim) * per);
}

// what the memory-side cache and the L2s hold together; a set of weights
// below this stays resident from one token to the next
constexpr size_t kCacheResidentBytes = (size_t)288 << 20;

template <int PHASE>
int
launch_phase (const Params &p, const vkl_layer_weights &lw, int layer,
              int grid, int G, size_t lds, hipStream_t s)
{
  if (int e = timer_mark (PHASE, false, s))
    return e;
  if (int e = p.m.wtype == 8
                  ? launch_phase_wt<PHASE, 8> (p, lw, layer, grid, G, lds, s)
                  : launch_phase_wt<PHASE, 1> (p, lw, layer, grid, G, lds, s))
    return e;
  return timer_mark (PHASE, true, s);
}

// attention of one head per workgroup + the Wo projection on G - n_heads more
template <int WT, int XCH>
int
launch_attn_wo_xch (const Params &p, const vkl_layer_weights &lw, int layer, int G, size_t lds,
                    hipStream_t s)
{
  static LdsLimit limit;
  if (int e = limit.raise ((const void *)decode_attn_wo_kernel<WT, XCH>, lds))
    return e;
  decode_attn_wo_kernel<WT, XCH>
      <<<dim3 ((unsigned)G), dim3 (kDecThreads), lds, s>>> (p, lw, layer, G - p.m.n_heads);
  return 0;
}

bool
attn_wo_fused (const Params &p, const vkl_decode_model *m, int G)
{
  return m->flags && !m->separate_attn_wo && (int)p.pos + 1 < attn_split_min (*m)
         && G >= 4 * m->n_heads && m->dim <= 8192 && (m->dim % 8) == 0;
}

int
launch_attn_wo (const Params &p, const vkl_layer_weights &lw, int layer, int G, size_t lds,
                hipStream_t s)
{
  if (int e = timer_mark (PH_ATTN, false, s))
    return e;
  int e;
  if (p.m.dim <= 4096)
    e = p.m.wtype == 8 ? launch_attn_wo_xch<8, 1> (p, lw, layer, G, lds, s)
                       : launch_attn_wo_xch<1, 1> (p, lw, layer, G, lds, s);
  else
    e = p.m.wtype == 8 ? launch_attn_wo_xch<8, 2> (p, lw, layer, G, lds, s)
                       : launch_attn_wo_xch<1, 2> (p, lw, layer, G, lds, s);
  if (e)
    return e;
  return timer_mark (PH_ATTN, true, s);
}

// attention of one layer: one workgroup per head, or the split form for long
// contexts
int
launch_attention (const Params &p, const vkl_decode_model *m,
                  const vkl_layer_weights &lw, int layer, int n_cu, size_t lds,
                  hipStream_t s)
{
  // p.pos is the position of a single step, or the last position of the
  // steps a replayed loop will cover in this form (the LDS need grows with it)
  const int L = (int)p.pos + 1;
  if (L < attn_split_min (*m))
    return launch_phase<PH_ATTN> (p, lw, layer, m->n_heads, m->n_heads, lds, s);
  // Enough chunks to occupy the GPU, and, up to the bound, so many that the
  // rows of a chunk are all in flight at once (kAttnSweeps sweeps of 256
  // lanes) at the longest context.  The count depends on the model and the
  // GPU only, not on the position: the parts of a head are then added in the
  // same grouping whether a step is launched by itself or replayed from a
  // graph that was captured for the longest context.
  int C = (2 * n_cu + m->n_heads - 1) / m->n_heads;
  const int rows_in_flight = kAttnSweeps * kAttnThreads / (m->head_dim / 8);
  C = std::max (C, (m->maxlen + rows_in_flight - 1) / rows_in_flight);
  C = C < 1 ? 1 : (C > kAttnChunks ? kAttnChunks : C);
  const int R = (m->maxlen + C - 1) / C; // most rows of a chunk
  if (R > kAttnChunkRows) // (contexts beyond 32768 positions)
    return launch_phase<PH_ATTN> (p, lw, layer, m->n_heads, m->n_heads, lds, s);
  const size_t lds_c = 1024 + 64 + (size_t)kAttnThreads * 8 * 4 + (size_t)R * 4;
  VKL_CHECK_ARG (lds_c <= 64 * 1024);
  if (int e = timer_mark (PH_ATTN, false, s))
    return e;
  const dim3 grid ((unsigned)C, (unsigned)m->n_heads);
  if (m->head_dim == 128)
    attn_chunk_kernel<128><<<grid, dim3 (kAttnThreads), lds_c, s>>> (p, lw, C);
  else
    attn_chunk_kernel<64><<<grid, dim3 (kAttnThreads), lds_c, s>>> (p, lw, C);
  return timer_mark (PH_ATTN, true, s);
}

} // namespace
} // namespace vkl

using namespace vkl;

extern "C" size_t
vkl_decode_scratch_bytes (const vkl_decode_model *m)
{
  if (!m)
    return 0;
  return carve (nullptr, m->dim, m->ffn, m->vocab, m->n_heads, m->maxlen, m->head_dim,
                m->n_layers).bytes;
}

extern "C" const void *
vkl_decode_logits_f16 (const vkl_decode_model *m)
{
  if (!m || !m->scratch)
    return nullptr;
  return carve (m->scratch, m->dim, m->ffn, m->vocab, m->n_heads, m->maxlen, m->head_dim,
                m->n_layers).logits16;
}

#ifdef VKL_TRACE
static unsigned long long *g_trace = nullptr;
extern "C" void
vkl_debug_set_trace (void *buf)
{
  g_trace = (unsigned long long *)buf;
}
#endif

namespace
{
// the launches of one token: one per phase (mode 0) or one per layer (mode 1)
int
launch_step (const Params &p, const vkl_decode_model *m, int mode, int n_cu, int G,
             size_t lds, hipStream_t s)
{
  // (one head per workgroup inside the layer launch: contexts long enough for
  // the split attention take the launches per phase)
  const bool per_layer = mode == 1 && layer_launch_supported (*m, G)
                         && (int)p.pos + 1 < attn_split_min (*m);
  // (in a replayed greedy loop the previous step's lm_head launch has left the
  // row; the loop launches this once in front of its first step)
  if (per_layer && !(p.loop && !p.sample))
    if (int e = launch_embed_row (p, s))
      return e;
  for (int l = 0; l < m->n_layers; ++l)
    {
      const vkl_layer_weights &lw = m->layers_h[l];
      if (per_layer)
        {
          if (int e = timer_mark (PH_LAYER, false, s))
            return e;
          if (int e = launch_layer (p, lw, l, G, s))
            return e;
          if (int e = timer_mark (PH_LAYER, true, s))
            return e;
          continue;
        }
      if (int e = launch_phase<PH_KQV> (p, lw, l, G, G, lds, s))
        return e;
      if (attn_wo_fused (p, m, G))
        {
          if (int e = launch_attn_wo (p, lw, l, G, lds, s))
            return e;
        }
      else
        {
          if (int e = launch_attention (p, m, lw, l, n_cu, lds, s))
            return e;
          if (int e = launch_phase<PH_WO> (p, lw, l, G, G, lds, s))
            return e;
        }
      if (int e = launch_phase<PH_UPGATE> (p, lw, l, G, G, lds, s))
        return e;
      if (int e = launch_phase<PH_DOWN> (p, lw, l, G, G, lds, s))
        return e;
    }
  const vkl_layer_weights none = {};
  if (int e = launch_phase<PH_HEAD> (p, none, 0, G, G, lds, s))
    return e;
  if (p.loop && p.sample)
    return sample_loop_launch (p.logits32, m->vocab, p.sample, (uint32_t *)p.loop, p.ids, s);
  // (otherwise the lm_head launch has picked the token: head_picks_token)
  return 0;
}

}

namespace vkl
{
// One token row times a matrix on the decode step's down-projection kernel:
// y[N] = W[N, K] x[K] (+ residual), W planar Q8_0 (wtype 8) or dense fp16.
bool
decode_gemv_supported (int N, int K, int wtype)
{
  return (wtype == 8 || wtype == 1) && N > 0 && (N % 2) == 0 && K > 0
         && (K % 32) == 0 && K <= 16384 && N <= (1 << 24)
         && lds_bytes_needed (0, K, 1, 64) <= 160 * 1024;
}

int
decode_gemv_launch (const void *x, const void *w, int wtype, int N, int K,
                    const void *residual, void *y, hipStream_t s)
{
  if (!decode_gemv_supported (N, K, wtype))
    return (int)hipErrorInvalidValue;
  static int n_cu = 0;
  if (n_cu == 0)
    {
      int dev = 0;
      VKL_HIP (hipGetDevice (&dev));
      VKL_HIP (hipDeviceGetAttribute (&n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    }
  Params p = {};
  p.m.dim = N, p.m.ffn = K, p.m.wtype = wtype;
  p.s.t = (uint16_t *)x;
  p.s.x = (uint16_t *)y;
  p.gemv_res = (const uint16_t *)residual;
  // one product cannot know whether its matrix is used again soon; a matrix
  // that cannot stay cached anyway is streamed
  p.stream_once = (double)N * K * (wtype == 8 ? 34.0 / 32.0 : 2.0) > (double)kCacheResidentBytes;
  vkl_layer_weights lw = {};
  lw.w_down = w;
  const int G = n_cu * 2;
  // staged activation row + reduction words (no norm weights are parked)
  const size_t lds = (size_t)K * 2 + 256 + 64;
  if (int e = wtype == 8 ? launch_phase_wt<PH_GEMV, 8> (p, lw, 0, G, G, lds, s)
                         : launch_phase_wt<PH_GEMV, 1> (p, lw, 0, G, G, lds, s))
    return e;
  return vkl_launch_status ();
}
}

extern "C" int
vkl_decode_step (const vkl_decode_model *m, const uint32_t *tok, uint32_t pos,
                 int mode, float *logits32, uint32_t *next_tok, void *stream)
{
  if (int e = check_model (m))
    return e;
  VKL_CHECK_ARG (tok != nullptr && pos < (uint32_t)m->maxlen);
  VKL_CHECK_ARG (mode >= 0 && mode <= 1);
  static int n_cu = 0;
  if (n_cu == 0)
    {
      int dev = 0;
      VKL_HIP (hipGetDevice (&dev));
      VKL_HIP (hipDeviceGetAttribute (
          &n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    }
  const size_t lds
      = lds_bytes_needed (m->dim, m->ffn, m->maxlen, m->head_dim);
  Params p = {};
  p.m = *m;
  p.s = carve (m->scratch, m->dim, m->ffn, m->vocab, m->n_heads, m->maxlen, m->head_dim,
                m->n_layers);
  p.tok = tok;
  p.pos = pos;
  p.logits32 = logits32 ? logits32 : p.s.logits32;
  p.next_tok = next_tok;
  p.loop = nullptr, p.ids = nullptr;
  p.gemv_res = nullptr;
  p.stream_once = step_weight_bytes (*m) > kCacheResidentBytes;
#ifdef VKL_TRACE
  p.trace = g_trace;
#endif
  hipStream_t s = (hipStream_t)stream;
  // two workgroups per compute unit (their registers and LDS fit side by
  // side), which doubles the weight bytes in flight while the activation row
  // is still being staged
  const int G = n_cu * 2;
  if (int e = launch_step (p, m, mode, n_cu, G, lds, s))
    return e;
  if (int e = timer_collect (s))
    return e;
  return vkl_launch_status ();
}

namespace
{
std::mutex g_flags_mu;
std::vector<void *> g_flags_free[16]; // per device: areas handed back (never freed)
std::vector<std::pair<void *, int> > g_flags_out; // areas in use and their device
}

extern "C" int
vkl_decode_flags_acquire (void **flags)
{
  VKL_CHECK_ARG (flags != nullptr);
  *flags = nullptr;
  int dev = 0;
  VKL_HIP (hipGetDevice (&dev));
  VKL_CHECK_ARG (dev >= 0 && dev < 16);
  std::lock_guard<std::mutex> lock (g_flags_mu);
  void *q = nullptr;
  if (!g_flags_free[dev].empty ())
    q = g_flags_free[dev].back (), g_flags_free[dev].pop_back ();
  else
    VKL_HIP (hipExtMallocWithFlags (&q, kFlagBytes, hipDeviceMallocUncached));
  const hipError_t e = hipMemset (q, 0, kFlagBytes);
  if (e != hipSuccess)
    {
      g_flags_free[dev].push_back (q);
      return (int)e;
    }
  g_flags_out.push_back ({ q, dev });
  *flags = q;
  return 0;
}

extern "C" int
vkl_decode_default_mode (const vkl_decode_model *m)
{
  // (measured at short contexts, greedy loop replayed from a graph, 8-10
  // layers of each shape: 7B Q8_0 53.2 against 57.4 us per layer, 7B FP16
  // 80.6 against 83.4, 13B Q8_0 85.0 against 79.5)
  return m && m->flags && m->dim <= 4096 && m->ffn <= 12288 ? 1 : 0;
}

extern "C" void
vkl_decode_flags_release (void *flags)
{
  if (!flags)
    return;
  std::lock_guard<std::mutex> lock (g_flags_mu);
  for (size_t i = 0; i < g_flags_out.size (); ++i)
    if (g_flags_out[i].first == flags)
      {
        g_flags_free[g_flags_out[i].second].push_back (flags);
        g_flags_out.erase (g_flags_out.begin () + (long)i);
        return;
      }
}

extern "C" int
vkl_decode_status (const vkl_decode_model *m, void *stream)
{
  VKL_CHECK_ARG (m != nullptr && m->scratch != nullptr);
  const Scratch sc = carve (m->scratch, m->dim, m->ffn, m->vocab, m->n_heads, m->maxlen,
                            m->head_dim, m->n_layers);
  hipStream_t s = (hipStream_t)stream;
  uint32_t gave_up = 0;
  VKL_HIP (hipMemcpyAsync (&gave_up, sc.sync + 1, sizeof (gave_up), hipMemcpyDeviceToHost, s));
  VKL_HIP (hipStreamSynchronize (s));
  if (!gave_up)
    return 0;
  if (getenv ("VKL_DECODE_VERBOSE"))
    fprintf (stderr, "vkl_decode_status: error word 0x%x\n", gave_up);
  VKL_HIP (hipMemsetAsync (sc.sync + 1, 0, sizeof (uint32_t), s));
  VKL_HIP (hipStreamSynchronize (s));
  return (int)hipErrorLaunchFailure;
}

namespace
{
__global__ void
set_loop_state_kernel (uint32_t *state, uint32_t index, uint32_t pos)
{
  state[0] = index;
  state[1] = pos;
}

__global__ void
set_sample_params_kernel (uint32_t *dst, uint32_t k, uint32_t p_bits, uint32_t seed_lo, uint32_t seed_hi)
{
  dst[0] = k, dst[1] = p_bits, dst[2] = seed_lo, dst[3] = seed_hi;
}

// One captured step per (model, id buffer, logits buffer, attention form).
struct StepGraph
{
  const void *scratch = nullptr, *ids = nullptr, *logits = nullptr;
  uint64_t model_hash = 0; // over every pointer, dimension and option the launches hold
  int long_ctx = 0;
  int mode = 0;
  int sampled = 0;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  uint64_t used = 0;
};
constexpr int kStepGraphs = 8;
StepGraph g_graphs[kStepGraphs];
uint64_t g_graph_clock = 0;
std::mutex g_graph_mu; // the cache above: loops of several host threads take turns

uint64_t
hash_model (const vkl_decode_model *m)
{
  uint64_t h = 1469598103934665603ull;
  auto mix = [&h] (const void *p, size_t n) {
    const uint8_t *b = (const uint8_t *)p;
    for (size_t i = 0; i < n; ++i)
      h = (h ^ b[i]) * 1099511628211ull;
  };
  mix (m, sizeof (*m));
  mix (m->layers_h, sizeof (vkl_layer_weights) * (size_t)m->n_layers);
  return h;
}

void
drop_graph (StepGraph &g)
{
  if (g.exec)
    (void)hipGraphExecDestroy (g.exec);
  if (g.graph)
    (void)hipGraphDestroy (g.graph);
  g = StepGraph ();
}
}

// Greedy steps replayed from a captured graph.  The launches of one token are
// recorded once per form of the attention phase (one workgroup per head below
// kAttnSplitMinLen positions, split above); token index and position live in
// device memory and are advanced by the step's last kernel, so every replay
// is the identical sequence of launches with identical arguments.
namespace
{
int
decode_loop (const vkl_decode_model *m, uint32_t *ids, uint32_t pos0, int n_steps, int mode,
             float *logits32, bool sampled, int topk, float topp, uint64_t seed, void *stream)
{
  if (int e = check_model (m))
    return e;
  VKL_CHECK_ARG (mode >= 0 && mode <= 1);
  VKL_CHECK_ARG (ids != nullptr && n_steps >= 0);
  VKL_CHECK_ARG ((uint64_t)pos0 + (uint64_t)n_steps <= (uint64_t)m->maxlen);
  if (n_steps == 0)
    return 0;
  int dev = 0, n_cu = 0;
  VKL_HIP (hipGetDevice (&dev));
  VKL_HIP (hipDeviceGetAttribute (&n_cu, hipDeviceAttributeMultiprocessorCount,
                                  dev));
  const size_t lds = lds_bytes_needed (m->dim, m->ffn, m->maxlen, m->head_dim);
  hipStream_t s = (hipStream_t)stream;
  Params p = {};
  p.m = *m;
  p.s = carve (m->scratch, m->dim, m->ffn, m->vocab, m->n_heads, m->maxlen, m->head_dim,
                m->n_layers);
  p.tok = nullptr;
  p.logits32 = logits32 ? logits32 : p.s.logits32;
  p.next_tok = nullptr;
  p.loop = p.s.sync + 16;
  p.ids = ids;
  p.sample = sampled ? p.s.sync + 20 : nullptr;
  p.gemv_res = nullptr;
  p.stream_once = step_weight_bytes (*m) > kCacheResidentBytes;
#ifdef VKL_TRACE
  p.trace = nullptr;
#endif
  const int G = n_cu * 2;
  std::lock_guard<std::mutex> lock (g_graph_mu);
  const bool timing = g_timer.on;
  g_timer.on = false;
  const uint64_t mh = hash_model (m);
  set_loop_state_kernel<<<dim3 (1), dim3 (1), 0, s>>> ((uint32_t *)p.loop, 0u, pos0);
  if (sampled)
    set_sample_params_kernel<<<dim3 (1), dim3 (1), 0, s>>> (p.s.sync + 20, (uint32_t)topk,
                                                            __builtin_bit_cast (uint32_t, topp),
                                                            (uint32_t)seed, (uint32_t)(seed >> 32));
  else if (mode == 1 && layer_launch_supported (*m, G))
    launch_embed_row (p, s); // the first step's row; every step leaves the next one's
  int err = 0;
  int done = 0;
  while (done < n_steps && !err)
    {
      // steps [done, upto) share one form of the attention phase
      const int L_first = (int)pos0 + done + 1;
      const int long_ctx = L_first >= attn_split_min (*m) ? 1 : 0;
      int upto = n_steps;
      if (!long_ctx)
        upto = (int)std::min<long long> (n_steps, (long long)attn_split_min (*m) - 1 - (long long)pos0);
      StepGraph *g = nullptr, *lru = &g_graphs[0];
      for (StepGraph &c : g_graphs)
        {
          if (c.exec && c.scratch == m->scratch && c.ids == ids
              && c.logits == p.logits32 && c.model_hash == mh
              && c.long_ctx == long_ctx && c.mode == mode && c.sampled == (int)sampled)
            g = &c;
          if (c.used < lru->used)
            lru = &c;
        }
      if (!g)
        {
          g = lru;
          drop_graph (*g);
          // the position only sizes the attention launch: the largest one
          // this form will see
          p.pos = long_ctx ? (uint32_t)m->maxlen - 1
                           : (uint32_t)std::min (attn_split_min (*m) - 2, m->maxlen - 1);
          hipError_t e = hipStreamBeginCapture (s, hipStreamCaptureModeThreadLocal);
          if (e != hipSuccess)
            {
              err = (int)e;
              break;
            }
          err = launch_step (p, m, mode, n_cu, G, lds, s);
          e = hipStreamEndCapture (s, &g->graph);
          if (!err && e != hipSuccess)
            err = (int)e;
          if (!err)
            {
              e = hipGraphInstantiate (&g->exec, g->graph, nullptr, nullptr, 0);
              if (e != hipSuccess)
                err = (int)e;
            }
          if (err)
            {
              drop_graph (*g);
              break;
            }
          g->scratch = m->scratch, g->ids = ids, g->logits = p.logits32;
          g->model_hash = mh, g->long_ctx = long_ctx, g->mode = mode, g->sampled = (int)sampled;
        }
      g->used = ++g_graph_clock;
      for (; done < upto && !err; ++done)
        err = (int)hipGraphLaunch (g->exec, s);
    }
  g_timer.on = timing;
  return err ? err : vkl_launch_status ();
}
}

extern "C" int
vkl_decode_loop (const vkl_decode_model *m, uint32_t *ids, uint32_t pos0,
                 int n_steps, int mode, float *logits32, void *stream)
{
  return decode_loop (m, ids, pos0, n_steps, mode, logits32, false, 1, -1.f, 0, stream);
}

extern "C" int
vkl_decode_loop_sampled (const vkl_decode_model *m, uint32_t *ids, uint32_t pos0, int n_steps,
                         int mode, float *logits32, int topk, float topp, uint64_t seed,
                         void *stream)
{
  VKL_CHECK_ARG (topp >= 0.f || topk >= 1);
  VKL_CHECK_ARG (topp < 0.f || topp <= 1.0f);
  return decode_loop (m, ids, pos0, n_steps, mode, logits32, true, topk, topp, seed, stream);
}

extern "C" int
vkl_decode_phase_timing (int enable)
{
  g_timer.on = enable != 0;
  g_timer.kind.clear ();
  return 0;
}

extern "C" int
vkl_decode_phase_times (double ms_sum[VKL_DECODE_PHASES],
                        uint64_t launches[VKL_DECODE_PHASES])
{
  VKL_CHECK_ARG (ms_sum && launches);
  for (int i = 0; i < VKL_DECODE_PHASES; ++i)
    {
      ms_sum[i] = g_timer.ms[i], launches[i] = g_timer.n[i];
      g_timer.ms[i] = 0.0, g_timer.n[i] = 0;
    }
  return 0;
}

extern "C" int
vkl_decode_phase_replay (const vkl_decode_model *m, int kind, uint32_t pos,
                         int rounds, void *stream, double *avg_ms,
                         uint64_t *launches)
{
  if (int e = check_model (m))
    return e;
  VKL_CHECK_ARG (((kind >= PH_KQV && kind <= PH_HEAD) || kind == PH_LAYER) && rounds > 0 && avg_ms);
  VKL_CHECK_ARG (pos < (uint32_t)m->maxlen);
  int dev = 0, n_cu = 0;
  VKL_HIP (hipGetDevice (&dev));
  VKL_HIP (hipDeviceGetAttribute (&n_cu, hipDeviceAttributeMultiprocessorCount,
                                  dev));
  const size_t lds = lds_bytes_needed (m->dim, m->ffn, m->maxlen, m->head_dim);
  Params p = {};
  p.m = *m;
  p.s = carve (m->scratch, m->dim, m->ffn, m->vocab, m->n_heads, m->maxlen, m->head_dim,
                m->n_layers);
  p.tok = (const uint32_t *)p.s.amax_idx; // any device word: ids >= vocab read row 0
  p.pos = pos;
  p.logits32 = p.s.logits32;
  p.next_tok = nullptr;
  p.loop = nullptr, p.ids = nullptr;
  p.gemv_res = nullptr;
  p.stream_once = step_weight_bytes (*m) > kCacheResidentBytes;
  hipStream_t s = (hipStream_t)stream;
  const int G = n_cu * 2;
  VKL_CHECK_ARG (kind != PH_LAYER
                 || (layer_launch_supported (*m, G) && (int)pos + 1 < attn_split_min (*m)));
  const bool was_on = g_timer.on;
  g_timer.on = false;
  hipEvent_t e0, e1;
  VKL_HIP (hipEventCreate (&e0));
  VKL_HIP (hipEventCreate (&e1));
  uint64_t n = 0;
  int err = 0;
  VKL_HIP (hipEventRecord (e0, s));
  for (int r = 0; r < rounds && !err; ++r)
    {
      if (kind == PH_HEAD)
        {
          const vkl_layer_weights none = {};
          err = launch_phase<PH_HEAD> (p, none, 0, G, G, lds, s), ++n;
          continue;
        }
      for (int l = 0; l < m->n_layers && !err; ++l, ++n)
        {
          const vkl_layer_weights &lw = m->layers_h[l];
          // layer 0's K/Q/V reads the embedding row instead of the residual
          // stream; replay it as an inner layer so every launch is alike
          const int li = kind == PH_KQV && l == 0 ? 1 : l;
          switch (kind)
            {
            case PH_KQV:
              err = launch_phase<PH_KQV> (p, lw, li, G, G, lds, s);
              break;
            case PH_ATTN:
              err = launch_attention (p, m, lw, l, n_cu, lds, s);
              break;
            case PH_WO:
              err = launch_phase<PH_WO> (p, lw, l, G, G, lds, s);
              break;
            case PH_UPGATE:
              err = launch_phase<PH_UPGATE> (p, lw, l, G, G, lds, s);
              break;
            case PH_LAYER:
              err = launch_layer (p, lw, l, G, s);
              break;
            default:
              err = launch_phase<PH_DOWN> (p, lw, l, G, G, lds, s);
              break;
            }
        }
    }
  hipError_t e = hipEventRecord (e1, s);
  if (e == hipSuccess)
    e = hipEventSynchronize (e1);
  float ms = 0.f;
  if (e == hipSuccess)
    e = hipEventElapsedTime (&ms, e0, e1);
  (void)hipEventDestroy (e0);
  (void)hipEventDestroy (e1);
  g_timer.on = was_on;
  if (err)
    return err;
  VKL_HIP (e);
  *avg_ms = n ? (double)ms / (double)n : 0.0;
  if (launches)
    *launches = n;
  return vkl_launch_status ();
}

extern "C" size_t
vkl_decode_phase_bytes (const vkl_decode_model *m, int kind, size_t L)
{
  if (!m || kind < 0 || kind >= VKL_DECODE_PHASES)
    return 0;
  const size_t dim = (size_t)m->dim, ffn = (size_t)m->ffn, V = (size_t)m->vocab;
  // a Q8_0 matrix [N, K]: N*K quants + N*K/32 fp16 scales
  const bool q8 = m->wtype == 8;
  auto mat = [q8] (size_t N, size_t K) {
    return q8 ? N * K + N * (K / 32) * 2 : N * K * 2;
  };
  switch (kind)
    {
    case PH_KQV: // x + norm weights in, three projections out
      return 3 * mat (dim, dim) + dim * 2 + dim * 4 + 3 * dim * 2;
    case PH_ATTN: // q/k/v in, K and V rows of L positions, new rows, output
      return 3 * dim * 2 + 2 * L * dim * 2 + 2 * dim * 2 + dim * 2;
    case PH_WO:
      return mat (dim, dim) + dim * 2 + 2 * dim * 2;
    case PH_UPGATE:
      return 2 * mat (ffn, dim) + dim * 2 + dim * 4 + ffn * 2;
    case PH_DOWN:
      return mat (dim, ffn) + ffn * 2 + 2 * dim * 2;
    case PH_HEAD:
      return mat (V, dim) + dim * 2 + dim * 4 + V * 2 + V * 4;
    case PH_LAYER: // the five phases; each handed-over row is written and read once
      return vkl_decode_phase_bytes (m, PH_KQV, L) + vkl_decode_phase_bytes (m, PH_ATTN, L)
             + vkl_decode_phase_bytes (m, PH_WO, L) + vkl_decode_phase_bytes (m, PH_UPGATE, L)
             + vkl_decode_phase_bytes (m, PH_DOWN, L);
    default:
      return (size_t)1024 * 8;
    }
}

namespace
{
__global__ __launch_bounds__ (1024) void
argmax_f32_kernel (const float *__restrict__ x, int n, uint32_t *out)
{
  __shared__ float sv[16];
  __shared__ uint32_t si[16];
  float v = -INFINITY;
  uint32_t idx = 0xffffffffu;
  for (int i = threadIdx.x; i < n; i += 1024)
    if (better (x[i], (uint32_t)i, v, idx))
      v = x[i], idx = (uint32_t)i;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    {
      const float ov = __shfl_xor (v, o, 64);
      const uint32_t oi = __shfl_xor (idx, o, 64);
      if (better (ov, oi, v, idx))
        v = ov, idx = oi;
    }
  if ((threadIdx.x & 63) == 0)
    sv[threadIdx.x >> 6] = v, si[threadIdx.x >> 6] = idx;
  __syncthreads ();
  if (threadIdx.x == 0)
    {
      for (int w = 1; w < 16; ++w)
        if (better (sv[w], si[w], v, idx))
          v = sv[w], idx = si[w];
      out[0] = idx == 0xffffffffu ? 0u : idx;
    }
}
}

extern "C" int
vkl_argmax_f32 (const float *x, int n, uint32_t *out, void *stream)
{
  VKL_CHECK_ARG (x && out && n > 0);
  argmax_f32_kernel<<<dim3 (1), dim3 (1024), 0, (hipStream_t)stream>>> (x, n,
                                                                        out);
  return vkl_launch_status ();
}
