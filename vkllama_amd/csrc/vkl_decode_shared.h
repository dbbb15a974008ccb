// Types and device code shared by the decode-step translation units: the
// scratch carve-up, the kernel parameters, the attention of one head and the
// final arg-max.
#ifndef VKL_DECODE_SHARED_H
#define VKL_DECODE_SHARED_H
#include "../../include/vkl_decode.h"
#include "vkl_decode_dev.h"

namespace vkl
{
namespace dec
{
struct Scratch
{
  uint16_t *x;        // [dim] residual stream
  uint16_t *kqv;      // [3*dim]: k | q | v
  uint16_t *att;      // [dim]
  uint16_t *t;        // [ffn] (twice the room)
  uint16_t *logits16; // [vocab]
  float *logits32;    // [vocab]
  float *amax_val;    // [1024]
  uint32_t *amax_idx; // [1024]
  uint32_t *sync;     // error word, loop state, counter and flags of the fused attention + Wo launch
  // one launch per layer (vkl_decode_layer.hip)
  uint16_t *xm;       // [dim] residual stream between the Wo and the down projection
  uint16_t *sink;     // [max(3*dim, ffn)] where a workgroup whose wait gave up drops its results
  uint32_t *lsync;    // arrival counters and flags of the stages, launch count
  // long-context attention, split over kAttnChunks chunks of the context
  float *part_max;    // [heads][kAttnChunks]
  float *part_sum;    // [heads][kAttnChunks]
  float *part_out;    // [heads][kAttnChunks][head_dim]
  uint32_t *attn_cnt; // [heads] chunks of the head that have published their part (zero between launches)
  size_t bytes;
};

constexpr int kLayerSyncBytes = 12288; // see vkl_decode_layer.hip
constexpr int kAttnChunks = 32;      // upper bound on chunks per head
constexpr int kAttnSplitMinLen = 1024; // shorter contexts use one workgroup per head (measured at 7B:
                                       // 10.5 against 12.4 us at 768 positions, 12.6 / 12.5 at 1024)
constexpr int kAttnSweeps = 8;        // sweeps of cache rows a chunk kernel keeps in flight
constexpr int kAttnChunkRows = 1024;  // most rows of a chunk (longer contexts use one workgroup per head)

__host__ __device__ inline size_t
align256 (size_t v)
{
  return (v + 255) & ~(size_t)255;
}

__host__ __device__ inline Scratch
carve (void *base, int dim, int ffn, int vocab, int heads, int maxlen, int hd,
       int n_layers)
{
  Scratch s;
  uint8_t *p = (uint8_t *)base;
  size_t o = 0;
  s.x = (uint16_t *)(p + o), o += align256 ((size_t)dim * 2);
  s.kqv = (uint16_t *)(p + o), o += align256 ((size_t)dim * 6);
  s.att = (uint16_t *)(p + o), o += align256 ((size_t)dim * 2);
  s.t = (uint16_t *)(p + o), o += align256 ((size_t)ffn * 4);
  s.logits16 = (uint16_t *)(p + o), o += align256 ((size_t)vocab * 2);
  s.logits32 = (float *)(p + o), o += align256 ((size_t)vocab * 4);
  s.amax_val = (float *)(p + o), o += 4096;
  s.amax_idx = (uint32_t *)(p + o), o += 4096;
  s.sync = (uint32_t *)(p + o), o += 4096;
  s.xm = (uint16_t *)(p + o), o += align256 ((size_t)dim * 2);
  s.sink = (uint16_t *)(p + o), o += align256 ((size_t)(3 * dim > ffn ? 3 * dim : ffn) * 2);
  s.lsync = (uint32_t *)(p + o), o += kLayerSyncBytes;
  s.part_max = (float *)(p + o), o += align256 ((size_t)heads * kAttnChunks * 4);
  s.part_sum = (float *)(p + o), o += align256 ((size_t)heads * kAttnChunks * 4);
  s.part_out = (float *)(p + o), o += align256 ((size_t)heads * kAttnChunks * hd * 4);
  s.attn_cnt = (uint32_t *)(p + o), o += align256 ((size_t)heads * 4);
  s.bytes = o;
  return s;
}

struct Params
{
  vkl_decode_model m;
  Scratch s;
  const uint32_t *tok;
  uint32_t pos;
  float *logits32;    // destination of the widened logits
  uint32_t *next_tok; // may be null
  // replayed loop (vkl_decode_loop): token index and position live in device
  // memory so that every step is the same sequence of launches
  const uint32_t *loop; // {index into ids, position}, or null
  uint32_t *ids;        // loop: input token ids[index], result to ids[index + 1]
  // loop only: if set, the step ends with a draw from the logits instead of
  // the arg-max ({k, bits of p, seed low, seed high} in device memory)
  const uint32_t *sample;
  const uint16_t *gemv_res; // stand-alone product (PH_GEMV): residual operand or null
  int stream_once; // the weights of a step exceed the caches: request them non-temporally
#ifdef VKL_TRACE
  unsigned long long *trace; // [phase slot][wg][8] wall-clock stamps
#endif
};

#ifdef VKL_TRACE
#define VKL_TR(slot)                                                          \
  if (threadIdx.x == 0 && p.trace)                                            \
    p.trace[((size_t)(layer * 8 + phase) * 1024 + wg) * 8 + (slot)]           \
        = wall_clock64 ();
#define VKL_TRP                                                               \
  (p.trace ? p.trace + ((size_t)(layer * 8 + phase) * 1024 + wg) * 8 : nullptr)
#else
#define VKL_TR(slot)
#define VKL_TRP nullptr
#endif

// position and token of the step: kernel arguments, or the device-resident
// loop state when the step is replayed from a graph
__device__ __forceinline__ uint32_t
step_pos (const Params &p)
{
  return p.loop ? ldg (p.loop + 1) : p.pos;
}

__device__ __forceinline__ const uint32_t *
step_tok (const Params &p)
{
  return p.loop ? p.ids + ldg (p.loop) : p.tok;
}

// ---------------------------------------------------------------------------
// activation staging
// ---------------------------------------------------------------------------
template <bool COH>
__device__ __forceinline__ uint32_t
ld_u32 (const uint32_t *p)
{
  if (COH)
    return ld_coherent_u32 (p);
  return ldg (p);
}

template <bool COH>
__device__ __forceinline__ void
st_u32 (uint32_t *p, uint32_t v)
{
  if (COH)
    st_coherent_u32 (p, v);
  else
    stg (p, v);
}

// sum over the workgroup; `red` is an LDS array of kDecWaves floats
__device__ __forceinline__ float
block_sum (float v, float *red)
{
  v = wave_sum (v);
  __syncthreads ();
  if ((threadIdx.x & 63) == 0)
    red[threadIdx.x >> 6] = v;
  __syncthreads ();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < kDecWaves; ++w)
    t += red[w];
  return t;
}


__device__ __forceinline__ bool
better (float v, uint32_t i, float bv, uint32_t bi)
{
  return v > bv || (v == bv && i < bi);
}


struct PipeBuf
{
  uint4 w[8];
  uint16_t d[8];
  uint32_t res; // mode 0: the two residual values of the item's unit
};


// ---------------------------------------------------------------------------
// attention for one head, context length L = pos + 1
// ---------------------------------------------------------------------------
// LDS use: qk[3*HD] fp16 (rotated q, rotated k, v), sc[maxlen] fp32,
// part[RPB][HD] fp32, red[2*kDecWaves].
struct NoWait
{
  __device__ __forceinline__ bool operator() () const { return true; }
};

// EARLY: the cached rows are requested first, then `wait` is called (it waits
// for the producers of this token's q, k and v inside the same launch; false:
// give up, nothing is stored), then q, k and v are read.
template <int HD, bool COH, bool EARLY = false, typename Wait = NoWait>
__device__ __forceinline__ void
attention_head (const Params &p, const vkl_layer_weights &lw, int head,
                uint8_t *lds, unsigned long long *tr = nullptr, Wait wait = Wait ())
{
#ifdef VKL_TRACE
#define VKL_TRA(slot)                                                         \
  if (tr && threadIdx.x == 0)                                                 \
    tr[slot] = wall_clock64 ();
#else
#define VKL_TRA(slot)
#endif
  constexpr int LPR = HD / 8;            // lanes per cache row (16 B each)
  constexpr int RPB = kDecThreads / LPR; // cache rows per sweep
  constexpr int PRE = 8;                 // sweeps prefetched up front
  const int dim = p.m.dim, maxlen = p.m.maxlen;
  const uint32_t pos = step_pos (p);
  const int L = (int)pos + 1;
  uint16_t *qk = (uint16_t *)lds;    // [3*HD]
  float *sc = (float *)(lds + 1024);      // [maxlen]
  float *part = sc + ((maxlen + 3) & ~3); // [RPB][HD], 16-byte aligned
  float *red = part + RPB * HD;           // [2*kDecWaves]
  uint16_t *kc = (uint16_t *)lw.kcache + (size_t)head * maxlen * HD;
  uint16_t *vc = (uint16_t *)lw.vcache + (size_t)head * maxlen * HD;
  const uint16_t *kin = p.s.kqv + head * HD;
  const uint16_t *qin = p.s.kqv + dim + head * HD;
  const uint16_t *vin = p.s.kqv + 2 * dim + head * HD;
  const int tid = threadIdx.x;
  const int sub = tid % LPR, grp = tid / LPR;

  // This token's q, k, v and its rotation factors are requested first and
  // the first sweeps of cached K and V rows right behind them: loads return
  // in order, so the few bytes the prologue needs are not queued behind the
  // cache rows.  Every load is unconditional, from a clamped address (a branch
  // around a load would make the wait below a wait for all of them): threads
  // without a q/k/v pair repeat pair 0, cache rows past the context repeat the
  // last row and are ignored where they would be used.
  const bool is_q = tid < HD / 2, is_k = !is_q && tid < HD;
  const bool is_v = tid >= HD && tid < HD + HD / 2;
  const int pi = is_q ? tid : (is_k ? tid - HD / 2 : (is_v ? tid - HD : 0));
  uint32_t inw = 0;
  float fc = 0.f, fs = 0.f;
  if (!EARLY)
    {
      inw = ld_u32<COH> ((const uint32_t *)(is_k ? kin : (is_v ? vin : qin)) + pi);
      fc = ldg (p.m.freqc + (size_t)pos * (HD / 2) + pi);
      fs = ldg (p.m.freqs + (size_t)pos * (HD / 2) + pi);
      // (the scheduler must not move the cache rows ahead of these)
      __builtin_amdgcn_sched_barrier (0);
    }
  uint4 kpre[PRE], vpre[PRE];
  const int lastrow = max ((int)pos - 1, 0);
#pragma unroll
  for (int j = 0; j < PRE; ++j)
    kpre[j] = ldg4 (kc + (size_t)min (grp + j * RPB, lastrow) * HD + sub * 8);
#pragma unroll
  for (int j = 0; j < PRE; ++j)
    vpre[j] = ldg4 (vc + (size_t)min (grp + j * RPB, lastrow) * HD + sub * 8);
  __builtin_amdgcn_sched_barrier (0);
  if (EARLY)
    {
      fc = ldg (p.m.freqc + (size_t)pos * (HD / 2) + pi);
      fs = ldg (p.m.freqs + (size_t)pos * (HD / 2) + pi);
      if (!wait ())
        return;
      inw = ld_u32<COH> ((const uint32_t *)(is_k ? kin : (is_v ? vin : qin)) + pi);
    }

  // RoPE on adjacent pairs at position pos.  The new K and V rows are used
  // from LDS here; they go to the cache at the end of the head (a store
  // under a branch at this point would turn the counted waits for the cache
  // rows into waits for everything in flight).
  const float ra = h2f ((uint16_t)(inw & 0xffff)), rb = h2f ((uint16_t)(inw >> 16));
  const uint32_t rot = (uint32_t)f2h (ra * fc - rb * fs)
                       | ((uint32_t)f2h (ra * fs + rb * fc) << 16);
  if (is_q || is_k)
    ((uint32_t *)qk)[(is_k ? HD / 2 : 0) + pi] = rot;
  if (is_v)
    ((uint32_t *)qk)[HD + pi] = inw;
  __syncthreads ();
  VKL_TRA (1);

  // scores[l] = fp16(dot(q, K[l]) / sqrt(HD)); LPR lanes share one cache row
  const float scale = 1.0f / sqrtf ((float)HD);
  const uint4 qv = ((const uint4 *)qk)[sub];
  float mx = -INFINITY; // of the scores this lane has written
  // lim: rows below it are scored (the cached rows; the token's own row, which
  // is in LDS, follows after the sweeps)
  auto score_row = [&] (int l, int lim, const uint4 kv) {
    float s = l < lim ? dot8_f16 (qv, kv, 0.f) : 0.f;
    s = row_sum<LPR> (s);
    if (l < lim && sub == 0)
      {
        const float r = h2f (f2h (s * scale + 0.f));
        sc[l] = r;
        mx = fmaxf (mx, r);
      }
  };
#pragma unroll
  for (int j = 0; j < PRE; ++j)
    {
      const int l = grp + j * RPB;
      if (j * RPB < (int)pos) // wave-uniform
        score_row (l, (int)pos, kpre[j]);
    }
  // the rest of the context, PRE sweeps at a time: unconditional loads from
  // clamped rows, all of a round in flight together (one load per iteration
  // would cost a trip to memory per sweep)
  for (int l0 = PRE * RPB; l0 < (int)pos; l0 += PRE * RPB)
    {
      uint4 kv[PRE];
#pragma unroll
      for (int j = 0; j < PRE; ++j)
        kv[j] = ldg4 (kc + (size_t)min (l0 + j * RPB + grp, lastrow) * HD + sub * 8);
#pragma unroll
      for (int j = 0; j < PRE; ++j)
        {
          const int l = l0 + j * RPB + grp;
          if (l0 + j * RPB < (int)pos) // uniform over the workgroup
            score_row (l, (int)pos, kv[j]);
        }
    }
  // the token's own row: every group forms it (no lane sits out of the
  // cross-lane sum), group 0 records it
  score_row (grp == 0 ? (int)pos : L, L, ((const uint4 *)(qk + HD))[sub]);
  // the maximum travels with the scores: one barrier covers both
  mx = wave_max (mx);
  if ((tid & 63) == 0)
    red[kDecWaves + (tid >> 6)] = mx;
  __syncthreads ();
  VKL_TRA (2);

  // softmax over the L scores; probabilities rounded to fp16
  mx = red[kDecWaves];
#pragma unroll
  for (int w = 1; w < kDecWaves; ++w)
    mx = fmaxf (mx, red[kDecWaves + w]);
  const float e0 = tid < L ? expf (sc[tid < L ? tid : 0] - mx) : 0.f;
  float sum = e0;
  for (int l = tid + kDecThreads; l < L; l += kDecThreads)
    sum += expf (sc[l] - mx);
  sum = wave_sum (sum);
  if ((tid & 63) == 0)
    red[tid >> 6] = sum;
  __syncthreads ();
  sum = 0.f;
#pragma unroll
  for (int w = 0; w < kDecWaves; ++w)
    sum += red[w];
  if (tid < L)
    sc[tid] = h2f (f2h (e0 / sum));
  for (int l = tid + kDecThreads; l < L; l += kDecThreads)
    sc[l] = h2f (f2h (expf (sc[l] - mx) / sum));
  __syncthreads ();
  VKL_TRA (3);

  // out[j] = fp16(sum_l P[l] V[l][j]); thread = (row group, 8 columns)
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
    acc[j] = 0.f;
  // no branch: a row past the context counts with probability 0 (its values
  // are those of a real row, see the clamped loads)
  // (p and v are fp16 values: their product is exact in fp32, so the fused
  // multiply-add rounds as a multiplication and an addition would)
  auto pv_add = [&] (float pl, const uint4 vv) {
    const uint32_t w[4] = { vv.x, vv.y, vv.z, vv.w };
#pragma unroll
    for (int j = 0; j < 4; ++j)
      {
        acc[2 * j] = __builtin_fmaf (pl, h2f ((uint16_t)(w[j] & 0xffff)), acc[2 * j]);
        acc[2 * j + 1] = __builtin_fmaf (pl, h2f ((uint16_t)(w[j] >> 16)), acc[2 * j + 1]);
      }
  };
  auto pv_row = [&] (int l, const uint4 vv) {
    pv_add (l < (int)pos ? sc[min (l, lastrow)] : 0.f, vv);
  };
#pragma unroll
  for (int j = 0; j < PRE; ++j)
    {
      const int l = grp + j * RPB;
      if (j * RPB < (int)pos) // wave-uniform
        pv_row (l, vpre[j]);
    }
  for (int l0 = PRE * RPB; l0 < (int)pos; l0 += PRE * RPB)
    {
      uint4 vv[PRE];
#pragma unroll
      for (int j = 0; j < PRE; ++j)
        vv[j] = ldg4 (vc + (size_t)min (l0 + j * RPB + grp, lastrow) * HD + sub * 8);
#pragma unroll
      for (int j = 0; j < PRE; ++j)
        {
          const int l = l0 + j * RPB + grp;
          if (l0 + j * RPB < (int)pos) // uniform over the workgroup
            pv_row (l, vv[j]);
        }
    }
  // the token's own row (from LDS) is the last of its group's rows
  pv_add (grp == (int)pos % RPB ? sc[pos] : 0.f, ((const uint4 *)(qk + 2 * HD))[sub]);
  ((float4 *)(part + grp * HD + sub * 8))[0] = make_float4 (acc[0], acc[1], acc[2], acc[3]);
  ((float4 *)(part + grp * HD + sub * 8))[1] = make_float4 (acc[4], acc[5], acc[6], acc[7]);
  __syncthreads ();
  VKL_TRA (6);
  // the RPB partial rows of a column are added by four lanes, a quarter of
  // the rows each, and those four by DPP; the lane of an even column then
  // takes the odd neighbour's result and stores the pair
  {
    const int c = tid >> 2, k = tid & 3;
    float o = 0.f;
    if (c < HD)
      {
#pragma unroll
        for (int g = 0; g < RPB / 4; ++g)
          o += part[(k * (RPB / 4) + g) * HD + c];
      }
    o = row_sum<4> (o);
    const float onext = dpp_get<0x104> (o); // row_shl:4: the lane four up
    if (c < HD && (tid & 7) == 0)
      st_u32<COH> ((uint32_t *)(p.s.att + head * HD) + (c >> 1),
                   (uint32_t)f2h (o) | ((uint32_t)f2h (onext) << 16));
  }
  __syncthreads ();
  if (is_k)
    stg ((uint32_t *)(kc + (size_t)pos * HD) + pi, rot);
  if (is_v)
    stg ((uint32_t *)(vc + (size_t)pos * HD) + pi, inw);
}

// where norm weights are parked in LDS: behind the staged row (whole KiB: a
// row fetched straight into LDS fills its last KiB) and the reduction words
__host__ __device__ inline size_t
lds_norm_offset (int dim, int ffn)
{
  const size_t kmax = (size_t)(dim > ffn ? dim : ffn);
  return ((kmax * 2 + 1023) & ~(size_t)1023) + 256;
}

__host__ __device__ inline size_t
lds_bytes_needed (int dim, int ffn, int maxlen, int hd)
{
  // staged activation row + reduction words + parked norm weights (whole KiB)
  const size_t stage = lds_norm_offset (dim, ffn) + (((size_t)dim * 4 + 1023) & ~(size_t)1023);
  const size_t rpb = kDecThreads / (hd / 8);
  const size_t attn = 1024 + (size_t)((maxlen + 3) & ~3) * 4 + rpb * hd * 4 + 256;
  return stage > attn ? stage : attn;
}


// the token's embedding row -> x (residual stream) by all threads of a
// workgroup: nblk workgroups share the row
template <int WT>
__device__ __forceinline__ void
embed_row (const Params &p, uint32_t tok, int blk, int nblk)
{
  const int dim = p.m.dim;
  if (tok >= (uint32_t)p.m.vocab)
    tok = 0;
  for (int i = (int)(blk * kDecThreads + threadIdx.x) * 8; i < dim; i += nblk * kDecThreads * 8)
    {
      uint32_t o[4];
      if (WT == 8)
        {
          const QMat tab = qmat (p.m.tok_embd, p.m.vocab, dim);
          const unsigned long long q
              = ldg ((const unsigned long long *)(tab.q + (size_t)tok * dim + i));
          const float sc = h2f (ldg (tab.d + (size_t)tok * (dim >> 5) + (i >> 5)));
#pragma unroll
          for (int j = 0; j < 4; ++j)
            {
              const int8_t b0 = (int8_t)((q >> (16 * j)) & 0xff);
              const int8_t b1 = (int8_t)((q >> (16 * j + 8)) & 0xff);
              o[j] = (uint32_t)f2h ((float)b0 * sc) | ((uint32_t)f2h ((float)b1 * sc) << 16);
            }
        }
      else
        {
          const uint4 v = ldg4 ((const uint16_t *)p.m.tok_embd + (size_t)tok * dim + i);
          o[0] = v.x, o[1] = v.y, o[2] = v.z, o[3] = v.w;
        }
      uint32_t *dst = (uint32_t *)(p.s.x + i);
      stg (dst, o[0]), stg (dst + 1, o[1]), stg (dst + 2, o[2]), stg (dst + 3, o[3]);
    }
}

// Returns the id to every thread (through LDS).
template <bool COH>
__device__ __forceinline__ uint32_t
final_argmax (const Params &p, int G, uint8_t *lds)
{
  // G per-workgroup partials -> first maximum
  float v = -INFINITY;
  uint32_t idx = 0xffffffffu;
  for (int i = threadIdx.x; i < G; i += kDecThreads)
    {
      const float pv = __uint_as_float (
          ld_u32<COH> ((const uint32_t *)(p.s.amax_val + i)));
      const uint32_t pi = ld_u32<COH> (p.s.amax_idx + i);
      if (better (pv, pi, v, idx))
        v = pv, idx = pi;
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1)
    {
      const float ov = __shfl_xor (v, o, 64);
      const uint32_t oi = __shfl_xor (idx, o, 64);
      if (better (ov, oi, v, idx))
        v = ov, idx = oi;
    }
  float *bv = (float *)lds;
  uint32_t *bi = (uint32_t *)(lds + 64);
  if ((threadIdx.x & 63) == 0)
    {
      bv[threadIdx.x >> 6] = v;
      bi[threadIdx.x >> 6] = idx;
    }
  __syncthreads ();
  if (threadIdx.x == 0)
    {
      for (int w = 1; w < kDecWaves; ++w)
        if (better (bv[w], bi[w], v, idx))
          v = bv[w], idx = bi[w];
      const uint32_t id = idx == 0xffffffffu ? 0u : idx;
      if (p.loop)
        {
          // hand the token to the next replay of the step
          const uint32_t i = ldg (p.loop), ps = ldg (p.loop + 1);
          stg (p.ids + i + 1, id);
          stg ((uint32_t *)p.loop, i + 1);
          stg ((uint32_t *)p.loop + 1, ps + 1);
        }
      else
        stg (p.next_tok, id);
      bi[kDecWaves] = id;
    }
  __syncthreads ();
  return bi[kDecWaves];
}

// Flags of vkl_decode_model::flags: five groups of eight (one per XCD), every
// flag on a 128-byte line of its own; groups 0..3 are the stages of the layer
// launch, group 4 belongs to the attention + Wo launch.
constexpr int kFlagGroupWords = 8 * 32;
constexpr int kFlagGroups = 5;
constexpr size_t kFlagBytes = (size_t)kFlagGroups * kFlagGroupWords * 4;

// One look at `nflags` flags (1 or 8, 32 words apart) through the scalar
// memory path (reads only; glc: past the scalar cache).  True: all equal `want`.
__device__ __forceinline__ bool
flags_equal_scalar (const uint32_t *flag, int nflags, uint32_t want)
{
  const uint64_t a = (uint64_t)flag;
  const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane ((int)(uint32_t)a);
  const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane ((int)(uint32_t)(a >> 32));
  const uint64_t base = ((uint64_t)hi << 32) | lo;
  if (nflags == 1)
    {
      uint32_t v;
      asm volatile("s_load_dword %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(base) : "memory");
      return v == want;
    }
  uint32_t v0, v1, v2, v3, v4, v5, v6, v7;
  asm volatile("s_load_dword %0, %8, 0x0 glc\n\t"
               "s_load_dword %1, %8, 0x80 glc\n\t"
               "s_load_dword %2, %8, 0x100 glc\n\t"
               "s_load_dword %3, %8, 0x180 glc\n\t"
               "s_load_dword %4, %8, 0x200 glc\n\t"
               "s_load_dword %5, %8, 0x280 glc\n\t"
               "s_load_dword %6, %8, 0x300 glc\n\t"
               "s_load_dword %7, %8, 0x380 glc\n\t"
               "s_waitcnt lgkmcnt(0)"
               : "=&s"(v0), "=&s"(v1), "=&s"(v2), "=&s"(v3), "=&s"(v4), "=&s"(v5), "=&s"(v6), "=&s"(v7)
               : "s"(base)
               : "memory");
  return v0 == want && v1 == want && v2 == want && v3 == want && v4 == want && v5 == want
         && v6 == want && v7 == want;
}

// One layer of the step as a single launch (vkl_decode_layer.hip): K/Q/V,
// attention with one workgroup per head, Wo, up/gate, down.  G workgroups that
// must all be resident at once.
bool layer_launch_supported (const vkl_decode_model &m, int G);
int launch_layer (const Params &p, const vkl_layer_weights &lw, int layer, int G, hipStream_t s);
// the token's embedding row -> residual stream (one small launch in front of layer 0)
int launch_embed_row (const Params &p, hipStream_t s);
} // namespace dec
// vkl_sample.hip: the draw that ends a step of a replayed loop; dev_params =
// {k, bits of p, seed low, seed high} in device memory, loop = {index,
// position}: writes ids[index + 1] and advances both loop words
int sample_loop_launch (const float *logits, int V, const uint32_t *dev_params, uint32_t *loop,
                        uint32_t *ids, hipStream_t s);
} // namespace vkl
#endif
