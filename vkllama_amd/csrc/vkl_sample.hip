// Token sampling on the device: top-k or top-p over one row of fp32 logits,
// so that sampled generation hands the next token to the next decode step
// without the logits leaving device memory.  The candidate set and its
// probabilities are those of the host samplers (largest logits first, ties
// toward the lower token id; softmax over the kept logits); the draw uses a
// counter-based generator, one uniform number per (seed, counter).
//
// One workgroup of 1024 threads:
//   1. every logit becomes a 64-bit key, order-preserving in the logit, with
//      the complemented token id below it, so that all keys differ;
//   2. the k-th largest key is found by radix selection, eight passes of one
//      byte with a 256-bin histogram in LDS;
//   3. the keys not below it (exactly k) are gathered and sorted (bitonic);
//   4. one thread walks the sorted candidates in order (at most 1024): the
//      softmax, for top-p the prefix whose mass reaches p, and the draw.  The
//      sums run in candidate order, as in the host samplers.
#include "../../include/vkl_hip.h"
#include "vkl_common.h"

namespace
{
constexpr int kSampThreads = 1024;
constexpr int kMaxCand = 1024;

__device__ __forceinline__ uint64_t
logit_key (float v, uint32_t id)
{
  const uint32_t b = __float_as_uint (v);
  const uint32_t u = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  return ((uint64_t)u << 32) | (uint64_t)(0xffffffffu - id);
}

__device__ __forceinline__ float
key_logit (uint64_t key)
{
  const uint32_t u = (uint32_t)(key >> 32);
  const uint32_t b = (u & 0x80000000u) ? (u & 0x7fffffffu) : ~u;
  return __uint_as_float (b);
}

// splitmix64 of (seed, counter) -> uniform in [0, 1) with 24 bits
__device__ __forceinline__ float
uniform01 (uint64_t seed, uint32_t counter)
{
  uint64_t z = seed + 0x9E3779B97F4A7C15ull * ((uint64_t)counter + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

struct SampleArgs
{
  const float *logits;
  int V, k;     // k: candidates kept by rank (top-p: the cap, kMaxCand)
  float p;      // < 0: top-k; else top-p
  uint64_t seed;
  uint32_t counter;
  const uint32_t *counter_dev; // if set, added to counter (e.g. a position kept on the device)
  uint32_t *tok;
  uint32_t *cand_ids; // optional: candidates of this draw, most likely first
  float *cand_probs;
  uint32_t *cand_n;
  // a step of a replayed decode loop (all three set): k, p and the seed come
  // from `dev` = {k, bits of p, seed low, seed high} in device memory, so that
  // one captured launch serves every request; loop = {index into ids,
  // position}; the token of position + 1 goes to ids[index + 1], drawn with
  // that position as the counter, and both loop words advance
  const uint32_t *dev;
  uint32_t *loop;
  uint32_t *ids;
};

__global__ __launch_bounds__ (kSampThreads) void
sample_kernel (const SampleArgs args)
{
  SampleArgs a = args;
  if (a.dev)
    {
      a.p = __uint_as_float (vkl::ldg (a.dev + 1));
      const int k = (int)vkl::ldg (a.dev);
      a.k = a.p >= 0.f ? kMaxCand : (k > kMaxCand ? kMaxCand : max (k, 1));
      a.seed = (uint64_t)vkl::ldg (a.dev + 2) | ((uint64_t)vkl::ldg (a.dev + 3) << 32);
    }
  __shared__ uint32_t hist[256];
  __shared__ uint64_t cand[kMaxCand];
  __shared__ uint64_t prefix_s;
  __shared__ uint32_t need_s, count_s;
  const int tid = threadIdx.x;
  const int keep = min (min (a.k, kMaxCand), a.V);

  // ---- the keep-th largest key ----------------------------------------------
  if (tid == 0)
    prefix_s = 0, need_s = (uint32_t)keep, count_s = 0;
  for (int pass = 7; pass >= 0; --pass)
    {
      if (tid < 256)
        hist[tid] = 0;
      __syncthreads ();
      const uint64_t prefix = prefix_s;
      const int shift = 8 * pass;
      for (int i = tid; i < a.V; i += kSampThreads)
        {
          const uint64_t key = logit_key (vkl::ldg (a.logits + i), (uint32_t)i);
          // keys that agree with the prefix in all bytes above this one
          if (pass == 7 || (key >> (shift + 8)) == (prefix >> (shift + 8)))
            atomicAdd (&hist[(uint32_t)(key >> shift) & 255u], 1u);
        }
      __syncthreads ();
      if (tid == 0)
        {
          uint32_t need = need_s, cum = 0;
          int bin = 255;
          for (; bin > 0; --bin)
            {
              if (cum + hist[bin] >= need)
                break;
              cum += hist[bin];
            }
          need_s = need - cum;
          prefix_s = prefix | ((uint64_t)bin << shift);
        }
      __syncthreads ();
    }
  const uint64_t kth = prefix_s;

  // ---- gather and sort the candidates ------------------------------------------
  int P = 1;
  while (P < keep)
    P <<= 1;
  for (int i = tid; i < P; i += kSampThreads)
    cand[i] = 0;
  __syncthreads ();
  for (int i = tid; i < a.V; i += kSampThreads)
    {
      const uint64_t key = logit_key (vkl::ldg (a.logits + i), (uint32_t)i);
      if (key >= kth)
        {
          const uint32_t slot = atomicAdd (&count_s, 1u);
          if (slot < (uint32_t)kMaxCand)
            cand[slot] = key;
        }
    }
  __syncthreads ();
  // bitonic sort, descending, over P slots (unused slots hold key 0, below
  // every real key)
  for (int size = 2; size <= P; size <<= 1)
    for (int stride = size >> 1; stride > 0; stride >>= 1)
      {
        for (int i = tid; i < P; i += kSampThreads)
          {
            const int j = i ^ stride;
            if (j > i)
              {
                const uint64_t x = cand[i], y = cand[j];
                const bool desc = (i & size) == 0;
                if (desc ? x < y : x > y)
                  cand[i] = y, cand[j] = x;
              }
          }
        __syncthreads ();
      }

  // ---- probabilities and the draw, in candidate order --------------------------
  __shared__ float ex[kMaxCand];      // exp(logit - top) of the candidates
  __shared__ float red[kSampThreads];
  const float top = key_logit (cand[0]);
  for (int i = tid; i < keep; i += kSampThreads)
    ex[i] = expf (key_logit (cand[i]) - top);
  // top-p: mass of the whole vocabulary relative to the top logit
  float part = 0.f;
  if (a.p >= 0.f)
    for (int i = tid; i < a.V; i += kSampThreads)
      part += expf (vkl::ldg (a.logits + i) - top);
  red[tid] = part;
  __syncthreads ();
  for (int s = kSampThreads / 2; s > 0; s >>= 1)
    {
      if (tid < s)
        red[tid] += red[tid + s];
      __syncthreads ();
    }
  if (tid != 0)
    return;
  int n = keep;
  if (a.p >= 0.f)
    {
      // tokens are added while the mass so far is below p
      const float total = red[0];
      float mass = 0.f;
      n = 0;
      while (n < keep && mass < a.p)
        {
          mass += ex[n] / total;
          ++n;
        }
      if (n == 0)
        n = 1;
    }
  float sum = 0.f;
  for (int i = 0; i < n; ++i)
    sum += ex[i];
  uint32_t ctr = a.counter + (a.counter_dev ? vkl::ldg (a.counter_dev) : 0u);
  uint32_t index = 0, position = 0;
  if (a.loop)
    {
      index = vkl::ldg (a.loop), position = vkl::ldg (a.loop + 1);
      ctr = a.counter + position + 1u;
    }
  const float target = uniform01 (a.seed, ctr);
  float cum = 0.f;
  int pick = -1;
  for (int i = 0; i < n; ++i)
    {
      const float pr = ex[i] / sum;
      if (a.cand_probs)
        a.cand_probs[i] = pr;
      if (a.cand_ids)
        a.cand_ids[i] = 0xffffffffu - (uint32_t)cand[i];
      cum += pr;
      if (pick < 0 && cum > target)
        pick = i;
    }
  if (pick < 0) // rounding left the total a hair below the target
    pick = n - 1;
  if (a.cand_n)
    *a.cand_n = (uint32_t)n;
  const uint32_t drawn = 0xffffffffu - (uint32_t)cand[pick];
  if (a.loop)
    {
      a.ids[index + 1] = drawn;
      a.loop[0] = index + 1u, a.loop[1] = position + 1u;
    }
  else
    *a.tok = drawn;
}
} // namespace

namespace vkl
{
// the draw of a replayed decode step (see SampleArgs::dev)
int
sample_loop_launch (const float *logits, int V, const uint32_t *dev_params, uint32_t *loop,
                    uint32_t *ids, hipStream_t s)
{
  SampleArgs a = {};
  a.logits = logits, a.V = V;
  a.k = 1, a.p = -1.f;
  a.dev = dev_params, a.loop = loop, a.ids = ids;
  sample_kernel<<<dim3 (1), dim3 (kSampThreads), 0, s>>> (a);
  return 0;
}
}

extern "C" int
vkl_sample_f32 (const float *logits, int V, int k, float p, uint64_t seed,
                uint32_t counter, const uint32_t *counter_dev, uint32_t *tok,
                uint32_t *cand_ids, float *cand_probs, uint32_t *cand_n,
                void *stream)
{
  VKL_CHECK_ARG (logits && tok && V > 0);
  VKL_CHECK_ARG (p >= 0.f || k >= 1);
  VKL_CHECK_ARG (p < 0.f || p <= 1.0f);
  SampleArgs a = {};
  a.logits = logits, a.V = V;
  a.k = p >= 0.f ? kMaxCand : (k > kMaxCand ? kMaxCand : k);
  a.p = p, a.seed = seed, a.counter = counter, a.counter_dev = counter_dev;
  a.tok = tok, a.cand_ids = cand_ids, a.cand_probs = cand_probs, a.cand_n = cand_n;
  sample_kernel<<<dim3 (1), dim3 (kSampThreads), 0, (hipStream_t)stream>>> (a);
  return vkl_launch_status ();
}
