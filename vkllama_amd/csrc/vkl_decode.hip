// Fused one-token decode step for Llama-2-shaped models with Q8_0 weights.
//
// Work decomposition (both launch modes): a grid of G workgroups of 512
// threads, G = number of compute units.  In a projection phase workgroup g
// owns the contiguous output rows [N*g/G, N*(g+1)/G) of the weight matrix, so
// it streams one contiguous span of the int8 plane; inside it wave w takes
// the row pairs 2w, 2w+16, ...; lane l of a wave handles the 16 quants at
// k = step*1024 + 16*l of each row (one dwordx4 load = half a Q8_0 block).
// The activation vector is staged once per phase in LDS as fp16 (with the
// RMSNorm folded in where the phase starts with one).  Attention runs one
// workgroup per head.
//
// Each phase is HBM-bound: 34 bytes per 32 weights are read exactly once, the
// activations (a few KiB) come from L2.
#include "../../include/vkl_decode.h"
#include "vkl_decode_dev.h"

namespace vkl
{
namespace
{
struct Scratch
{
  uint16_t *x;    // [dim] residual stream
  uint16_t *kqv;  // [3*dim]: k | q | v
  uint16_t *att;  // [dim]
  uint16_t *t;    // [ffn]
  uint16_t *logits16; // [vocab]
  float *logits32;    // [vocab]
  float *amax_val;    // [1024]
  uint32_t *amax_idx; // [1024]
  uint32_t *sync;     // barrier counter + error flag
  size_t bytes;
};

__host__ __device__ inline size_t
align256 (size_t v)
{
  return (v + 255) & ~(size_t)255;
}

__host__ __device__ inline Scratch
carve (void *base, int dim, int ffn, int vocab)
{
  Scratch s;
  uint8_t *p = (uint8_t *)base;
  size_t o = 0;
  s.x = (uint16_t *)(p + o), o += align256 ((size_t)dim * 2);
  s.kqv = (uint16_t *)(p + o), o += align256 ((size_t)dim * 6);
  s.att = (uint16_t *)(p + o), o += align256 ((size_t)dim * 2);
  s.t = (uint16_t *)(p + o), o += align256 ((size_t)ffn * 2);
  s.logits16 = (uint16_t *)(p + o), o += align256 ((size_t)vocab * 2);
  s.logits32 = (float *)(p + o), o += align256 ((size_t)vocab * 4);
  s.amax_val = (float *)(p + o), o += 4096;
  s.amax_idx = (uint32_t *)(p + o), o += 4096;
  s.sync = (uint32_t *)(p + o), o += 256;
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
};

// ---------------------------------------------------------------------------
// activation staging
// ---------------------------------------------------------------------------
template <bool COH>
__device__ __forceinline__ uint32_t
ld_u32 (const uint32_t *p)
{
  if (COH)
    return ld_coherent_u32 (p);
  return *p;
}

template <bool COH>
__device__ __forceinline__ void
st_u32 (uint32_t *p, uint32_t v)
{
  if (COH)
    st_coherent_u32 (p, v);
  else
    *p = v;
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

// xl[0..Kp) <- fp16 activation row (K valid, zero padded), from global memory
template <bool COH>
__device__ __forceinline__ void
stage_raw (const uint16_t *src, int K, int Kp, uint16_t *xl)
{
  const uint32_t *s32 = (const uint32_t *)src;
  uint32_t *x32 = (uint32_t *)xl;
  for (int i = threadIdx.x; i < Kp / 2; i += kDecThreads)
    {
      uint32_t v = 0;
      if (2 * i + 1 < K)
        v = ld_u32<COH> (s32 + i);
      else if (2 * i < K)
        v = src[2 * i];
      x32[i] = v;
    }
}

// xl <- one row of a planar Q8_0 table, dequantised: fp16(float(q) * d)
__device__ __forceinline__ void
stage_embed_q8 (const QMat tab, size_t row, int K, int Kp, uint16_t *xl)
{
  const uint32_t *q32 = (const uint32_t *)(tab.q + row * Kp);
  const uint16_t *d = tab.d + row * (Kp >> 5);
  uint32_t *x32 = (uint32_t *)xl;
  for (int i = threadIdx.x; i < Kp / 4; i += kDecThreads)
    {
      const uint32_t w = q32[i];
      const float sc = h2f (d[i >> 3]);
      uint16_t h[4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
        {
          const int8_t b = (int8_t)((w >> (8 * j)) & 0xff);
          h[j] = 4 * i + j < K ? f2h ((float)b * sc) : (uint16_t)0;
        }
      x32[2 * i] = (uint32_t)h[0] | ((uint32_t)h[1] << 16);
      x32[2 * i + 1] = (uint32_t)h[2] | ((uint32_t)h[3] << 16);
    }
}

__device__ __forceinline__ void
stage_embed_f16 (const uint16_t *tab, size_t row, int K, int Kp, uint16_t *xl)
{
  for (int i = threadIdx.x; i < Kp; i += kDecThreads)
    xl[i] = i < K ? tab[row * K + i] : (uint16_t)0;
}

// in-place RMSNorm of the staged row: y = fp16(x * w * rsqrt(mean(x^2)+eps))
__device__ __forceinline__ void
norm_staged (uint16_t *xl, int K, const float *w, float eps, float *red)
{
  float s = 0.f;
  for (int i = threadIdx.x; i < K; i += kDecThreads)
    {
      const float v = h2f (xl[i]);
      s += v * v;
    }
  const float total = block_sum (s, red);
  const float alpha = 1.0f / sqrtf (total / (float)K + eps);
  for (int i = threadIdx.x; i < K; i += kDecThreads)
    xl[i] = f2h (h2f (xl[i]) * w[i] * alpha);
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
};

__device__ __forceinline__ bool
better (float v, uint32_t i, float bv, uint32_t bi)
{
  return v > bv || (v == bv && i < bi);
}

// MODE 0: y = x W^T (+ residual);  MODE 1: three matrices, three outputs;
// MODE 2: y = silu(x W1^T) * (x W0^T)   (W0 = up, W1 = gate)
template <int MODE, int NMAT, bool COH>
__device__ __forceinline__ void
gemv_phase (const QMat *mats, int N, int K, const uint16_t *xl,
            const Epilogue &e, int wg, int G, float *red)
{
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int Kp = ((K + 31) >> 5) << 5, nb = Kp >> 5;
  const int lo = (int)((long long)N * wg / G) & ~1;
  int hi = (int)((long long)N * (wg + 1) / G) & ~1;
  if (wg == G - 1)
    hi = N;
  float best_v = -INFINITY;
  uint32_t best_i = 0xffffffffu;

  for (int r0 = lo + 2 * wave; r0 < hi; r0 += 2 * kDecWaves)
    {
      const int r1 = min (r0 + 1, N - 1);
      float acc[NMAT][2];
#pragma unroll
      for (int t = 0; t < NMAT; ++t)
        acc[t][0] = acc[t][1] = 0.f;
      const size_t q0 = (size_t)r0 * Kp, q1 = (size_t)r1 * Kp;
      const size_t d0 = (size_t)r0 * nb, d1 = (size_t)r1 * nb;
#pragma unroll 2
      for (int kk = lane * 16; kk < Kp; kk += VKL_WAVE * 16)
        {
          uint4 w[NMAT][2];
          uint16_t d[NMAT][2];
#pragma unroll
          for (int t = 0; t < NMAT; ++t)
            {
              w[t][0] = *(const uint4 *)(mats[t].q + q0 + kk);
              w[t][1] = *(const uint4 *)(mats[t].q + q1 + kk);
              d[t][0] = mats[t].d[d0 + (kk >> 5)];
              d[t][1] = mats[t].d[d1 + (kk >> 5)];
            }
          const uint4 *xp = (const uint4 *)(xl + kk);
          const uint4 x0 = xp[0], x1 = xp[1];
          const h16x2 xv[8]
              = { __builtin_bit_cast (h16x2, x0.x), __builtin_bit_cast (h16x2, x0.y),
                  __builtin_bit_cast (h16x2, x0.z), __builtin_bit_cast (h16x2, x0.w),
                  __builtin_bit_cast (h16x2, x1.x), __builtin_bit_cast (h16x2, x1.y),
                  __builtin_bit_cast (h16x2, x1.z), __builtin_bit_cast (h16x2, x1.w) };
#pragma unroll
          for (int t = 0; t < NMAT; ++t)
            {
              acc[t][0] += dot16_q8 (w[t][0], xv, 0.f) * h2f (d[t][0]);
              acc[t][1] += dot16_q8 (w[t][1], xv, 0.f) * h2f (d[t][1]);
            }
        }
#pragma unroll
      for (int t = 0; t < NMAT; ++t)
        {
          acc[t][0] = wave_sum (acc[t][0]);
          acc[t][1] = wave_sum (acc[t][1]);
        }
      if (lane != 0)
        continue;
      const bool two = r0 + 1 < N;
      if (MODE == 1)
        {
#pragma unroll
          for (int t = 0; t < NMAT; ++t)
            {
              const uint32_t pk = (uint32_t)f2h (acc[t][0])
                                  | ((uint32_t)f2h (acc[t][1]) << 16);
              if (two)
                st_u32<COH> ((uint32_t *)(e.y[t] + r0), pk);
              else
                e.y[t][r0] = (uint16_t)pk;
            }
          continue;
        }
      uint16_t h0, h1;
      if (MODE == 2)
        {
          h0 = f2h (silu (acc[NMAT - 1][0]) * acc[0][0]);
          h1 = f2h (silu (acc[NMAT - 1][1]) * acc[0][1]);
        }
      else
        {
          h0 = f2h (acc[0][0]);
          h1 = f2h (acc[0][1]);
          if (e.residual)
            {
              uint32_t rr;
              if (two)
                rr = ld_u32<COH> ((const uint32_t *)(e.residual + r0));
              else
                rr = e.residual[r0];
              h0 = f2h (h2f (h0) + h2f ((uint16_t)(rr & 0xffff)));
              h1 = f2h (h2f (h1) + h2f ((uint16_t)(rr >> 16)));
            }
        }
      const uint32_t pk = (uint32_t)h0 | ((uint32_t)h1 << 16);
      if (two)
        st_u32<COH> ((uint32_t *)(e.y[0] + r0), pk);
      else
        e.y[0][r0] = h0;
      if (MODE == 0 && e.y32)
        {
          e.y32[r0] = h2f (h0);
          if (two)
            e.y32[r0 + 1] = h2f (h1);
        }
      if (MODE == 0 && e.amax_val)
        {
          if (better (h2f (h0), (uint32_t)r0, best_v, best_i))
            best_v = h2f (h0), best_i = (uint32_t)r0;
          if (two && better (h2f (h1), (uint32_t)r0 + 1, best_v, best_i))
            best_v = h2f (h1), best_i = (uint32_t)r0 + 1;
        }
    }

  if (MODE == 0 && e.amax_val)
    {
      // lane 0 of each wave holds that wave's best; combine in LDS
      float *bv = red;
      uint32_t *bi = (uint32_t *)(red + kDecWaves);
      __syncthreads ();
      if (lane == 0)
        {
          bv[wave] = best_v;
          bi[wave] = best_i;
        }
      __syncthreads ();
      if (threadIdx.x == 0)
        {
          float v = bv[0];
          uint32_t i = bi[0];
          for (int w = 1; w < kDecWaves; ++w)
            if (better (bv[w], bi[w], v, i))
              v = bv[w], i = bi[w];
          st_u32<COH> ((uint32_t *)(e.amax_val + wg), __float_as_uint (v));
          st_u32<COH> (e.amax_idx + wg, i);
        }
    }
}

// ---------------------------------------------------------------------------
// attention for one head, context length L = pos + 1
// ---------------------------------------------------------------------------
// LDS use: qk[3*HD] fp16 (rotated q, rotated k, v), sc[maxlen] fp32, part[...]
template <int HD, bool COH>
__device__ __forceinline__ void
attention_head (const Params &p, const vkl_layer_weights &lw, int head,
                uint8_t *lds)
{
  constexpr int LPR = HD / 8;             // lanes per cache row (16 B each)
  constexpr int RPB = kDecThreads / LPR;  // rows handled per sweep
  const int dim = p.m.dim, maxlen = p.m.maxlen;
  const uint32_t pos = p.pos;
  const int L = (int)pos + 1;
  uint16_t *qk = (uint16_t *)lds;                    // [3*HD]
  float *sc = (float *)(lds + 1024);                 // [maxlen]
  float *part = sc + maxlen;                         // [RPB][HD]
  float *red = part + RPB * HD;                      // [2*kDecWaves]
  uint16_t *kc = (uint16_t *)lw.kcache + (size_t)head * maxlen * HD;
  uint16_t *vc = (uint16_t *)lw.vcache + (size_t)head * maxlen * HD;
  const uint16_t *kin = p.s.kqv + head * HD;
  const uint16_t *qin = p.s.kqv + dim + head * HD;
  const uint16_t *vin = p.s.kqv + 2 * dim + head * HD;

  // RoPE on adjacent pairs at position pos; K and V rows go to the cache
  const int tid = threadIdx.x;
  if (tid < HD) // HD/2 pairs of q, HD/2 pairs of k
    {
      const bool is_k = tid >= HD / 2;
      const int i = is_k ? tid - HD / 2 : tid;
      const uint32_t v = ld_u32<COH> ((const uint32_t *)(is_k ? kin : qin) + i);
      const float c = p.m.freqc[(size_t)pos * (HD / 2) + i];
      const float s = p.m.freqs[(size_t)pos * (HD / 2) + i];
      const float a = h2f ((uint16_t)(v & 0xffff)), b = h2f ((uint16_t)(v >> 16));
      const uint32_t r = (uint32_t)f2h (a * c - b * s)
                         | ((uint32_t)f2h (a * s + b * c) << 16);
      ((uint32_t *)qk)[(is_k ? HD / 2 : 0) + i] = r;
      if (is_k)
        ((uint32_t *)(kc + (size_t)pos * HD))[i] = r;
    }
  else if (tid < HD + HD / 2)
    {
      const int i = tid - HD;
      const uint32_t v = ld_u32<COH> ((const uint32_t *)vin + i);
      ((uint32_t *)(vc + (size_t)pos * HD))[i] = v;
      ((uint32_t *)qk)[HD + i] = v;
    }
  __syncthreads ();

  // scores[l] = fp16(dot(q, K[l]) / sqrt(HD)); LPR lanes share one cache row
  const int sub = tid % LPR, grp = tid / LPR;
  const float scale = 1.0f / sqrtf ((float)HD);
  const uint4 qv = ((const uint4 *)qk)[sub];
  for (int l0 = 0; l0 < L; l0 += RPB)
    {
      const int l = l0 + grp;
      float s = 0.f;
      if (l < L)
        {
          const uint4 kv = l == (int)pos
                               ? ((const uint4 *)(qk + HD))[sub]
                               : ((const uint4 *)(kc + (size_t)l * HD))[sub];
          s = dot8_f16 (qv, kv, 0.f);
        }
#pragma unroll
      for (int o = LPR >> 1; o > 0; o >>= 1)
        s += __shfl_xor (s, o, 64);
      if (l < L && sub == 0)
        sc[l] = h2f (f2h (s * scale + 0.f));
    }
  __syncthreads ();

  // softmax over the L scores; probabilities rounded to fp16
  float mx = -INFINITY;
  for (int l = tid; l < L; l += kDecThreads)
    mx = fmaxf (mx, sc[l]);
  mx = wave_max (mx);
  if ((tid & 63) == 0)
    red[kDecWaves + (tid >> 6)] = mx;
  __syncthreads ();
  mx = red[kDecWaves];
#pragma unroll
  for (int w = 1; w < kDecWaves; ++w)
    mx = fmaxf (mx, red[kDecWaves + w]);
  float sum = 0.f;
  for (int l = tid; l < L; l += kDecThreads)
    sum += expf (sc[l] - mx);
  sum = block_sum (sum, red);
  for (int l = tid; l < L; l += kDecThreads)
    sc[l] = h2f (f2h (expf (sc[l] - mx) / sum));
  __syncthreads ();

  // out[j] = fp16(sum_l P[l] V[l][j]); thread = (row group, 8 columns)
  float acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
    acc[j] = 0.f;
  for (int l = grp; l < L; l += RPB)
    {
      const float pl = sc[l];
      const uint4 vv = l == (int)pos
                           ? ((const uint4 *)(qk + 2 * HD))[sub]
                           : ((const uint4 *)(vc + (size_t)l * HD))[sub];
      const uint32_t w[4] = { vv.x, vv.y, vv.z, vv.w };
#pragma unroll
      for (int j = 0; j < 4; ++j)
        {
          acc[2 * j] += pl * h2f ((uint16_t)(w[j] & 0xffff));
          acc[2 * j + 1] += pl * h2f ((uint16_t)(w[j] >> 16));
        }
    }
#pragma unroll
  for (int j = 0; j < 8; ++j)
    part[grp * HD + sub * 8 + j] = acc[j];
  __syncthreads ();
  if (tid < HD / 2)
    {
      float o0 = 0.f, o1 = 0.f;
      for (int g = 0; g < RPB; ++g)
        {
          o0 += part[g * HD + 2 * tid];
          o1 += part[g * HD + 2 * tid + 1];
        }
      st_u32<COH> ((uint32_t *)(p.s.att + head * HD) + tid,
                   (uint32_t)f2h (o0) | ((uint32_t)f2h (o1) << 16));
    }
  __syncthreads ();
}

__host__ __device__ inline size_t
lds_bytes_needed (int dim, int ffn, int maxlen, int hd)
{
  const size_t kmax = (size_t)(dim > ffn ? dim : ffn);
  const size_t stage = ((kmax + 31) / 32 * 32) * 2 + 256;
  const size_t rpb = kDecThreads / (hd / 8);
  const size_t attn = 1024 + (size_t)maxlen * 4 + rpb * hd * 4 + 256;
  return stage > attn ? stage : attn;
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
  PH_ARGMAX
};

template <bool COH>
__device__ __forceinline__ void
run_phase (const Params &p, int layer, int phase, int wg, int G, uint8_t *lds)
{
  const vkl_decode_model &m = p.m;
  const int dim = m.dim, ffn = m.ffn;
  const int dimp = ((dim + 31) >> 5) << 5, ffnp = ((ffn + 31) >> 5) << 5;
  uint16_t *xl = (uint16_t *)lds;
  const int kstage = phase == PH_DOWN ? ffnp : dimp;
  float *red = (float *)(lds + (size_t)kstage * 2); // 2*kDecWaves floats
  Epilogue e = {};
  switch (phase)
    {
    case PH_KQV:
      {
        const vkl_layer_weights &lw = m.layers[layer];
        if (layer == 0)
          {
            uint32_t tok = p.tok[0];
            if (tok >= (uint32_t)m.vocab)
              tok = 0;
            stage_embed_q8 (qmat (m.tok_embd, m.vocab, dim), tok, dim, dimp, xl);
            __syncthreads ();
            if (wg == 0) // the residual stream starts as the embedding row
              for (int i = threadIdx.x; i < dim / 2; i += kDecThreads)
                st_u32<COH> ((uint32_t *)p.s.x + i, ((const uint32_t *)xl)[i]);
          }
        else
          {
            stage_raw<COH> (p.s.x, dim, dimp, xl);
            __syncthreads ();
          }
        norm_staged (xl, dim, lw.attn_norm, m.eps, red);
        const QMat mats[3] = { qmat (lw.wk, dim, dim), qmat (lw.wq, dim, dim),
                               qmat (lw.wv, dim, dim) };
        e.y[0] = p.s.kqv, e.y[1] = p.s.kqv + dim, e.y[2] = p.s.kqv + 2 * dim;
        gemv_phase<1, 3, COH> (mats, dim, dim, xl, e, wg, G, red);
        break;
      }
    case PH_ATTN:
      {
        const vkl_layer_weights &lw = m.layers[layer];
        for (int h = wg; h < m.n_heads; h += G)
          {
            if (m.head_dim == 128)
              attention_head<128, COH> (p, lw, h, lds);
            else
              attention_head<64, COH> (p, lw, h, lds);
          }
        break;
      }
    case PH_WO:
      {
        const vkl_layer_weights &lw = m.layers[layer];
        stage_raw<COH> (p.s.att, dim, dimp, xl);
        __syncthreads ();
        const QMat mats[1] = { qmat (lw.wo, dim, dim) };
        e.y[0] = p.s.x, e.residual = p.s.x;
        gemv_phase<0, 1, COH> (mats, dim, dim, xl, e, wg, G, red);
        break;
      }
    case PH_UPGATE:
      {
        const vkl_layer_weights &lw = m.layers[layer];
        stage_raw<COH> (p.s.x, dim, dimp, xl);
        __syncthreads ();
        norm_staged (xl, dim, lw.ffn_norm, m.eps, red);
        const QMat mats[2] = { qmat (lw.w_up, ffn, dim),
                               qmat (lw.w_gate, ffn, dim) };
        e.y[0] = p.s.t;
        gemv_phase<2, 2, COH> (mats, ffn, dim, xl, e, wg, G, red);
        break;
      }
    case PH_DOWN:
      {
        const vkl_layer_weights &lw = m.layers[layer];
        stage_raw<COH> (p.s.t, ffn, ffnp, xl);
        __syncthreads ();
        const QMat mats[1] = { qmat (lw.w_down, dim, ffn) };
        e.y[0] = p.s.x, e.residual = p.s.x;
        gemv_phase<0, 1, COH> (mats, dim, ffn, xl, e, wg, G, red);
        break;
      }
    case PH_HEAD:
      {
        stage_raw<COH> (p.s.x, dim, dimp, xl);
        __syncthreads ();
        norm_staged (xl, dim, m.output_norm, m.final_eps, red);
        const QMat mats[1] = { qmat (m.output, m.vocab, dim) };
        e.y[0] = p.s.logits16, e.y32 = p.logits32;
        e.amax_val = p.s.amax_val, e.amax_idx = p.s.amax_idx;
        gemv_phase<0, 1, COH> (mats, m.vocab, dim, xl, e, wg, G, red);
        break;
      }
    case PH_ARGMAX:
      {
        if (wg != 0 || !p.next_tok)
          break;
        // G partials -> first maximum
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
            p.next_tok[0] = idx;
          }
        break;
      }
    }
}

__global__ __launch_bounds__ (kDecThreads) void
decode_phase_kernel (const Params p, int layer, int phase)
{
  extern __shared__ __align__ (16) uint8_t lds[];
  run_phase<false> (p, layer, phase, (int)blockIdx.x, (int)gridDim.x, lds);
}

int
check_model (const vkl_decode_model *m)
{
  VKL_CHECK_ARG (m != nullptr);
  VKL_CHECK_ARG (m->wtype == 8);
  VKL_CHECK_ARG (m->dim > 0 && m->n_layers > 0 && m->n_heads > 0);
  VKL_CHECK_ARG (m->head_dim == 64 || m->head_dim == 128);
  VKL_CHECK_ARG (m->n_heads * m->head_dim == m->dim);
  VKL_CHECK_ARG ((m->dim % 32) == 0 && (m->ffn % 32) == 0 && m->ffn > 0);
  VKL_CHECK_ARG (m->vocab > 0 && (m->vocab % 2) == 0 && m->maxlen > 0);
  VKL_CHECK_ARG (m->layers && m->tok_embd && m->output && m->output_norm);
  VKL_CHECK_ARG (m->freqc && m->freqs && m->scratch);
  VKL_CHECK_ARG (lds_bytes_needed (m->dim, m->ffn, m->maxlen, m->head_dim)
                 <= 160 * 1024);
  return 0;
}
} // namespace
} // namespace vkl

using namespace vkl;

extern "C" size_t
vkl_decode_scratch_bytes (const vkl_decode_model *m)
{
  if (!m)
    return 0;
  return carve (nullptr, m->dim, m->ffn, m->vocab).bytes;
}

extern "C" const void *
vkl_decode_logits_f16 (const vkl_decode_model *m)
{
  if (!m || !m->scratch)
    return nullptr;
  return carve (m->scratch, m->dim, m->ffn, m->vocab).logits16;
}

extern "C" int
vkl_decode_step (const vkl_decode_model *m, const uint32_t *tok, uint32_t pos,
                 int mode, float *logits32, uint32_t *next_tok, void *stream)
{
  if (int e = check_model (m))
    return e;
  VKL_CHECK_ARG (tok != nullptr && pos < (uint32_t)m->maxlen);
  VKL_CHECK_ARG (mode == 0);
  static int n_cu = 0;
  static size_t lds_set = 0;
  if (n_cu == 0)
    {
      int dev = 0;
      VKL_HIP (hipGetDevice (&dev));
      VKL_HIP (hipDeviceGetAttribute (
          &n_cu, hipDeviceAttributeMultiprocessorCount, dev));
    }
  const size_t lds
      = lds_bytes_needed (m->dim, m->ffn, m->maxlen, m->head_dim);
  if (lds > lds_set)
    {
      VKL_HIP (hipFuncSetAttribute (
          (const void *)decode_phase_kernel,
          hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
      lds_set = lds;
    }
  Params p;
  p.m = *m;
  p.s = carve (m->scratch, m->dim, m->ffn, m->vocab);
  p.tok = tok;
  p.pos = pos;
  p.logits32 = logits32 ? logits32 : p.s.logits32;
  p.next_tok = next_tok;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid ((unsigned)n_cu), block (kDecThreads);
  for (int l = 0; l < m->n_layers; ++l)
    for (int ph = PH_KQV; ph <= PH_DOWN; ++ph)
      decode_phase_kernel<<<ph == PH_ATTN ? dim3 ((unsigned)m->n_heads) : grid,
                            block, lds, s>>> (p, l, ph);
  decode_phase_kernel<<<grid, block, lds, s>>> (p, 0, PH_HEAD);
  if (next_tok)
    decode_phase_kernel<<<dim3 (1), block, lds, s>>> (p, 0, PH_ARGMAX);
  return vkl_launch_status ();
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
