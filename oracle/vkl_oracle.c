/*
 * CPU oracle for the llama2 token loop -- TEST INFRASTRUCTURE ONLY.
 * See vkl_oracle.h.  Built with -ffp-contract=off so that every fp32
 * operation below rounds exactly as written.
 *
 * Summation order: the reference's dot-product shaders split a row over a
 * subgroup of 32 lanes laid out as [8 blocks, 4 sub-chunks] and combine the
 * lanes with subgroupAdd, whose order Vulkan leaves to the implementation.
 * The oracle keeps the per-lane order of the shader source and combines the
 * 32 lanes with a pairwise tree (lane i += lane i+s, s = 16,8,4,2,1).
 *
 * Pins: every function here is checked in tests/test_oracle_pins.py against
 * closed forms, invariants or fp64 brute force; the reference holds no golden
 * vectors for this path (its tests draw unseeded random inputs).
 * Parity unpinned (the reference cannot run here and never fixes them):
 *   - the fp16 rounding of a freshly quantised Q8_0 scale (RNE chosen);
 *   - FP16 Q/K/V projections (the reference always runs the Q8_0 shader);
 *   - the cross-lane order of subgroupAdd;
 *   - tie order of the host std::sort sampler (lowest index chosen).
 */
#include "vkl_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef __F16C__
#include <immintrin.h>
#endif

/* ------------------------------------------------------------------------ */
/* fp16                                                                      */
/* ------------------------------------------------------------------------ */
typedef union
{
  uint32_t u;
  float f;
} fu32;

uint16_t
vko_f32_to_f16 (float f)
{
  fu32 v, magic;
  v.f = f;
  uint32_t sign = (v.u >> 16) & 0x8000u;
  v.u &= 0x7fffffffu;
  uint16_t o;
  if (v.u >= ((127u + 16u) << 23)) /* >= 65536, inf or nan */
    {
      o = (v.u > (255u << 23)) ? 0x7e00 : 0x7c00;
    }
  else if (v.u < (113u << 23)) /* result is subnormal or zero */
    {
      magic.u = ((127u - 15u) + (23u - 10u) + 1u) << 23;
      v.f += magic.f; /* the fp32 add performs the RNE rounding */
      o = (uint16_t)(v.u - magic.u);
    }
  else
    {
      uint32_t mant_odd = (v.u >> 13) & 1u;
      v.u += ((uint32_t)(15 - 127) << 23) + 0xfffu;
      v.u += mant_odd;
      o = (uint16_t)(v.u >> 13);
    }
  return (uint16_t)(o | sign);
}

uint16_t
vko_f32_to_f16_hw (float f)
{
#ifdef __F16C__
  return (uint16_t)_cvtss_sh (f, _MM_FROUND_TO_NEAREST_INT);
#else
  return vko_f32_to_f16 (f);
#endif
}

static float f16_table[65536];
static int f16_table_ready = 0;

static float
f16_to_f32_slow (uint16_t h)
{
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1f;
  uint32_t frac = h & 0x3ffu;
  fu32 v;
  if (exp == 0)
    {
      /* subnormal: frac * 2^-24, exact in fp32 */
      v.f = (float)frac * 5.9604644775390625e-8f;
      v.u |= sign;
    }
  else if (exp == 0x1f)
    {
      v.u = sign | 0x7f800000u | (frac << 13);
    }
  else
    {
      v.u = sign | ((exp - 15 + 127) << 23) | (frac << 13);
    }
  return v.f;
}

static void
f16_table_init (void)
{
  if (f16_table_ready)
    return;
  for (uint32_t i = 0; i < 65536; ++i)
    f16_table[i] = f16_to_f32_slow ((uint16_t)i);
  __atomic_store_n (&f16_table_ready, 1, __ATOMIC_RELEASE);
}

__attribute__ ((constructor)) static void
vko_init (void)
{
  f16_table_init ();
}

float
vko_f16_to_f32 (uint16_t h)
{
  return f16_table[h];
}

#define H2F(h) (f16_table[(h)])
#define F2H(f) vko_f32_to_f16_hw (f)

/* src/core/float.h:52-112: truncates the mantissa, clamps to max normal. */
uint16_t
vko_ref_host_f32_to_f16 (float f)
{
  fu32 v;
  v.f = f;
  uint16_t sign = (uint16_t)((v.u >> 16) & 0x8000u);
  uint32_t exp = (v.u >> 23) & 0xff, frac = v.u & 0x7fffffu;
  float a = fabsf (f);
  if (exp == 0 && frac == 0)
    return sign;
  if (isnan (f))
    return (uint16_t)(sign | 0x7c00 | 1);
  if (isinf (f))
    return (uint16_t)(sign | 0x7c00);
  if (a > 65504.0f)
    return (uint16_t)(sign | (0x1e << 10) | 1023);
  if (a < 5.96046448e-8f)
    return 0;
  if (a < 6.103515625e-5)
    return (uint16_t)(sign | (((frac >> 14) + 512) & 0x3ff));
  return (uint16_t)(sign | ((exp - 127 + 15) << 10) | (frac >> 13));
}

/* ------------------------------------------------------------------------ */
/* Q8_0                                                                      */
/* ------------------------------------------------------------------------ */
void
vko_q8_0_quantize_row (const float *src, size_t n, uint8_t *dst,
                       int scale_bytes)
{
  size_t nb = (n + VKO_Q8_0_BLOCK - 1) / VKO_Q8_0_BLOCK;
  for (size_t b = 0; b < nb; ++b)
    {
      size_t start = b * VKO_Q8_0_BLOCK, end = start + VKO_Q8_0_BLOCK;
      float amax = fabsf (src[start]);
      for (size_t i = start; i < end && i < n; ++i)
        {
          float a = fabsf (src[i]);
          amax = a > amax ? a : amax;
        }
      float scale = amax / 127.0f;
      float inv = scale > 0 ? 127.0f / amax : 0.0f;
      if (scale_bytes == 4)
        {
          memcpy (dst, &scale, 4);
          dst += 4;
        }
      else
        {
          uint16_t h = vko_f32_to_f16 (scale);
          memcpy (dst, &h, 2);
          dst += 2;
        }
      for (size_t i = start; i < end; ++i)
        {
          int8_t q = 0;
          if (i < n)
            q = (int8_t)roundf (src[i] * inv);
          *dst++ = (uint8_t)q;
        }
    }
}

void
vko_q8_0_dequantize_row (const uint8_t *src, size_t n, float *dst,
                         int scale_bytes)
{
  size_t nb = (n + VKO_Q8_0_BLOCK - 1) / VKO_Q8_0_BLOCK;
  size_t bb = (size_t)scale_bytes + VKO_Q8_0_BLOCK;
  for (size_t b = 0; b < nb; ++b)
    {
      const uint8_t *blk = src + b * bb;
      float d;
      if (scale_bytes == 4)
        memcpy (&d, blk, 4);
      else
        {
          uint16_t h;
          memcpy (&h, blk, 2);
          d = H2F (h);
        }
      const int8_t *q = (const int8_t *)(blk + scale_bytes);
      for (size_t i = 0; i < VKO_Q8_0_BLOCK; ++i)
        {
          size_t o = b * VKO_Q8_0_BLOCK + i;
          if (o >= n)
            break;
          dst[o] = (float)q[i] * d;
        }
    }
}

static inline float
blk_scale (const uint8_t *blk)
{
  uint16_t h;
  memcpy (&h, blk, 2);
  return H2F (h);
}

/* ------------------------------------------------------------------------ */
/* embedding                                                                 */
/* ------------------------------------------------------------------------ */
void
vko_embedding_q8_0 (const uint8_t *table, uint32_t VH, uint32_t VW,
                    const uint32_t *toks, uint32_t n, uint32_t unk,
                    uint16_t *out)
{
  uint32_t nb = (VW + VKO_Q8_0_BLOCK - 1) / VKO_Q8_0_BLOCK;
  for (uint32_t t = 0; t < n; ++t)
    {
      uint32_t tok = toks[t];
      if (tok >= VH)
        tok = unk;
      const uint8_t *row = table + (size_t)tok * nb * VKO_Q8_0_BYTES;
      for (uint32_t b = 0; b < nb; ++b)
        {
          const uint8_t *blk = row + (size_t)b * VKO_Q8_0_BYTES;
          float d = blk_scale (blk);
          const int8_t *q = (const int8_t *)(blk + 2);
          for (uint32_t i = 0; i < VKO_Q8_0_BLOCK; ++i)
            {
              uint32_t o = b * VKO_Q8_0_BLOCK + i;
              if (o >= VW)
                break;
              out[(size_t)t * VW + o] = F2H ((float)q[i] * d);
            }
        }
    }
}

void
vko_embedding_f16 (const uint16_t *table, uint32_t VH, uint32_t VW,
                   const uint32_t *toks, uint32_t n, uint32_t unk,
                   uint16_t *out)
{
  for (uint32_t t = 0; t < n; ++t)
    {
      uint32_t tok = toks[t];
      if (tok >= VH)
        tok = unk;
      memcpy (out + (size_t)t * VW, table + (size_t)tok * VW,
              (size_t)VW * 2);
    }
}

/* ------------------------------------------------------------------------ */
/* RMSNorm                                                                   */
/* ------------------------------------------------------------------------ */
void
vko_rmsnorm_f16 (const uint16_t *x, const float *w, int rows, int W,
                 float eps, uint16_t *out)
{
  enum { T = 512 }; /* src/shaders/rms_norm_conf.h:3 */
  for (int r = 0; r < rows; ++r)
    {
      const uint16_t *xr = x + (size_t)r * W;
      float sum[T];
      for (int t = 0; t < T; ++t)
        {
          float s = 0.f;
          for (int i = t; i < W; i += T)
            {
              float v = H2F (xr[i]);
              s += v * v;
            }
          sum[t] = s;
        }
      for (int i = T / 2; i > 0; i /= 2)
        for (int t = 0; t < i; ++t)
          sum[t] += sum[t + i];
      float alpha = 1.0f / sqrtf (sum[0] / (float)W + eps);
      for (int i = 0; i < W; ++i)
        {
          float v = H2F (xr[i]);
          out[(size_t)r * W + i] = F2H (v * w[i] * alpha);
        }
    }
}

/* ------------------------------------------------------------------------ */
/* dot-product kernels                                                       */
/* ------------------------------------------------------------------------ */
/* The shaders combine the 32 lanes of a subgroup with subgroupAdd, whose
 * order of additions Vulkan leaves to the implementation.  Order 0 (the
 * default, and the one every fixture is written with) halves the lanes
 * pairwise; 1 adds them one after the other; 2 pairs neighbours first (the
 * butterfly a cross-lane reduction in hardware makes); 3 adds them one after
 * the other from the last lane down; 4 adds four groups of eight lanes
 * sequentially and then the groups.  The switch exists for
 * tests that ask how far the reference's own freedom moves a result. */
static int g_lane_order = 0;

void
vko_set_lane_order (int order)
{
  g_lane_order = order;
}

static inline float
lanes32_add (float *l)
{
  if (g_lane_order == 1)
    {
      float s = l[0];
      for (int i = 1; i < 32; ++i)
        s += l[i];
      return s;
    }
  if (g_lane_order == 2)
    {
      for (int s = 1; s < 32; s <<= 1)
        for (int i = 0; i < 32; i += 2 * s)
          l[i] += l[i + s];
      return l[0];
    }
  if (g_lane_order == 3)
    {
      float s = l[31];
      for (int i = 30; i >= 0; --i)
        s += l[i];
      return s;
    }
  if (g_lane_order == 4)
    {
      /* four quads of eight lanes one after the other, then the quads */
      float q[4];
      for (int g = 0; g < 4; ++g)
        {
          q[g] = l[8 * g];
          for (int i = 1; i < 8; ++i)
            q[g] += l[8 * g + i];
        }
      return (q[0] + q[1]) + (q[2] + q[3]);
    }
  for (int s = 16; s > 0; s >>= 1)
    for (int i = 0; i < s; ++i)
      l[i] += l[i + s];
  return l[0];
}

static inline float
act_apply (float v, int act)
{
  return act == 1 ? v / (1.0f + expf (-v)) : v;
}

/* one Q8_0 row against an fp32 copy of the activation row (padded with
 * zeros to nb*32): lane (bi%8, il) accumulates sum_8(a*q) * d */
static inline float
q8_row_dot (const float *af, const uint8_t *row, int nb)
{
  float lane[32];
  for (int i = 0; i < 32; ++i)
    lane[i] = 0.f;
  for (int bi = 0; bi < nb; ++bi)
    {
      const uint8_t *blk = row + (size_t)bi * VKO_Q8_0_BYTES;
      float d = blk_scale (blk);
      const int8_t *q = (const int8_t *)(blk + 2);
      const float *a = af + (size_t)bi * 32;
      int ix = bi & 7;
      for (int il = 0; il < 4; ++il)
        {
          float sum_b = 0.f;
          for (int i = 0; i < 8; ++i)
            sum_b += a[il * 8 + i] * (float)q[il * 8 + i];
          lane[ix * 4 + il] += sum_b * d;
        }
    }
  return lanes32_add (lane);
}

static float *
act_row_f32 (const uint16_t *x, int K, int nb)
{
  float *af = (float *)malloc ((size_t)nb * 32 * sizeof (float));
  for (int k = 0; k < nb * 32; ++k)
    af[k] = k < K ? H2F (x[k]) : 0.f;
  return af;
}

void
vko_matmul_q8_0 (const uint16_t *x, const uint8_t *w, int M, int N, int K,
                 float scale, float bias, int act, uint16_t *y)
{
  int nb = (K + 31) / 32;
  for (int m = 0; m < M; ++m)
    {
      float *af = act_row_f32 (x + (size_t)m * K, K, nb);
#pragma omp parallel for schedule(static)
      for (int n = 0; n < N; ++n)
        {
          float s = q8_row_dot (af, w + (size_t)n * nb * VKO_Q8_0_BYTES, nb);
          float v = s * scale + bias;
          y[(size_t)m * N + n] = F2H (act_apply (v, act));
        }
      free (af);
    }
}

void
vko_kqv_q8_0 (const uint16_t *x, const uint8_t *wk, const uint8_t *wq,
              const uint8_t *wv, int M, int N, int K, uint16_t *k,
              uint16_t *q, uint16_t *v)
{
  int nb = (K + 31) / 32;
  size_t rb = (size_t)nb * VKO_Q8_0_BYTES;
  for (int m = 0; m < M; ++m)
    {
      float *af = act_row_f32 (x + (size_t)m * K, K, nb);
#pragma omp parallel for schedule(static)
      for (int n = 0; n < N; ++n)
        {
          k[(size_t)m * N + n] = F2H (q8_row_dot (af, wk + n * rb, nb));
          q[(size_t)m * N + n] = F2H (q8_row_dot (af, wq + n * rb, nb));
          v[(size_t)m * N + n] = F2H (q8_row_dot (af, wv + n * rb, nb));
        }
      free (af);
    }
}

void
vko_ffn_upgate_q8_0 (const uint16_t *x, const uint8_t *wup,
                     const uint8_t *wgate, int M, int N, int K, uint16_t *out)
{
  int nb = (K + 31) / 32;
  size_t rb = (size_t)nb * VKO_Q8_0_BYTES;
  for (int m = 0; m < M; ++m)
    {
      float *af = act_row_f32 (x + (size_t)m * K, K, nb);
#pragma omp parallel for schedule(static)
      for (int n = 0; n < N; ++n)
        {
          float up = q8_row_dot (af, wup + n * rb, nb);
          float g = q8_row_dot (af, wgate + n * rb, nb);
          /* ffn_up_and_gate_q8_0.comp:127-128 */
          float v = g / (1.0f + expf (-g)) * up;
          out[(size_t)m * N + n] = F2H (v);
        }
      free (af);
    }
}

/* matmul_b0_tb_fp16_v2.comp:61-110: K in blocks of 64, lane (bi%8, il) sums
 * 16 products then adds into its accumulator.  The shader has no K tail
 * guard; the oracle treats elements past K as zero. */
static inline float
f16_row_dot_tb (const float *af, const uint16_t *b, int K)
{
  float lane[32];
  for (int i = 0; i < 32; ++i)
    lane[i] = 0.f;
  int nb = (K + 63) / 64;
  for (int bi = 0; bi < nb; ++bi)
    {
      int ix = bi & 7;
      for (int il = 0; il < 4; ++il)
        {
          float sum_b = 0.f;
          int base = bi * 64 + il * 16;
          for (int i = 0; i < 16; ++i)
            {
              int k = base + i;
              if (k < K)
                sum_b += af[k] * H2F (b[k]);
            }
          lane[ix * 4 + il] += sum_b;
        }
    }
  return lanes32_add (lane);
}

void
vko_matmul_f16_tb (const uint16_t *a, const uint16_t *b, int C, int M, int N,
                   int K, size_t acs, size_t ahs, size_t bcs, size_t bhs,
                   float scale, float bias, int act, uint16_t *y)
{
  for (int c = 0; c < C; ++c)
    for (int m = 0; m < M; ++m)
      {
        const uint16_t *ar = a + c * acs + m * ahs;
        float *af = (float *)malloc ((size_t)K * sizeof (float));
        for (int k = 0; k < K; ++k)
          af[k] = H2F (ar[k]);
#pragma omp parallel for schedule(static) if (N >= 256)
        for (int n = 0; n < N; ++n)
          {
            float s = f16_row_dot_tb (af, b + c * bcs + n * bhs, K);
            float v = s * scale + bias;
            y[((size_t)c * M + m) * N + n] = F2H (act_apply (v, act));
          }
        free (af);
      }
}

/* matmul_broadcast0_fp16_v2.comp:52-104, transpose_b == 0: lane i strides K
 * by 32, four at a time through dot(vec4, vec4), then a scalar tail. */
void
vko_matmul_f16_nn (const uint16_t *a, const uint16_t *b, int C, int M, int N,
                   int K, size_t acs, size_t ahs, size_t bcs, size_t bhs,
                   float scale, float bias, int act, uint16_t *y)
{
  for (int c = 0; c < C; ++c)
    for (int m = 0; m < M; ++m)
      {
        const uint16_t *ar = a + c * acs + m * ahs;
#pragma omp parallel for schedule(static) if (N >= 256)
        for (int n = 0; n < N; ++n)
          {
            const uint16_t *bc = b + c * bcs + n;
            float lane[32];
            for (int l = 0; l < 32; ++l)
              {
                float sum = 0.f;
                int i = l;
                for (; i + 3 * 32 < K; i += 4 * 32)
                  {
                    float d = H2F (ar[i]) * H2F (bc[(size_t)i * bhs]);
                    d += H2F (ar[i + 32]) * H2F (bc[(size_t)(i + 32) * bhs]);
                    d += H2F (ar[i + 64]) * H2F (bc[(size_t)(i + 64) * bhs]);
                    d += H2F (ar[i + 96]) * H2F (bc[(size_t)(i + 96) * bhs]);
                    sum += d;
                  }
                for (; i < K; i += 32)
                  sum += H2F (ar[i]) * H2F (bc[(size_t)i * bhs]);
                lane[l] = sum;
              }
            float v = lanes32_add (lane) * scale + bias;
            y[((size_t)c * M + m) * N + n] = F2H (act_apply (v, act));
          }
      }
}

void
vko_ffn_upgate_f16 (const uint16_t *x, const uint16_t *wup,
                    const uint16_t *wgate, int M, int N, int K, uint16_t *out)
{
  for (int m = 0; m < M; ++m)
    {
      float *af = (float *)malloc ((size_t)K * sizeof (float));
      for (int k = 0; k < K; ++k)
        af[k] = H2F (x[(size_t)m * K + k]);
#pragma omp parallel for schedule(static)
      for (int n = 0; n < N; ++n)
        {
          float up = f16_row_dot_tb (af, wup + (size_t)n * K, K);
          float g = f16_row_dot_tb (af, wgate + (size_t)n * K, K);
          float v = g / (1.0f + expf (-g)) * up;
          out[(size_t)m * N + n] = F2H (v);
        }
      free (af);
    }
}

/* ------------------------------------------------------------------------ */
/* RoPE, KV cache, softmax, element-wise, argmax, transpose                  */
/* ------------------------------------------------------------------------ */
void
vko_rope_tables (int maxlen, int dim, float *freqc, float *freqs)
{
  int half = dim / 2;
  float *freq = (float *)malloc ((size_t)half * sizeof (float));
  float n = 0.f;
  for (int k = 0; k < half; ++k)
    {
      freq[k] = 1.0f / powf (10000.0f, n / (float)dim);
      n += 2.0f;
    }
  for (int i = 0; i < maxlen; ++i)
    for (int k = 0; k < half; ++k)
      {
        float f = freq[k] * (float)i;
        freqc[(size_t)i * half + k] = cosf (f);
        freqs[(size_t)i * half + k] = sinf (f);
      }
  free (freq);
}

void
vko_rope_f16 (uint16_t *x, int C, int H, int W, const float *freqc,
              const float *freqs, uint32_t offset)
{
  int half = W / 2;
  for (int c = 0; c < C; ++c)
    for (int y = 0; y < H; ++y)
      for (int i = 0; i < half; ++i)
        {
          size_t fi = ((size_t)y + offset) * half + i;
          float fc = freqc[fi], fs = freqs[fi];
          size_t i0 = ((size_t)c * H + y) * W + 2 * i, i1 = i0 + 1;
          float q0 = H2F (x[i0]), q1 = H2F (x[i1]);
          float r0 = q0 * fc - q1 * fs;
          float r1 = q0 * fs + q1 * fc;
          x[i0] = F2H (r0);
          x[i1] = F2H (r1);
        }
}

void
vko_update_kvcache_f16 (uint16_t *cache, const uint16_t *kv, int C, int HO,
                        int H, int W, uint32_t offset)
{
  for (int c = 0; c < C; ++c)
    for (int y = 0; y < H; ++y)
      {
        uint32_t uy = (offset + (uint32_t)y) % (uint32_t)HO;
        memcpy (cache + ((size_t)c * HO + uy) * W,
                kv + ((size_t)c * H + y) * W, (size_t)W * 2);
      }
}

void
vko_softmax_f16 (const uint16_t *x, int C, int H, int W, int seq_mask,
                 uint32_t offset, uint16_t *out)
{
  for (int c = 0; c < C; ++c)
    for (int y = 0; y < H; ++y)
      {
        const uint16_t *r = x + ((size_t)c * H + y) * W;
        uint16_t *o = out + ((size_t)c * H + y) * W;
        /* the maximum covers masked entries as well (softmax_fp16.comp:37-46) */
        float mx = H2F (r[0]);
        for (int i = 0; i < W; ++i)
          {
            float v = H2F (r[i]);
            mx = v > mx ? v : mx;
          }
        float lane[32];
        for (int l = 0; l < 32; ++l)
          {
            float s = 0.f;
            for (int i = l; i < W; i += 32)
              {
                if (seq_mask > 0 && (uint32_t)i > (uint32_t)y + offset)
                  continue;
                s += expf (H2F (r[i]) - mx);
              }
            lane[l] = s;
          }
        float sum = lanes32_add (lane);
        for (int i = 0; i < W; ++i)
          {
            if (seq_mask > 0 && (uint32_t)i > (uint32_t)y + offset)
              o[i] = 0;
            else
              o[i] = F2H (expf (H2F (r[i]) - mx) / sum);
          }
      }
}

void
vko_elementwise_f16 (const uint16_t *x, const uint16_t *y, size_t n, int op,
                     uint16_t *out)
{
  for (size_t i = 0; i < n; ++i)
    {
      float a = H2F (x[i]), b = H2F (y[i]), v;
      switch (op)
        {
        case 0: v = a + b; break;
        case 1: v = a - b; break;
        case 2: v = a * b; break;
        default: v = a / b; break;
        }
      out[i] = F2H (v);
    }
}

void
vko_argmax_f16 (const uint16_t *x, int rows, int W, uint32_t *out)
{
  for (int r = 0; r < rows; ++r)
    {
      const uint16_t *xr = x + (size_t)r * W;
      float best = H2F (xr[0]);
      uint32_t bi = 0;
      for (int i = 1; i < W; ++i)
        {
          float v = H2F (xr[i]);
          if (v > best)
            {
              best = v;
              bi = (uint32_t)i;
            }
        }
      out[r] = bi;
    }
}

uint32_t
vko_argmax_f32 (const float *x, int n)
{
  float best = x[0];
  uint32_t bi = 0;
  for (int i = 1; i < n; ++i)
    if (x[i] > best)
      {
        best = x[i];
        bi = (uint32_t)i;
      }
  return bi;
}

void
vko_transpose102_f16 (const uint16_t *x, int C, int H, int W, uint16_t *out)
{
  for (int c = 0; c < C; ++c)
    for (int h = 0; h < H; ++h)
      memcpy (out + ((size_t)h * C + c) * W, x + ((size_t)c * H + h) * W,
              (size_t)W * 2);
}

/* ------------------------------------------------------------------------ */
/* model                                                                     */
/* ------------------------------------------------------------------------ */
struct vko_state
{
  int n_layers, heads, hd, maxlen, dim;
  uint16_t **kc, **vc; /* [heads, maxlen, hd] per layer */
  float *freqc, *freqs;
  uint16_t *hidden;
  int hidden_rows;
};

vko_state *
vko_state_create (const vko_model *m)
{
  vko_state *s = (vko_state *)calloc (1, sizeof (*s));
  s->n_layers = m->n_layers;
  s->heads = m->n_heads;
  s->hd = m->head_dim;
  s->maxlen = m->maxlen;
  s->dim = m->dim;
  s->kc = (uint16_t **)calloc ((size_t)m->n_layers, sizeof (void *));
  s->vc = (uint16_t **)calloc ((size_t)m->n_layers, sizeof (void *));
  size_t n = (size_t)m->n_heads * m->maxlen * m->head_dim;
  for (int l = 0; l < m->n_layers; ++l)
    {
      s->kc[l] = (uint16_t *)calloc (n, 2);
      s->vc[l] = (uint16_t *)calloc (n, 2);
    }
  /* src/ops/rope.cpp:73-92 builds 2*maxlen rows and uploads the first half
   * of the bytes, i.e. rows [0, maxlen). */
  size_t tn = (size_t)m->maxlen * (m->head_dim / 2);
  s->freqc = (float *)malloc (tn * sizeof (float));
  s->freqs = (float *)malloc (tn * sizeof (float));
  vko_rope_tables (m->maxlen, m->head_dim, s->freqc, s->freqs);
  return s;
}

void
vko_state_destroy (vko_state *s)
{
  if (!s)
    return;
  for (int l = 0; l < s->n_layers; ++l)
    {
      free (s->kc[l]);
      free (s->vc[l]);
    }
  free (s->kc);
  free (s->vc);
  free (s->freqc);
  free (s->freqs);
  free (s->hidden);
  free (s);
}

const uint16_t *
vko_state_kcache (const vko_state *s, int layer)
{
  return s->kc[layer];
}

const uint16_t *
vko_state_vcache (const vko_state *s, int layer)
{
  return s->vc[layer];
}

const uint16_t *
vko_state_hidden (const vko_state *s, int *rows)
{
  if (rows)
    *rows = s->hidden_rows;
  return s->hidden;
}

static void
linear (const vko_model *m, const uint16_t *x, const void *w, int M, int N,
        int K, uint16_t *y)
{
  if (m->wtype == 8)
    vko_matmul_q8_0 (x, (const uint8_t *)w, M, N, K, 1.0f, 0.f, 0, y);
  else
    vko_matmul_f16_tb (x, (const uint16_t *)w, 1, M, N, K, 0, (size_t)K, 0,
                       (size_t)K, 1.0f, 0.f, 0, y);
}

/* src/ops/multiheadattention_v2.cpp:140-325 */
static void
attention (const vko_model *m, vko_state *s, int layer, const uint16_t *x,
           int S, size_t offset, int clip, uint16_t *out /* [S|1, dim] */)
{
  int d = m->dim, H = m->n_heads, hd = m->head_dim, maxlen = m->maxlen;
  size_t n = (size_t)S * d;
  uint16_t *k = (uint16_t *)malloc (n * 2), *q = (uint16_t *)malloc (n * 2),
           *v = (uint16_t *)malloc (n * 2);
  if (m->wtype == 8)
    vko_kqv_q8_0 (x, (const uint8_t *)m->wk[layer],
                  (const uint8_t *)m->wq[layer],
                  (const uint8_t *)m->wv[layer], S, d, d, k, q, v);
  else
    {
      /* the reference has no FP16 KQV shader; defined here as three
       * matmul_b0_tb_fp16_v2 products (parity unpinned) */
      linear (m, x, m->wk[layer], S, d, d, k);
      linear (m, x, m->wq[layer], S, d, d, q);
      linear (m, x, m->wv[layer], S, d, d, v);
    }
  /* [S, H, hd] -> (clip: last row of q) -> [H, S|1, hd] */
  int Sq = clip ? 1 : S;
  uint16_t *kt = (uint16_t *)malloc (n * 2), *vt = (uint16_t *)malloc (n * 2),
           *qt = (uint16_t *)malloc ((size_t)Sq * d * 2);
  vko_transpose102_f16 (k, S, H, hd, kt);
  vko_transpose102_f16 (v, S, H, hd, vt);
  vko_transpose102_f16 (clip ? q + (size_t)(S - 1) * d : q, Sq, H, hd, qt);
  /* rope: row y of the tensor handed to the op uses position y + offset;
   * after the clip the single query row is row 0 (reference quirk) */
  uint32_t qoff = (uint32_t)offset;
  if (clip && !m->lastblock_rope_quirk)
    qoff = (uint32_t)(offset + S - 1);
  vko_rope_f16 (qt, H, Sq, hd, s->freqc, s->freqs, qoff);
  vko_rope_f16 (kt, H, S, hd, s->freqc, s->freqs, (uint32_t)offset);
  vko_update_kvcache_f16 (s->kc[layer], kt, H, maxlen, S, hd,
                          (uint32_t)offset);
  vko_update_kvcache_f16 (s->vc[layer], vt, H, maxlen, S, hd,
                          (uint32_t)offset);
  int L = (offset + (size_t)S) < (size_t)maxlen ? (int)(offset + (size_t)S) : maxlen;
  uint16_t *sc = (uint16_t *)malloc ((size_t)H * Sq * L * 2);
  uint16_t *pr = (uint16_t *)malloc ((size_t)H * Sq * L * 2);
  float scale = 1.0f / sqrtf ((float)hd);
  vko_matmul_f16_tb (qt, s->kc[layer], H, Sq, L, hd, (size_t)Sq * hd,
                     (size_t)hd, (size_t)maxlen * hd, (size_t)hd, scale, 0.f,
                     0, sc);
  vko_softmax_f16 (sc, H, Sq, L, 1, (uint32_t)(L - Sq), pr);
  uint16_t *ho = (uint16_t *)malloc ((size_t)H * Sq * hd * 2);
  vko_matmul_f16_nn (pr, s->vc[layer], H, Sq, hd, L, (size_t)Sq * L,
                     (size_t)L, (size_t)maxlen * hd, (size_t)hd, 1.0f, 0.f, 0,
                     ho);
  uint16_t *cat = (uint16_t *)malloc ((size_t)Sq * d * 2);
  vko_transpose102_f16 (ho, H, Sq, hd, cat);
  linear (m, cat, m->wo[layer], Sq, d, d, out);
  free (k); free (q); free (v); free (kt); free (vt); free (qt);
  free (sc); free (pr); free (ho); free (cat);
}

int
vko_forward (const vko_model *m, vko_state *s, const uint32_t *toks,
             int n_toks, size_t offset, float *logits)
{
  int d = m->dim, S = n_toks, F = m->ffn;
  if (S <= 0 || offset + (size_t)S > (size_t)m->maxlen)
    return -1;
  uint16_t *x = (uint16_t *)malloc ((size_t)S * d * 2);
  uint16_t *nrm = (uint16_t *)malloc ((size_t)S * d * 2);
  uint16_t *att = (uint16_t *)malloc ((size_t)S * d * 2);
  uint16_t *t = (uint16_t *)malloc ((size_t)S * F * 2);
  uint16_t *ff = (uint16_t *)malloc ((size_t)S * d * 2);
  if (m->wtype == 8)
    vko_embedding_q8_0 ((const uint8_t *)m->tok_embd, (uint32_t)m->vocab,
                        (uint32_t)d, toks, (uint32_t)S, 0, x);
  else
    vko_embedding_f16 ((const uint16_t *)m->tok_embd, (uint32_t)m->vocab,
                       (uint32_t)d, toks, (uint32_t)S, 0, x);
  int rows = S;
  for (int l = 0; l < m->n_layers; ++l)
    {
      int clip = (l == m->n_layers - 1);
      /* models/llama2.h:160-213 */
      vko_rmsnorm_f16 (x, m->attn_norm[l], rows, d, m->eps, nrm);
      attention (m, s, l, nrm, rows, offset, clip, att);
      uint16_t *res = x;
      if (clip)
        {
          res = x + (size_t)(rows - 1) * d;
          rows = 1;
        }
      /* added = fp16(attn + in), written into the residual operand */
      vko_elementwise_f16 (att, res, (size_t)rows * d, 0, x);
      vko_rmsnorm_f16 (x, m->ffn_norm[l], rows, d, m->eps, nrm);
      if (m->wtype == 8)
        vko_ffn_upgate_q8_0 (nrm, (const uint8_t *)m->w_up[l],
                             (const uint8_t *)m->w_gate[l], rows, F, d, t);
      else
        vko_ffn_upgate_f16 (nrm, (const uint16_t *)m->w_up[l],
                            (const uint16_t *)m->w_gate[l], rows, F, d, t);
      linear (m, t, m->w_down[l], rows, d, F, ff);
      vko_elementwise_f16 (ff, x, (size_t)rows * d, 0, x);
    }
  free (s->hidden);
  s->hidden = (uint16_t *)malloc ((size_t)rows * d * 2);
  memcpy (s->hidden, x, (size_t)rows * d * 2);
  s->hidden_rows = rows;
  /* models/llama2.h:283-298 */
  vko_rmsnorm_f16 (x, m->output_norm, rows, d, m->final_eps, nrm);
  uint16_t *lg = (uint16_t *)malloc ((size_t)rows * m->vocab * 2);
  linear (m, nrm, m->output, rows, m->vocab, d, lg);
  for (int i = 0; i < m->vocab; ++i)
    logits[i] = H2F (lg[(size_t)(rows - 1) * m->vocab + i]);
  free (lg); free (x); free (nrm); free (att); free (t); free (ff);
  return 0;
}

int
vko_generate_greedy (const vko_model *m, vko_state *s, const uint32_t *prompt,
                     int n_prompt, int n_gen, uint32_t *out_ids,
                     float *first_logits)
{
  float *logits = (float *)malloc ((size_t)m->vocab * sizeof (float));
  int rc = vko_forward (m, s, prompt, n_prompt, 0, logits);
  if (rc)
    {
      free (logits);
      return rc;
    }
  if (first_logits)
    memcpy (first_logits, logits, (size_t)m->vocab * sizeof (float));
  int n_toks = n_prompt;
  uint32_t tok = vko_argmax_f32 (logits, m->vocab);
  out_ids[0] = tok;
  ++n_toks;
  for (int i = 1; i < n_gen; ++i)
    {
      /* app/llama2_infer.cpp:168-176: model({last}, toks.size()-1) */
      rc = vko_forward (m, s, &tok, 1, (size_t)(n_toks - 1), logits);
      if (rc)
        break;
      tok = vko_argmax_f32 (logits, m->vocab);
      out_ids[i] = tok;
      ++n_toks;
    }
  free (logits);
  return rc;
}
