// Attention of many query rows over the K/V rows of a prompt, one kernel per
// call: scores, masked softmax and the product with V without the [H, S, L]
// score and probability tensors ever reaching memory.
//
// One pass over the keys with a running maximum (online softmax): per tile of
// 64 keys the scores are formed (rounded to fp16 like the stand-alone product:
// score = fp16(scale * q.k)), the maximum m is raised if needed - the products
// accumulated so far and the sum of exponentials are then multiplied by
// exp(m_old - m_new) -, the weights fp16(exp(score - m)) go into the second
// product as they are, and the division by the sum of exponentials comes last,
// in fp32, before the one rounding of the output.  The separate operators round
// the NORMALISED probability to fp16 instead (p = fp16(exp(score - max) / sum));
// the two differ by at most two half-ulp roundings of a weight, i.e. by
// 2 * 2^-12 * sum_l p[l] |v[l]|, inside the 1e-2 the outputs are held to.  (A first
// version walked the keys twice - maximum and sum first, then the very
// probabilities of the operators - and took twice as long: two exponentials
// per score and the scores computed twice.)
//
// Workgroup = 4 waves = 128 query rows of one head, 32 per wave; the keys come
// through LDS in tiles of 64.  Both products run on v_mfma_f32_32x32x16_f16 in
// the transposed form, so that a lane's accumulator registers belong to ONE
// query:
//   S^T[key, q] = sum_d K[key, d] Q[q, d]      A = K tile (LDS), B = Q (regs)
//   O^T[d, q]   = sum_key V^T[d, key] P^T[key, q]   A = V^T tile (LDS), B = P^T
// Lane l of a wave owns query l % 32.  Of a 32-key block its 16 accumulator
// registers hold the keys 8*(r/4) + 4*(l/32) + r%4, so maximum and sum over
// keys are sums over a lane's own registers (the two lane halves are merged
// after every tile), and the weights it forms are, as they lie, the B
// operand of the second product: registers 8t .. 8t+7 are the eight k values
// of lane half l/32 in k-step t.  The V tile is written to LDS transposed and
// with its keys permuted to that same order (slot 16t + 8h + j holds key
// 16t + 8*(j/4) + 4h + j%4 of the block), so the A operand of the second
// product is one 16-byte LDS read.
//
// A second, small kernel in this file prepares the inputs of the first from
// the projection outputs: RoPE of Q (in place) and K, and the K/V cache write.
#include "../../include/vkl_hip.h"
#include "vkl_common.h"

namespace
{
typedef _Float16 half8 __attribute__ ((ext_vector_type (8)));
typedef float float16v __attribute__ ((ext_vector_type (16)));
typedef uint32_t u32x2 __attribute__ ((ext_vector_type (2)));

constexpr int kBQ = 128;      // query rows per workgroup
constexpr int kBKey = 64;     // keys per tile
constexpr int kThreads = 256;
constexpr float kNeg = -1.0e30f; // "no key seen yet": finite, so that kNeg - kNeg = 0

struct AttnArgs
{
  const uint16_t *q, *k, *v;
  uint16_t *out;
  int H, S, L, ntq;
  size_t qcs, qhs, kcs, khs, vcs, vhs, ors, ohs;
  float scale;
};

__device__ __align__ (16) const uint32_t g_zero16[4] = { 0, 0, 0, 0 };

__device__ __forceinline__ float
fast_exp (float x)
{
  return __builtin_amdgcn_exp2f (x * 1.44269504088896340736f);
}

__device__ __forceinline__ half8
as_half8 (const uint4 v)
{
  return __builtin_bit_cast (half8, v);
}

template <int HD> struct Tile
{
  static constexpr int CPR = HD / 8;                       // 16-byte chunks per row
  static constexpr int KCH = kBKey * CPR / kThreads;       // K chunks per thread
  static constexpr int VIT = (kBKey / 2) * CPR / kThreads; // (key pair, chunk) items per thread
  uint4 k[KCH];
  uint4 v[VIT][2];
};

// K rows [t*64, t*64+64) of the head, as they lie; rows beyond L read zeros
template <int HD>
__device__ __forceinline__ void
load_k (const AttnArgs &a, const uint16_t *kb, int t, Tile<HD> &r)
{
  constexpr int CPR = Tile<HD>::CPR;
  const void *zeros = g_zero16;
#pragma unroll
  for (int i = 0; i < Tile<HD>::KCH; ++i)
    {
      const int c = threadIdx.x + i * kThreads;
      const int row = t * kBKey + c / CPR;
      r.k[i] = vkl::ldg4 (row < a.L ? (const void *)(kb + (size_t)row * a.khs + (c % CPR) * 8)
                                    : zeros);
    }
}

// key of slot s (0..63) of a tile
__device__ __forceinline__ int
slot_key (int s)
{
  const int blk = s >> 5, t = (s >> 4) & 1, h = (s >> 3) & 1, j = s & 7;
  return 32 * blk + 16 * t + 8 * (j >> 2) + 4 * h + (j & 3);
}

template <int HD>
__device__ __forceinline__ void
load_v (const AttnArgs &a, const uint16_t *vb, int t, Tile<HD> &r)
{
  const void *zeros = g_zero16;
#pragma unroll
  for (int i = 0; i < Tile<HD>::VIT; ++i)
    {
      const int it = threadIdx.x + i * kThreads;
      const int pair = it & 31, dc = it >> 5;
      // slots 2*pair and 2*pair+1 hold two adjacent keys
      const int row = t * kBKey + slot_key (2 * pair);
      r.v[i][0] = vkl::ldg4 (row < a.L ? (const void *)(vb + (size_t)row * a.vhs + dc * 8) : zeros);
      r.v[i][1] = vkl::ldg4 (row + 1 < a.L ? (const void *)(vb + (size_t)(row + 1) * a.vhs + dc * 8)
                                           : zeros);
    }
}

template <int HD>
__device__ __forceinline__ void
store_k (const Tile<HD> &r, uint16_t *Ks)
{
  constexpr int CPR = Tile<HD>::CPR, LDK = HD + 8;
#pragma unroll
  for (int i = 0; i < Tile<HD>::KCH; ++i)
    {
      const int c = threadIdx.x + i * kThreads;
      *(uint4 *)(Ks + (c / CPR) * LDK + (c % CPR) * 8) = r.k[i];
    }
}

// V^T: row = d, column = slot; a thread writes the two keys of its pair as one
// 32-bit word per d
template <int HD>
__device__ __forceinline__ void
store_v (const Tile<HD> &r, uint16_t *Vt)
{
  constexpr int LDV = kBKey + 8;
#pragma unroll
  for (int i = 0; i < Tile<HD>::VIT; ++i)
    {
      const int it = threadIdx.x + i * kThreads;
      const int pair = it & 31, dc = it >> 5;
      const uint32_t va[4] = { r.v[i][0].x, r.v[i][0].y, r.v[i][0].z, r.v[i][0].w };
      const uint32_t vb[4] = { r.v[i][1].x, r.v[i][1].y, r.v[i][1].z, r.v[i][1].w };
      uint32_t *dst = (uint32_t *)(Vt + (size_t)(dc * 8) * LDV + 2 * pair);
#pragma unroll
      for (int e = 0; e < 4; ++e)
        {
          dst[(2 * e) * (LDV / 2)] = (va[e] & 0xffffu) | (vb[e] << 16);
          dst[(2 * e + 1) * (LDV / 2)] = (va[e] >> 16) | (vb[e] & 0xffff0000u);
        }
    }
}

// S^T of one 32-key block: rows = keys 32*blk .. +31 of the tile in LDS
template <int HD>
__device__ __forceinline__ float16v
score_block (const uint16_t *Ks, int blk, const half8 (&qf)[HD / 16], int lane)
{
  constexpr int LDK = HD + 8;
  float16v acc;
#pragma unroll
  for (int r = 0; r < 16; ++r)
    acc[r] = 0.f;
  const uint16_t *kp = Ks + (32 * blk + (lane & 31)) * LDK + (lane >> 5) * 8;
#pragma unroll
  for (int kt = 0; kt < HD / 16; ++kt)
    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16 (*(const half8 *)(kp + kt * 16), qf[kt], acc,
                                                  0, 0, 0);
  return acc;
}

template <int HD>
__global__ __launch_bounds__ (kThreads, 2) void
attn_prefill_kernel (const AttnArgs a)
{
  constexpr int KT = HD / 16, DB = HD / 32;
  constexpr int LDK = HD + 8, LDV = kBKey + 8;
  __shared__ __align__ (16) uint16_t Ks[kBKey * LDK];
  __shared__ __align__ (16) uint16_t Vt[HD * LDV];

  // Heavy query tiles (the last ones: most keys) first.  With a head count
  // that is a multiple of 8 the workgroups of one head share id % 8, which
  // keeps the head's K and V in the L2 of one XCD.
  const int b = blockIdx.x;
  int head, qt;
  if ((a.H & 7) == 0)
    {
      // j: position in the XCD's queue.  Its 32 compute units take the first
      // 32 workgroups, then the next 32 beside them, and so on: every other
      // such layer runs the tiles in the opposite order, so that a heavy tile
      // and a light one share a compute unit.
      const int j = b >> 3;
      head = (b & 7) + 8 * (j / a.ntq);
      qt = ((j >> 5) & 1) ? j % a.ntq : a.ntq - 1 - (j % a.ntq);
    }
  else
    {
      head = b / a.ntq;
      qt = a.ntq - 1 - (b % a.ntq);
    }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lq = lane & 31, hh = lane >> 5;
  const int q0 = qt * kBQ;
  const int qrow = q0 + wave * 32 + lq; // this lane's query
  const int shift = a.L - a.S;          // key l is visible iff l <= qrow + shift
  const int kmax = min (a.L, q0 + kBQ + shift);
  const int ntile = (kmax + kBKey - 1) / kBKey;
  const int wave_last = q0 + wave * 32 + 31 + shift; // last key any query of the wave sees
  const uint16_t *kb = a.k + (size_t)head * a.kcs;
  const uint16_t *vb = a.v + (size_t)head * a.vcs;

  half8 qf[KT];
  {
    const uint16_t *qp = a.q + (size_t)head * a.qcs + (size_t)min (qrow, a.S - 1) * a.qhs + hh * 8;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
      qf[kt] = as_half8 (vkl::ldg4 (qp + kt * 16));
  }

  Tile<HD> tl;
  // One pass over the keys with a running maximum: the accumulated products
  // and the sum of exponentials are rescaled whenever the maximum grows, and
  // the division by the sum comes last.
  float m = kNeg, sum = 0.f;
  float16v oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      oacc[db][r] = 0.f;
  load_k<HD> (a, kb, 0, tl);
  load_v<HD> (a, vb, 0, tl);
  for (int t = 0; t < ntile; ++t)
    {
      __syncthreads ();
      store_k<HD> (tl, Ks);
      store_v<HD> (tl, Vt);
      __syncthreads ();
      if (t + 1 < ntile)
        {
          load_k<HD> (a, kb, t + 1, tl);
          load_v<HD> (a, vb, t + 1, tl);
        }
      if (t * kBKey > wave_last)
        continue;
      // scores of the tile's 64 keys, rounded to fp16 like the stand-alone
      // product; a key the query must not see counts as "never seen"
      float sv[2][16];
      float bm = kNeg;
      const bool inner = t * kBKey + kBKey - 1 <= q0 + wave * 32 + shift; // every key visible to every query of the wave
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
        {
          const float16v acc = score_block<HD> (Ks, blk, qf, lane);
          const int key0 = t * kBKey + 32 * blk + 4 * hh;
#pragma unroll
          for (int r = 0; r < 16; ++r)
            {
              const int key = key0 + 8 * (r >> 2) + (r & 3);
              const float sc = vkl::h2f (vkl::f2h (acc[r] * a.scale));
              sv[blk][r] = inner || key <= qrow + shift ? sc : kNeg;
              bm = fmaxf (bm, sv[blk][r]);
            }
        }
      // the two halves of the lanes hold different keys of the same query and
      // feed one product: they need the same maximum
      bm = fmaxf (bm, __shfl_xor (bm, 32, 64));
      const float mn = fmaxf (m, bm);
      if (__builtin_amdgcn_ballot_w64 (mn != m) != 0)
        {
          const float alpha = fast_exp (m - mn); // 0 before the first key, 1 where the maximum stays
          sum *= alpha;
#pragma unroll
          for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r)
              oacc[db][r] *= alpha;
          m = mn;
        }
      half8 pf[2][2];
#pragma unroll
      for (int blk = 0; blk < 2; ++blk)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          {
            // exp (kNeg - m) = 0.  The sum takes the weight as the product
            // below consumes it, rounded to fp16: the weights then add up to
            // one exactly.
            const _Float16 e = (_Float16)fast_exp (sv[blk][r] - m);
            sum += (float)e;
            pf[blk][r >> 3][r & 7] = e;
          }
#pragma unroll
      for (int db = 0; db < DB; ++db)
        {
          const uint16_t *vp = Vt + (size_t)(32 * db + lq) * LDV + 8 * hh;
#pragma unroll
          for (int blk = 0; blk < 2; ++blk)
#pragma unroll
            for (int t2 = 0; t2 < 2; ++t2)
              oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16 (
                  *(const half8 *)(vp + 32 * blk + 16 * t2), pf[blk][t2], oacc[db], 0, 0, 0);
        }
    }
  // the other half of the lanes has summed the other keys of the same query
  sum += __shfl_xor (sum, 32, 64);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r)
      oacc[db][r] *= inv;

  if (qrow >= a.S)
    return;
  uint16_t *op = a.out + (size_t)qrow * a.ors + (size_t)head * a.ohs;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g)
      {
        const int d = 32 * db + 8 * g + 4 * hh;
        u32x2 w;
        w.x = (uint32_t)vkl::f2h (oacc[db][4 * g]) | ((uint32_t)vkl::f2h (oacc[db][4 * g + 1]) << 16);
        w.y = (uint32_t)vkl::f2h (oacc[db][4 * g + 2])
              | ((uint32_t)vkl::f2h (oacc[db][4 * g + 3]) << 16);
        *(VKL_GLOBAL u32x2 *)(op + d) = w;
      }
}
// ---------------------------------------------------------------------------
// RoPE of Q and K and the K/V cache write, straight from the [S, H*hd]
// outputs of the projections: one thread per 8 consecutive elements of a
// (row, head).  Q is rotated in place (the attention kernel reads it with a
// row stride of H*hd), the rotated K and V go to cache rows (k_pos0 + s) %
// maxlen of their head.  Arithmetic of one pair as in the RoPE operator:
// (a, b) -> (fp16(a c - b s), fp16(a s + b c)) with fp32 tables.
// ---------------------------------------------------------------------------
struct RopeKvArgs
{
  uint16_t *q;
  const uint16_t *k, *v;
  uint16_t *kcache, *vcache;
  const float *fc, *fs;
  int S, H, hd, maxlen;
  int q_row0, q_rows;       // rows of q that are rotated, and their positions
  uint32_t q_pos0, k_pos0;  // q row q_row0 + i is at q_pos0 + i; k row s at k_pos0 + s
  size_t rs;                // row stride of q, k, v (elements)
};

__device__ __forceinline__ uint4
rotate8 (const uint4 x, const float *fc, const float *fs)
{
  const uint4 c4 = vkl::ldg4 (fc), s4 = vkl::ldg4 (fs);
  const float c[4] = { __uint_as_float (c4.x), __uint_as_float (c4.y), __uint_as_float (c4.z),
                       __uint_as_float (c4.w) };
  const float sn[4] = { __uint_as_float (s4.x), __uint_as_float (s4.y), __uint_as_float (s4.z),
                        __uint_as_float (s4.w) };
  const uint32_t w[4] = { x.x, x.y, x.z, x.w };
  uint32_t o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
    {
      const float a = vkl::h2f ((uint16_t)(w[j] & 0xffff)), b = vkl::h2f ((uint16_t)(w[j] >> 16));
      const float r0 = a * c[j] - b * sn[j];
      const float r1 = a * sn[j] + b * c[j];
      o[j] = (uint32_t)vkl::f2h (r0) | ((uint32_t)vkl::f2h (r1) << 16);
    }
  return make_uint4 (o[0], o[1], o[2], o[3]);
}

__global__ __launch_bounds__ (256) void
rope_kvwrite_kernel (const RopeKvArgs a, size_t total)
{
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= total)
    return;
  const int cpr = a.hd / 8;
  const int c = (int)(t % cpr);
  const int h = (int)((t / cpr) % a.H);
  const int s = (int)(t / ((size_t)cpr * a.H));
  const size_t src = (size_t)s * a.rs + (size_t)h * a.hd + c * 8;
  const int half = a.hd / 2;
  const uint32_t kpos = a.k_pos0 + (uint32_t)s;
  const size_t dst = ((size_t)h * a.maxlen + kpos % (uint32_t)a.maxlen) * a.hd + c * 8;
  const uint4 kr = rotate8 (vkl::ldg4 (a.k + src), a.fc + (size_t)kpos * half + c * 4,
                            a.fs + (size_t)kpos * half + c * 4);
  *(uint4 *)(a.kcache + dst) = kr;
  *(uint4 *)(a.vcache + dst) = vkl::ldg4 (a.v + src);
  if (s >= a.q_row0 && s < a.q_row0 + a.q_rows)
    {
      const uint32_t qpos = a.q_pos0 + (uint32_t)(s - a.q_row0);
      *(uint4 *)(a.q + src) = rotate8 (vkl::ldg4 (a.q + src), a.fc + (size_t)qpos * half + c * 4,
                                       a.fs + (size_t)qpos * half + c * 4);
    }
}
} // namespace

extern "C" int
vkl_rope_kvwrite_f16 (void *q, const void *k, const void *v, int S, int H,
                      int hd, size_t row_stride, int q_row0, int q_rows,
                      uint32_t q_pos0, uint32_t k_pos0, const float *freqc,
                      const float *freqs, int table_rows, void *kcache,
                      void *vcache, int maxlen, void *stream)
{
  VKL_CHECK_ARG (q && k && v && freqc && freqs && kcache && vcache);
  VKL_CHECK_ARG (S > 0 && H > 0 && hd > 0 && (hd % 8) == 0 && maxlen > 0 && S <= maxlen);
  VKL_CHECK_ARG (q_row0 >= 0 && q_rows >= 0 && q_row0 + q_rows <= S);
  // every position must have a row in the cos / sin tables
  VKL_CHECK_ARG ((size_t)k_pos0 + S <= (size_t)table_rows
                 && (size_t)q_pos0 + q_rows <= (size_t)table_rows);
  VKL_CHECK_ARG ((row_stride % 8) == 0 && row_stride >= (size_t)H * hd);
  VKL_CHECK_ARG (((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0
                 && ((uintptr_t)kcache % 16) == 0 && ((uintptr_t)vcache % 16) == 0
                 && ((uintptr_t)freqc % 16) == 0 && ((uintptr_t)freqs % 16) == 0);
  RopeKvArgs a;
  a.q = (uint16_t *)q, a.k = (const uint16_t *)k, a.v = (const uint16_t *)v;
  a.kcache = (uint16_t *)kcache, a.vcache = (uint16_t *)vcache;
  a.fc = freqc, a.fs = freqs;
  a.S = S, a.H = H, a.hd = hd, a.maxlen = maxlen;
  a.q_row0 = q_row0, a.q_rows = q_rows, a.q_pos0 = q_pos0, a.k_pos0 = k_pos0;
  a.rs = row_stride;
  const size_t total = (size_t)S * H * (hd / 8);
  rope_kvwrite_kernel<<<dim3 ((unsigned)((total + 255) / 256)), dim3 (256), 0, (hipStream_t)stream>>> (
      a, total);
  return vkl_launch_status ();
}

extern "C" int
vkl_attn_prefill_causal_f16 (const void *q, const void *k, const void *v,
                             int H, int S, int L, int hd, size_t qcs,
                             size_t qhs, size_t kcs, size_t khs, size_t vcs,
                             size_t vhs, float scale, void *out, size_t ors,
                             size_t ohs, void *stream)
{
  VKL_CHECK_ARG (q && k && v && out);
  VKL_CHECK_ARG (H > 0 && S > 0 && L >= S);
  VKL_CHECK_ARG (hd == 64 || hd == 128);
  // 16-byte vector loads, 8-byte stores
  VKL_CHECK_ARG (((uintptr_t)q % 16) == 0 && ((uintptr_t)k % 16) == 0 && ((uintptr_t)v % 16) == 0
                 && ((uintptr_t)out % 8) == 0);
  VKL_CHECK_ARG ((qcs % 8) == 0 && (qhs % 8) == 0 && (kcs % 8) == 0 && (khs % 8) == 0
                 && (vcs % 8) == 0 && (vhs % 8) == 0 && (ors % 4) == 0 && (ohs % 4) == 0);
  AttnArgs a;
  a.q = (const uint16_t *)q, a.k = (const uint16_t *)k, a.v = (const uint16_t *)v;
  a.out = (uint16_t *)out;
  a.H = H, a.S = S, a.L = L, a.ntq = (S + kBQ - 1) / kBQ;
  a.qcs = qcs, a.qhs = qhs, a.kcs = kcs, a.khs = khs, a.vcs = vcs, a.vhs = vhs;
  a.ors = ors, a.ohs = ohs, a.scale = scale;
  const dim3 grid ((unsigned)(a.ntq * H));
  if (hd == 128)
    attn_prefill_kernel<128><<<grid, dim3 (kThreads), 0, (hipStream_t)stream>>> (a);
  else
    attn_prefill_kernel<64><<<grid, dim3 (kThreads), 0, (hipStream_t)stream>>> (a);
  return vkl_launch_status ();
}
