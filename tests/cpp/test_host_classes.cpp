// Tests of the C++ drop-in classes (vkllama_amd/src/core, src/ops) in their
// own language, shaped like the reference's gtest files (tests/test_*.cpp of
// the reference): random inputs, the operator under test on the GPU, a plain
// float reference on the host, the reference's tolerances (1e-2 absolute for
// element-wise and normalisation ops, 1e-1 absolute for dot products) plus a
// relative bound.  gtest and Eigen are not in the image, so the harness and
// the host references are a few dozen lines of plain C++.
//
//   test_host_classes --cpu   host-only checks (no device is touched)
//   test_host_classes         everything (needs a GPU)
// Exit status 0 when every check passed.
#include "vkl_decode.h"
#include "src/core/command.h"
#include "src/core/float.h"
#include "src/core/gpu_device.h"
#include "src/core/quants.h"
#include "src/core/tensor.h"
#include "src/ops/argop.h"
#include "src/ops/cast.h"
#include "src/ops/elementwise.h"
#include "src/ops/embedding.h"
#include "src/ops/feed_forward.h"
#include "src/ops/mat_mul.h"
#include "src/ops/multiheadattention_v2.h"
#include "src/ops/rms_norm.h"
#include "src/ops/rope.h"
#include "src/ops/slice.h"
#include "src/ops/concat.h"
#include "src/ops/reduce.h"
#include "src/ops/read_kvcache_op.h"
#include "src/ops/softmax.h"
#include "src/ops/transpose.h"
#include "src/ops/update_kv_cache.h"
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <random>
#include <string>
#include <vector>

using namespace vkllama;

namespace
{
int g_failed = 0, g_checks = 0;
std::string g_test;

#define CHECK(cond)                                                           \
  do                                                                          \
    {                                                                         \
      ++g_checks;                                                             \
      if (!(cond))                                                            \
        {                                                                     \
          ++g_failed;                                                         \
          fprintf (stderr, "FAIL %s:%d [%s] %s\n", __FILE__, __LINE__,        \
                   g_test.c_str (), #cond);                                   \
        }                                                                     \
    }                                                                         \
  while (0)

#define CHECK_OK(expr)                                                        \
  do                                                                          \
    {                                                                         \
      ++g_checks;                                                             \
      auto s__ = (expr);                                                      \
      if (!s__.ok ())                                                         \
        {                                                                     \
          ++g_failed;                                                         \
          fprintf (stderr, "FAIL %s:%d [%s] %s -> %s\n", __FILE__, __LINE__,  \
                   g_test.c_str (), #expr, s__.ToString ().c_str ());         \
          return;                                                             \
        }                                                                     \
    }                                                                         \
  while (0)

typedef std::vector<float> vec;
typedef std::vector<__vkllama_fp16_t> hvec;

std::mt19937 g_rng (20240611);

vec
randn (size_t n, float std = 1.f)
{
  std::normal_distribution<float> d (0.f, std);
  vec v (n);
  for (auto &x : v)
    x = d (g_rng);
  return v;
}

// values rounded to fp16 precision, and their fp16 bits
hvec
to_half (vec &v)
{
  hvec h (v.size ());
  for (size_t i = 0; i < v.size (); ++i)
    {
      h[i] = __fp32_to_fp16_rne (v[i]);
      v[i] = __fp16_to_fp32 (h[i].u16);
    }
  return h;
}

vec
to_float (const hvec &h)
{
  vec v (h.size ());
  for (size_t i = 0; i < h.size (); ++i)
    v[i] = __fp16_to_fp32 (h[i].u16);
  return v;
}

struct Ctx
{
  GPUDevice dev;
  Command cmd;
  Ctx () : dev (0), cmd (&dev) {}
};

// fp16 tensor [c, h, w] holding v (v is rounded to fp16 in place)
absl::StatusOr<Tensor>
half_tensor (Ctx &c, vec &v, int ch, int h, int w)
{
  hvec bits = to_half (v);
  Tensor t (ch, h, w, &c.dev, FP16);
  VKLLAMA_STATUS_OK (t.create ());
  VKLLAMA_STATUS_OK (c.cmd.upload (bits.data (), bits.size (), t));
  return t;
}

absl::StatusOr<Tensor>
float_tensor (Ctx &c, const vec &v, int ch, int h, int w)
{
  Tensor t (ch, h, w, &c.dev, FP32);
  VKLLAMA_STATUS_OK (t.create ());
  VKLLAMA_STATUS_OK (c.cmd.upload (v.data (), v.size (), t));
  return t;
}

// Q8_0 tensor [1, rows, K] from float weights; w is replaced by the
// dequantised values the device will see
absl::StatusOr<Tensor>
q8_tensor (Ctx &c, vec &w, int rows, int K)
{
  const auto prop = get_dtype_property (Q8_0);
  const size_t rb = (size_t)(K + 31) / 32 * prop.bytes_per_block;
  std::vector<int8_t> raw (rows * rb);
  for (int r = 0; r < rows; ++r)
    {
      VKLLAMA_STATUS_OK (qint8_0_quantize_row (w.data () + (size_t)r * K,
                                               raw.data () + r * rb, K));
      VKLLAMA_STATUS_OK (qint8_0_dequantize_row (raw.data () + r * rb,
                                                 w.data () + (size_t)r * K, K));
    }
  Tensor t (1, rows, K, &c.dev, Q8_0);
  VKLLAMA_STATUS_OK (t.create ());
  VKLLAMA_STATUS_OK (c.cmd.upload_bytes ((const uint8_t *)raw.data (),
                                         raw.size (), t));
  return t;
}

absl::StatusOr<vec>
fetch_half (Ctx &c, Tensor t)
{
  hvec bits (t.size ());
  VKLLAMA_STATUS_OK (c.cmd.download (t, bits.data (), bits.size ()));
  VKLLAMA_STATUS_OK (c.cmd.submit_and_wait ());
  return to_float (bits);
}

// largest |a - b| and largest |a - b| / max(|b|, 1e-2 max|b|)
void
compare (const vec &a, const vec &b, float &abs_err, float &rel_err)
{
  float mx = 0.f;
  for (float x : b)
    mx = std::max (mx, fabsf (x));
  abs_err = rel_err = 0.f;
  for (size_t i = 0; i < b.size (); ++i)
    {
      const float d = fabsf (a[i] - b[i]);
      abs_err = std::max (abs_err, d);
      rel_err = std::max (rel_err, d / std::max (fabsf (b[i]), 1e-2f * mx));
    }
}

float
round_half (float v)
{
  return __fp16_to_fp32 (__fp32_to_fp16_rne (v).u16);
}

// ------------------------------------------------------------------- CPU ---
void
test_cpu_float_and_quants ()
{
  g_test = "float/quants (host)";
  // the reference's host conversion truncates (src/core/float.h:86-94); the
  // rounding one is what kernels and uploads use
  CHECK (__fp32_to_fp16 (1.0f).u16 == 0x3c00);
  CHECK (__fp32_to_fp16 (1.0009765f).u16 == 0x3c00);     // truncated down
  CHECK (__fp32_to_fp16_rne (1.0009765f).u16 == 0x3c01); // nearest
  CHECK (__fp32_to_fp16 (1e6f).u16 == 0x7bff);           // clamps to max normal
  CHECK (__fp16_to_fp32 (0x3555) > 0.3332f && __fp16_to_fp32 (0x3555) < 0.3334f);
  for (uint32_t b = 0; b < 0x7c00; b += 37) // exact round trip of every value
    CHECK (__fp32_to_fp16_rne (__fp16_to_fp32 ((uint16_t)b)).u16 == b);

  // Q8_0 round trip as tests/test_quants.cpp of the reference: U(-5, 5),
  // n = 95 (tail padding), |x - deq| <= 1e-1
  const auto prop = get_dtype_property (Q8_0);
  CHECK (prop.items_per_block == 32 && prop.bytes_per_block == 34);
  std::uniform_real_distribution<float> u (-5.f, 5.f);
  vec x (95), back (95);
  for (auto &v : x)
    v = u (g_rng);
  std::vector<int8_t> raw (3 * 34);
  CHECK (qint8_0_quantize_row (x.data (), raw.data (), x.size ()).ok ());
  CHECK (qint8_0_dequantize_row (raw.data (), back.data (), back.size ()).ok ());
  for (size_t i = 0; i < x.size (); ++i)
    CHECK (fabsf (x[i] - back[i]) <= 1e-1f);
  // the tail of the last block is zero
  CHECK (raw[2 * 34 + 2 + 31] == 0);
  // the block maximum lands on +-127, ties round away from zero
  vec y (32, 0.f);
  y[3] = -2.54f, y[4] = 0.01f; // 0.01 * 127 / 2.54 = 0.5 -> 1
  CHECK (qint8_0_quantize_row (y.data (), raw.data (), 32).ok ());
  CHECK (raw[2 + 3] == -127 && raw[2 + 4] == 1 && raw[2 + 5] == 0);
}

// the launch form a model's decode steps take when nobody chooses one
void
test_cpu_default_decode_mode ()
{
  vkl_decode_model d;
  memset (&d, 0, sizeof (d));
  int area = 0;
  d.dim = 4096, d.ffn = 11008, d.flags = &area;
  CHECK (vkl_decode_default_mode (&d) == 1); // 7B rows: one launch per layer
  d.flags = nullptr;
  CHECK (vkl_decode_default_mode (&d) == 0); // nothing to wait on: launches per phase
  d.flags = &area, d.dim = 5120, d.ffn = 13824;
  CHECK (vkl_decode_default_mode (&d) == 0); // 13B rows measured slower in one launch
  d.dim = 256, d.ffn = 704;
  CHECK (vkl_decode_default_mode (&d) == 1);
  CHECK (vkl_decode_default_mode (nullptr) == 0);
}

void
test_cpu_tensor_shapes ()
{
  g_test = "Tensor shapes (host)";
  Tensor t (3, 5, 64, nullptr, FP16);
  CHECK (t.channels () == 3 && t.height () == 5 && t.width () == 64);
  CHECK (t.size () == 3 * 5 * 64 && t.elem_bytes () == 2);
  CHECK (!t.create ().ok ()); // no device
  Tensor q (1, 7, 100, nullptr, Q8_0);
  CHECK (q.elem_bytes () == 1);
  Tensor e;
  CHECK (e.size () == 0);
}

// ------------------------------------------------------------------- GPU ---
void
test_tensor_and_command (Ctx &c)
{
  g_test = "Tensor/Command";
  Tensor t (2, 3, 40, &c.dev, FP16);
  CHECK_OK (t.create ());
  CHECK (t.ws () == 2 && t.hs () == 80 && t.cs () == 240 && t.bytes () == 480);
  Tensor copy = t; // shared handle
  CHECK (copy.data () == t.data ());
  Tensor v = t.view (2, 3, 20);
  CHECK (v.hs () == t.hs () && v.width () == 20 && v.data () == t.data ());
  CHECK_OK (t.reshape (1, 6, 40));
  CHECK (t.cs () == 6 * 80);
  CHECK (!t.reshape (1, 6, 41).ok ());

  vec x = randn (2 * 3 * 40);
  auto tx = half_tensor (c, x, 2, 3, 40);
  CHECK_OK (tx.status ());
  auto back = fetch_half (c, *tx);
  CHECK_OK (back.status ());
  CHECK (*back == x);

  // Q8_0 upload is repacked on the device; download restores the GGUF blocks
  vec w = randn (9 * 100, 0.05f);
  const size_t rb = 4 * 34;
  std::vector<int8_t> raw (9 * rb), got (9 * rb);
  for (int r = 0; r < 9; ++r)
    CHECK (qint8_0_quantize_row (w.data () + r * 100, raw.data () + r * rb, 100).ok ());
  Tensor tq (1, 9, 100, &c.dev, Q8_0);
  CHECK_OK (tq.create ());
  CHECK (tq.bytes () == raw.size ());
  CHECK_OK (c.cmd.upload_bytes ((const uint8_t *)raw.data (), raw.size (), tq));
  CHECK_OK (c.cmd.download (tq, got.data (), got.size ()));
  CHECK_OK (c.cmd.submit_and_wait ());
  CHECK (raw == got);
  // a partial Q8_0 upload is refused, an oversized one too
  CHECK (c.cmd.upload_bytes ((const uint8_t *)raw.data (), raw.size () - 34, tq).code ()
         == absl::StatusCode::kInvalidArgument);
  CHECK (c.cmd.upload (x.data (), x.size (), *tx).code ()
         == absl::StatusCode::kOutOfRange);
}

void
test_rmsnorm (Ctx &c, int C, int H, int W)
{
  g_test = "RMSNorm " + std::to_string (C) + "x" + std::to_string (H) + "x" + std::to_string (W);
  vec x = randn ((size_t)C * H * W), w = randn (W);
  auto tx = half_tensor (c, x, C, H, W);
  auto tw = float_tensor (c, w, 1, 1, W);
  CHECK_OK (tx.status ());
  CHECK_OK (tw.status ());
  RMSNorm op (&c.dev, &c.cmd, *tw, 1e-3f);
  CHECK_OK (op.init ());
  auto out = op (*tx);
  CHECK_OK (out.status ());
  auto got = fetch_half (c, *out);
  CHECK_OK (got.status ());
  vec want (x.size ());
  for (int r = 0; r < C * H; ++r)
    {
      double ss = 0;
      for (int i = 0; i < W; ++i)
        ss += (double)x[r * W + i] * x[r * W + i];
      const float alpha = 1.0f / sqrtf ((float)(ss / W) + 1e-3f);
      for (int i = 0; i < W; ++i)
        want[r * W + i] = x[r * W + i] * w[i] * alpha;
    }
  float ae, re;
  compare (*got, want, ae, re);
  CHECK (ae <= 1e-2f); // tolerance of tests/test_rmsnorm.cpp in the reference
  CHECK (re <= 4e-3f);
  // a tensor of the wrong type is refused
  Tensor f32 (C, H, W, &c.dev, FP32);
  CHECK_OK (f32.create ());
  CHECK (op (f32).status ().code () == absl::StatusCode::kInvalidArgument);
}

void
test_matmul_q8 (Ctx &c, int M, int N, int K, int act)
{
  g_test = "MatMul Q8_0 M" + std::to_string (M) + " N" + std::to_string (N) + " K" + std::to_string (K);
  vec x = randn ((size_t)M * K), w = randn ((size_t)N * K, 0.05f);
  auto tx = half_tensor (c, x, 1, M, K);
  auto tw = q8_tensor (c, w, N, K);
  CHECK_OK (tx.status ());
  CHECK_OK (tw.status ());
  MatMul op (&c.dev, &c.cmd, *tw, 0.5f, 0.25f, act, 0, true, FP16, Q8_0);
  CHECK_OK (op.init ());
  auto out = op (*tx);
  CHECK_OK (out.status ());
  CHECK (out->height () == (size_t)M && out->width () == (size_t)N);
  auto got = fetch_half (c, *out);
  CHECK_OK (got.status ());
  vec want ((size_t)M * N);
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n)
      {
        double s = 0;
        for (int k = 0; k < K; ++k)
          s += (double)x[m * K + k] * w[(size_t)n * K + k];
        float v = (float)s * 0.5f + 0.25f;
        if (act == 1)
          v = v / (1.0f + expf (-v));
        want[m * N + n] = v;
      }
  float ae, re;
  compare (*got, want, ae, re);
  CHECK (ae <= 1e-1f); // tests/test_matmul.cpp of the reference
  CHECK (re <= 1e-2f);
}

// MatMul::set_residual: the product with the residual added in its launch
// equals the product followed by an ElementWise add, value for value, for the
// one call it was set for
void
test_matmul_residual (Ctx &c, int M, int N, int K)
{
  g_test = "MatMul residual M" + std::to_string (M) + " N" + std::to_string (N) + " K" + std::to_string (K);
  vec x = randn ((size_t)M * K), w = randn ((size_t)N * K, 0.05f), r = randn ((size_t)M * N);
  auto tx = half_tensor (c, x, 1, M, K);
  auto tw = q8_tensor (c, w, N, K);
  auto tr = half_tensor (c, r, 1, M, N);
  CHECK_OK (tx.status ());
  CHECK_OK (tw.status ());
  CHECK_OK (tr.status ());
  MatMul fused (&c.dev, &c.cmd, *tw, 1.0f, 0.f, 0, 0, true, FP16, Q8_0);
  MatMul plain (&c.dev, &c.cmd, *tw, 1.0f, 0.f, 0, 0, true, FP16, Q8_0);
  ElementWise add (&c.dev, &c.cmd, 0, FP16);
  CHECK_OK (fused.init ());
  CHECK_OK (plain.init ());
  CHECK_OK (add.init ());
  fused.set_residual (&*tr);
  auto a = fused (*tx);
  CHECK_OK (a.status ());
  auto got = fetch_half (c, *a);
  CHECK_OK (got.status ());
  auto b = plain (*tx);
  CHECK_OK (b.status ());
  auto prod = fetch_half (c, *b); // before the add writes in place
  CHECK_OK (prod.status ());
  auto sum = add (*b, *tr);
  CHECK_OK (sum.status ());
  auto want = fetch_half (c, *sum);
  CHECK_OK (want.status ());
  CHECK (*got == *want);
  // the residual held for one call only
  auto again = fused (*tx);
  CHECK_OK (again.status ());
  auto got2 = fetch_half (c, *again);
  CHECK_OK (got2.status ());
  CHECK (*got2 == *prod);
  // a residual of another shape is refused
  auto bad = half_tensor (c, r, 1, N, M);
  CHECK_OK (bad.status ());
  if (M != N)
    {
      fused.set_residual (&*bad);
      CHECK (fused (*tx).status ().code () == absl::StatusCode::kInvalidArgument);
    }
}

void
test_matmul_f16 (Ctx &c)
{
  g_test = "MatMul fp16";
  // scores: [C, M, K] x [C, N, K]^T, and probabilities x values: [C, M, K] x [C, K, N]
  const int C = 4, M = 5, N = 37, K = 64;
  vec a = randn ((size_t)C * M * K), b = randn ((size_t)C * N * K);
  auto ta = half_tensor (c, a, C, M, K);
  auto tb = half_tensor (c, b, C, N, K);
  CHECK_OK (ta.status ());
  CHECK_OK (tb.status ());
  MatMul tbop (&c.dev, &c.cmd, 0.125f, 0.f, 0, 0, true);
  CHECK_OK (tbop.init ());
  auto s = tbop (*ta, *tb);
  CHECK_OK (s.status ());
  auto got = fetch_half (c, *s);
  CHECK_OK (got.status ());
  vec want ((size_t)C * M * N);
  for (int ch = 0; ch < C; ++ch)
    for (int m = 0; m < M; ++m)
      for (int n = 0; n < N; ++n)
        {
          double acc = 0;
          for (int k = 0; k < K; ++k)
            acc += (double)a[(ch * M + m) * K + k] * b[((size_t)ch * N + n) * K + k];
          want[(ch * M + m) * N + n] = 0.125f * (float)acc;
        }
  float ae, re;
  compare (*got, want, ae, re);
  CHECK (ae <= 1e-1f && re <= 1e-2f);

  vec p ((size_t)C * M * N);
  std::uniform_real_distribution<float> u (0.f, 0.1f);
  for (auto &v : p)
    v = u (g_rng);
  vec vv = randn ((size_t)C * N * K);
  auto tp = half_tensor (c, p, C, M, N);
  auto tv = half_tensor (c, vv, C, N, K);
  CHECK_OK (tp.status ());
  CHECK_OK (tv.status ());
  MatMul nnop (&c.dev, &c.cmd, 1.f, 0.f, 0, 0, false);
  CHECK_OK (nnop.init ());
  auto o = nnop (*tp, *tv);
  CHECK_OK (o.status ());
  auto goto_ = fetch_half (c, *o);
  CHECK_OK (goto_.status ());
  vec wo ((size_t)C * M * K);
  for (int ch = 0; ch < C; ++ch)
    for (int m = 0; m < M; ++m)
      for (int j = 0; j < K; ++j)
        {
          double acc = 0;
          for (int l = 0; l < N; ++l)
            acc += (double)p[(ch * M + m) * N + l] * vv[((size_t)ch * N + l) * K + j];
          wo[(ch * M + m) * K + j] = (float)acc;
        }
  compare (*goto_, wo, ae, re);
  CHECK (ae <= 1e-1f && re <= 1e-2f);
  // shape mismatch is reported, not launched
  CHECK (tbop (*ta, *tp).status ().code () == absl::StatusCode::kInvalidArgument);
}

void
test_elementwise_cast_argmax (Ctx &c)
{
  g_test = "ElementWise/Cast/ArgMax";
  const int C = 2, H = 7, W = 130;
  vec a = randn ((size_t)C * H * W), b = randn ((size_t)C * H * W);
  auto ta = half_tensor (c, a, C, H, W);
  auto tb = half_tensor (c, b, C, H, W);
  CHECK_OK (ta.status ());
  CHECK_OK (tb.status ());
  ElementWise add (&c.dev, &c.cmd, 0);
  CHECK_OK (add.init ());
  auto sum = add (*ta, *tb); // y = x + y, in place into y
  CHECK_OK (sum.status ());
  CHECK (sum->data () == tb->data ());
  auto got = fetch_half (c, *sum);
  CHECK_OK (got.status ());
  for (size_t i = 0; i < a.size (); ++i)
    CHECK ((*got)[i] == round_half (a[i] + b[i]));

  Cast widen (&c.dev, &c.cmd, FP16, FP32);
  CHECK_OK (widen.init ());
  auto f = widen (*ta);
  CHECK_OK (f.status ());
  vec f32 (a.size ());
  CHECK_OK (c.cmd.download (*f, f32.data (), f32.size ()));
  CHECK_OK (c.cmd.submit_and_wait ());
  CHECK (f32 == a); // exact

  // first maximum wins (tests/test_argop.cpp of the reference compares with
  // Eigen's argmax, which returns the first one)
  vec m ((size_t)H * W, 0.f);
  for (int r = 0; r < H; ++r)
    {
      const int c0 = (r * 17) % (W - 6);
      m[r * W + c0] = 3.f, m[r * W + c0 + 5] = 3.f; // two equal maxima
    }
  auto tm = half_tensor (c, m, 1, H, W);
  CHECK_OK (tm.status ());
  ArgMax amax (&c.dev, &c.cmd);
  CHECK_OK (amax.init ());
  auto idx = amax (*tm);
  CHECK_OK (idx.status ());
  std::vector<uint32_t> ids (H);
  CHECK_OK (c.cmd.download (*idx, ids.data (), ids.size ()));
  CHECK_OK (c.cmd.submit_and_wait ());
  for (int r = 0; r < H; ++r)
    {
      uint32_t first = 0;
      for (int i = 0; i < W; ++i)
        if (m[r * W + i] > m[r * W + first])
          first = i;
      CHECK (ids[r] == first);
    }
}

void
test_embedding (Ctx &c)
{
  g_test = "Embedding Q8_0";
  const int V = 50, W = 96;
  vec table = randn ((size_t)V * W, 0.1f);
  auto tt = q8_tensor (c, table, V, W);
  CHECK_OK (tt.status ());
  std::vector<uint32_t> toks = { 0, 49, 7, 50, 1u << 31 }; // ids >= V read UNK
  Tensor ti (1, 1, (int)toks.size (), &c.dev, UINT32, true);
  CHECK_OK (ti.create ());
  CHECK_OK (c.cmd.upload (toks.data (), toks.size (), ti));
  Embedding op (&c.dev, &c.cmd, *tt, 3u, Q8_0); // dtype = the table's
  CHECK_OK (op.init ());
  auto out = op (ti);
  CHECK_OK (out.status ());
  auto got = fetch_half (c, *out);
  CHECK_OK (got.status ());
  for (size_t t = 0; t < toks.size (); ++t)
    {
      const uint32_t row = toks[t] < (uint32_t)V ? toks[t] : 3u;
      for (int i = 0; i < W; ++i)
        CHECK ((*got)[t * W + i] == round_half (table[(size_t)row * W + i]));
    }
}

void
test_rope_softmax_kv (Ctx &c)
{
  g_test = "Rope/Softmax/UpdateKVCache";
  const int H = 3, S = 4, hd = 64, maxlen = 1024;
  Rope rope (&c.dev, &c.cmd, maxlen, hd);
  CHECK_OK (rope.init ());
  for (size_t off : { (size_t)0, (size_t)100, (size_t)1020 }) // tests/test_rope.cpp offsets
    {
      vec x = randn ((size_t)H * S * hd);
      auto tx = half_tensor (c, x, H, S, hd);
      CHECK_OK (tx.status ());
      auto out = rope (*tx, off);
      CHECK_OK (out.status ());
      auto got = fetch_half (c, *out);
      CHECK_OK (got.status ());
      float worst = 0.f;
      for (int h = 0; h < H; ++h)
        for (int s = 0; s < S; ++s)
          for (int i = 0; i < hd / 2; ++i)
            {
              const float freq = 1.0f / powf (10000.0f, (float)(2 * i) / (float)hd);
              const float ang = freq * (float)(s + off);
              const float a = x[(h * S + s) * hd + 2 * i], b = x[(h * S + s) * hd + 2 * i + 1];
              worst = std::max (worst, fabsf ((*got)[(h * S + s) * hd + 2 * i] - (a * cosf (ang) - b * sinf (ang))));
              worst = std::max (worst, fabsf ((*got)[(h * S + s) * hd + 2 * i + 1] - (a * sinf (ang) + b * cosf (ang))));
            }
      CHECK (worst <= 1e-2f);
    }

  // masked softmax: row s of S sees columns 0 .. s + (L - S)
  const int L = 9;
  vec sc = randn ((size_t)H * S * L, 2.f);
  auto ts = half_tensor (c, sc, H, S, L);
  CHECK_OK (ts.status ());
  Softmax sm (&c.dev, &c.cmd, true);
  CHECK_OK (sm.init ());
  auto p = sm (*ts, L - S);
  CHECK_OK (p.status ());
  auto gp = fetch_half (c, *p);
  CHECK_OK (gp.status ());
  for (int r = 0; r < H * S; ++r)
    {
      const int s = r % S, last = s + (L - S);
      float mx = -1e30f, sum = 0.f, total = 0.f;
      for (int l = 0; l < L; ++l)
        mx = std::max (mx, sc[r * L + l]); // the shader's maximum runs over the whole row
      for (int l = 0; l <= last; ++l)
        sum += expf (sc[r * L + l] - mx);
      for (int l = 0; l < L; ++l)
        {
          const float want = l <= last ? expf (sc[r * L + l] - mx) / sum : 0.f;
          CHECK (fabsf ((*gp)[r * L + l] - want) <= 1e-2f);
          if (l > last)
            CHECK ((*gp)[r * L + l] == 0.f);
          total += (*gp)[r * L + l];
        }
      CHECK (fabsf (total - 1.f) <= 1e-2f);
    }

  // cache update wraps modulo the cache length (offset 1022 of 1024 in
  // tests/test_update_kv_cache.cpp of the reference)
  vec cache = randn ((size_t)H * maxlen * hd), kv = randn ((size_t)H * S * hd);
  auto tc = half_tensor (c, cache, H, maxlen, hd);
  auto tk = half_tensor (c, kv, H, S, hd);
  CHECK_OK (tc.status ());
  CHECK_OK (tk.status ());
  UpdateKVCache upd (&c.dev, &c.cmd, FP16);
  CHECK_OK (upd.init ());
  CHECK_OK (upd (*tc, *tk, 1022));
  auto gc = fetch_half (c, *tc);
  CHECK_OK (gc.status ());
  for (int h = 0; h < H; ++h)
    for (int s = 0; s < S; ++s)
      for (int i = 0; i < hd; ++i)
        cache[((size_t)h * maxlen + (1022 + s) % maxlen) * hd + i] = kv[(h * S + s) * hd + i];
  CHECK (*gc == cache);
}

void
test_slice_transpose (Ctx &c)
{
  g_test = "Slice/Transpose";
  const int C = 3, H = 5, W = 16;
  vec x = randn ((size_t)C * H * W);
  auto tx = half_tensor (c, x, C, H, W);
  CHECK_OK (tx.status ());
  Slice slice (&c.dev, &c.cmd, FP16);
  CHECK_OK (slice.init ());
  auto s = slice (*tx, { 1, 2, 4 }, { 2, 3, 8 });
  CHECK_OK (s.status ());
  auto gs = fetch_half (c, *s);
  CHECK_OK (gs.status ());
  for (int ch = 0; ch < 2; ++ch)
    for (int h = 0; h < 3; ++h)
      for (int w = 0; w < 8; ++w)
        CHECK ((*gs)[(ch * 3 + h) * 8 + w] == x[((ch + 1) * H + h + 2) * W + w + 4]);
  CHECK (slice (*tx, { 2, 0, 0 }, { 2, 1, 1 }).status ().code () == absl::StatusCode::kOutOfRange);

  Transpose tr (&c.dev, &c.cmd, 0, FP16); // [C, H, W] -> [H, C, W]
  CHECK_OK (tr.init ());
  auto t = tr (*tx);
  CHECK_OK (t.status ());
  CHECK (t->channels () == (size_t)H && t->height () == (size_t)C);
  auto gt = fetch_half (c, *t);
  CHECK_OK (gt.status ());
  for (int ch = 0; ch < C; ++ch)
    for (int h = 0; h < H; ++h)
      for (int w = 0; w < W; ++w)
        CHECK ((*gt)[(h * C + ch) * W + w] == x[(ch * H + h) * W + w]);
}

void
test_feed_forward (Ctx &c, int M)
{
  g_test = "FeedForward Q8_0 M" + std::to_string (M);
  const int dim = 256, ffn = 352;
  vec x = randn ((size_t)M * dim), w1 = randn ((size_t)ffn * dim, 0.05f),
      w2 = randn ((size_t)dim * ffn, 0.05f), w3 = randn ((size_t)ffn * dim, 0.05f);
  auto tx = half_tensor (c, x, 1, M, dim);
  auto t1 = q8_tensor (c, w1, ffn, dim);
  auto t2 = q8_tensor (c, w2, dim, ffn);
  auto t3 = q8_tensor (c, w3, ffn, dim);
  CHECK_OK (tx.status ());
  CHECK_OK (t1.status ());
  CHECK_OK (t2.status ());
  CHECK_OK (t3.status ());
  FeedForward ff (&c.dev, &c.cmd, *t1, *t2, *t3, true, Q8_0); // [out, in] weights
  CHECK_OK (ff.init ());
  auto out = ff (*tx);
  CHECK_OK (out.status ());
  auto got = fetch_half (c, *out);
  CHECK_OK (got.status ());
  // y = w2 (silu(w1 x) * (w3 x)), the formula of tests/test_feedforward.cpp
  vec want ((size_t)M * dim);
  for (int m = 0; m < M; ++m)
    {
      vec t (ffn);
      for (int f = 0; f < ffn; ++f)
        {
          double g = 0, u = 0;
          for (int k = 0; k < dim; ++k)
            {
              g += (double)x[m * dim + k] * w1[(size_t)f * dim + k];
              u += (double)x[m * dim + k] * w3[(size_t)f * dim + k];
            }
          t[f] = round_half ((float)(g / (1.0 + exp (-g)) * u));
        }
      for (int d = 0; d < dim; ++d)
        {
          double s = 0;
          for (int f = 0; f < ffn; ++f)
            s += (double)t[f] * w2[(size_t)d * ffn + f];
          want[m * dim + d] = (float)s;
        }
    }
  float ae, re;
  compare (*got, want, ae, re);
  CHECK (ae <= 1e-1f && re <= 1e-2f);
}

void
test_attention (Ctx &c, int S, bool clip)
{
  g_test = std::string ("MultiHeadAttentionV2 S") + std::to_string (S) + (clip ? " clipped" : "");
  const int dim = 256, heads = 4, hd = 64, maxlen = 32;
  vec x = randn ((size_t)S * dim), wk = randn ((size_t)dim * dim, 0.05f),
      wq = randn ((size_t)dim * dim, 0.05f), wv = randn ((size_t)dim * dim, 0.05f),
      wo = randn ((size_t)dim * dim, 0.05f);
  auto tx = half_tensor (c, x, 1, S, dim);
  auto tk = q8_tensor (c, wk, dim, dim);
  auto tq = q8_tensor (c, wq, dim, dim);
  auto tv = q8_tensor (c, wv, dim, dim);
  auto to = q8_tensor (c, wo, dim, dim);
  CHECK_OK (tx.status ());
  CHECK_OK (tk.status ());
  CHECK_OK (tq.status ());
  CHECK_OK (tv.status ());
  CHECK_OK (to.status ());
  // `dim` of the operator is the head width (heads = rows of Wk / dim)
  MultiHeadAttentionV2 attn (&c.dev, &c.cmd, *tk, *tq, *tv, *to, maxlen, hd, true, FP16, true, clip);
  attn.set_lastblock_rope_quirk (false);
  CHECK_OK (attn.init ());
  auto out = attn (*tx, 0);
  CHECK_OK (out.status ());
  const int rows = clip ? 1 : S;
  CHECK (out->height () == (size_t)rows && out->width () == (size_t)dim);
  auto got = fetch_half (c, *out);
  CHECK_OK (got.status ());

  // causal attention in float with fp16 rounding of the projections
  auto project = [&] (const vec &w, const vec &in, int n) {
    vec y ((size_t)n * dim);
    for (int s = 0; s < n; ++s)
      for (int d = 0; d < dim; ++d)
        {
          double acc = 0;
          for (int k = 0; k < dim; ++k)
            acc += (double)in[s * dim + k] * w[(size_t)d * dim + k];
          y[s * dim + d] = round_half ((float)acc);
        }
    return y;
  };
  vec K = project (wk, x, S), Q = project (wq, x, S), V = project (wv, x, S);
  auto rot = [&] (vec &t) {
    for (int s = 0; s < S; ++s)
      for (int h = 0; h < heads; ++h)
        for (int i = 0; i < hd / 2; ++i)
          {
            const float ang = (float)s / powf (10000.0f, (float)(2 * i) / (float)hd);
            float &a = t[s * dim + h * hd + 2 * i], &b = t[s * dim + h * hd + 2 * i + 1];
            const float ra = a * cosf (ang) - b * sinf (ang), rb = a * sinf (ang) + b * cosf (ang);
            a = round_half (ra), b = round_half (rb);
          }
  };
  rot (K);
  rot (Q);
  vec att ((size_t)S * dim);
  for (int h = 0; h < heads; ++h)
    for (int s = 0; s < S; ++s)
      {
        vec p (S, 0.f);
        float mx = -1e30f, sum = 0.f;
        for (int l = 0; l <= s; ++l)
          {
            double acc = 0;
            for (int i = 0; i < hd; ++i)
              acc += (double)Q[s * dim + h * hd + i] * K[l * dim + h * hd + i];
            p[l] = round_half ((float)acc / sqrtf ((float)hd));
            mx = std::max (mx, p[l]);
          }
        for (int l = 0; l <= s; ++l)
          sum += expf (p[l] - mx);
        for (int i = 0; i < hd; ++i)
          {
            double acc = 0;
            for (int l = 0; l <= s; ++l)
              acc += (double)round_half (expf (p[l] - mx) / sum) * V[l * dim + h * hd + i];
            att[s * dim + h * hd + i] = round_half ((float)acc);
          }
      }
  vec full = project (wo, att, S);
  vec want (full.end () - (size_t)rows * dim, full.end ());
  float ae, re;
  compare (*got, want, ae, re);
  CHECK (ae <= 1e-1f && re <= 2e-2f);
  // the context may not run past the cache
  CHECK (attn (*tx, maxlen).status ().code () == absl::StatusCode::kOutOfRange);
}

void
test_concat_reduce_readkv (Ctx &c)
{
  g_test = "Concat/Reduce/ReadKVCache";
  // tests/test_concat.cpp of the reference joins two tensors along each axis
  for (int axis = 0; axis < 3; ++axis)
    {
      const int C = 3, H = 5, W = 16;
      int d1[3] = { C, H, W };
      d1[axis] += 2 + axis;
      vec a = randn ((size_t)C * H * W), b = randn ((size_t)d1[0] * d1[1] * d1[2]);
      auto ta = half_tensor (c, a, C, H, W);
      auto tb = half_tensor (c, b, d1[0], d1[1], d1[2]);
      CHECK_OK (ta.status ());
      CHECK_OK (tb.status ());
      Concat cat (&c.dev, &c.cmd, 2, axis, FP16);
      CHECK_OK (cat.init ());
      auto out = cat ({ *ta, *tb });
      CHECK_OK (out.status ());
      const int OC = axis == 0 ? C + d1[0] : C, OH = axis == 1 ? H + d1[1] : H,
                OW = axis == 2 ? W + d1[2] : W;
      CHECK (out->channels () == (size_t)OC && out->height () == (size_t)OH
             && out->width () == (size_t)OW);
      auto g = fetch_half (c, *out);
      CHECK_OK (g.status ());
      for (int ch = 0; ch < OC; ++ch)
        for (int h = 0; h < OH; ++h)
          for (int w = 0; w < OW; ++w)
            {
              const bool in_a = ch < C && h < H && w < W;
              const float want
                  = in_a ? a[((size_t)ch * H + h) * W + w]
                         : b[((size_t)(ch - (axis == 0 ? C : 0)) * d1[1] + (h - (axis == 1 ? H : 0)))
                                 * d1[2]
                             + (w - (axis == 2 ? W : 0))];
              CHECK ((*g)[((size_t)ch * OH + h) * OW + w] == want);
            }
      Concat bad (&c.dev, &c.cmd, 3, axis, FP16);
      CHECK_OK (bad.init ());
      CHECK (bad ({ *ta, *tb }).status ().code () == absl::StatusCode::kInvalidArgument);
    }
  {
    // tests/test_reduce.cpp: sum / max / min / mean over the last axis, 1e-2
    const int C = 3, H = 7, W = 300;
    vec x = randn ((size_t)C * H * W);
    auto tx = half_tensor (c, x, C, H, W);
    CHECK_OK (tx.status ());
    for (int op = 0; op < 4; ++op)
      {
        Reduce red (&c.dev, &c.cmd, op, FP16);
        CHECK_OK (red.init ());
        auto out = red (*tx);
        CHECK_OK (out.status ());
        CHECK (out->channels () == (size_t)C && out->height () == (size_t)H && out->width () == 1);
        auto g = fetch_half (c, *out);
        CHECK_OK (g.status ());
        for (int r = 0; r < C * H; ++r)
          {
            double v = op == 0 || op == 3 ? 0.0 : x[(size_t)r * W];
            for (int w = 0; w < W; ++w)
              {
                const double e = x[(size_t)r * W + w];
                v = op == 0 || op == 3 ? v + e : (op == 1 ? std::max (v, e) : std::min (v, e));
              }
            if (op == 3)
              v /= W;
            if (op == 1 || op == 2)
              CHECK ((*g)[r] == (float)v);
            else
              CHECK (fabs ((*g)[r] - v) <= 1e-2 * std::max (1.0, fabs (v)));
          }
      }
  }
  {
    // ring read: rows (offset + y) % H
    const int C = 4, H = 16, W = 8;
    vec x = randn ((size_t)C * H * W);
    auto tx = half_tensor (c, x, C, H, W);
    CHECK_OK (tx.status ());
    ReadKVCache rd (&c.dev, &c.cmd);
    CHECK_OK (rd.init ());
    auto out = rd (*tx, 13, 6);
    CHECK_OK (out.status ());
    CHECK (out->channels () == (size_t)C && out->height () == 6 && out->width () == (size_t)W);
    auto g = fetch_half (c, *out);
    CHECK_OK (g.status ());
    for (int ch = 0; ch < C; ++ch)
      for (int y = 0; y < 6; ++y)
        for (int w = 0; w < W; ++w)
          CHECK ((*g)[((size_t)ch * 6 + y) * W + w] == x[((size_t)ch * H + (y + 13) % H) * W + w]);
    CHECK (rd (*tx, 0, 17).status ().code () == absl::StatusCode::kOutOfRange);
  }
}

void
run_gpu ()
{
  Ctx c;
  g_test = "GPUDevice";
  CHECK_OK (c.dev.init ());
  CHECK_OK (c.cmd.init ());
  CHECK (c.dev.subgroup_size () == 64);
  CHECK (c.dev.support_16bit_storage () && c.dev.support_8bit_storage ());
  test_tensor_and_command (c);
  test_rmsnorm (c, 1, 1, 128);
  test_rmsnorm (c, 3, 1023, 63);
  test_matmul_q8 (c, 1, 512, 1376, 0);
  test_matmul_q8 (c, 3, 130, 512, 1);
  test_matmul_q8 (c, 70, 96, 256, 0);
  test_matmul_residual (c, 1, 512, 1376);  // one row: the decode step's streaming kernel
  test_matmul_residual (c, 20, 130, 2048); // few-row kernel and its reduction
  test_matmul_residual (c, 70, 96, 2048);  // tile kernel with the k-split
  test_matmul_residual (c, 150, 300, 256); // tile kernel
  test_matmul_f16 (c);
  test_elementwise_cast_argmax (c);
  test_embedding (c);
  test_rope_softmax_kv (c);
  test_slice_transpose (c);
  test_concat_reduce_readkv (c);
  test_feed_forward (c, 1);
  test_feed_forward (c, 20);
  test_attention (c, 6, false);
  test_attention (c, 6, true);
  test_attention (c, 1, false);
}
}

int
main (int argc, char **argv)
{
  const bool cpu_only = argc > 1 && !strcmp (argv[1], "--cpu");
  test_cpu_float_and_quants ();
  test_cpu_tensor_shapes ();
  test_cpu_default_decode_mode ();
  if (!cpu_only)
    run_gpu ();
  printf ("%s: %d checks, %d failed\n", cpu_only ? "host-only" : "all", g_checks,
          g_failed);
  return g_failed ? 1 : 0;
}
