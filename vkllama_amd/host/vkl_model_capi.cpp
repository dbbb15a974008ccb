// extern "C" wrappers around vkllama::Model and the synthetic-weight helpers
// (include/vkl_model.h).
#include "vkl_model.h"
#include "models/gguflib.h"
#include "models/llama2.h"
#include "vkl_decode.h"
#include "vkl_hip.h"
#include <cmath>
#include <map>
#include <string>
#include <vector>

struct vkl_model
{
  vkllama::Model *model = nullptr;
  std::string last_error;
  std::vector<gguf_value> values;
  std::vector<std::string> names;
};

namespace
{
int
fail (vkl_model *m, const absl::Status &s)
{
  if (m)
    m->last_error = s.ToString ();
  return (int)s.code ();
}
}

extern "C" int
vkl_model_create (int dev, const vkl_model_hparams *hp,
                  const vkl_tensor_desc *tensors, size_t n_tensors,
                  vkl_model **out)
{
  if (!hp || !tensors || !out)
    return (int)absl::StatusCode::kInvalidArgument;
  auto *m = new vkl_model ();
  *out = m;
  std::map<std::string, gguf_key> kv;
  std::map<std::string, gguf_tensor> ts;
  m->values.resize (4);
  m->values[0].uint32 = hp->head_count;
  m->values[1].uint32 = hp->block_count;
  m->values[2].float32 = hp->rms_eps;
  m->values[3].uint32 = hp->context_length;
  const char *keys[4]
      = { "llama.attention.head_count", "llama.block_count",
          "llama.attention.layer_norm_rms_epsilon", "llama.context_length" };
  for (int i = 0; i < 4; ++i)
    {
      gguf_key k = {};
      k.name = keys[i];
      k.namelen = strlen (keys[i]);
      k.type = i == 2 ? 6u : 4u; // GGUF value types FLOAT32 / UINT32
      k.val = &m->values[i];
      kv[keys[i]] = k;
    }
  m->names.reserve (n_tensors);
  for (size_t i = 0; i < n_tensors; ++i)
    {
      if (!tensors[i].name || !tensors[i].data)
        return fail (m, absl::InvalidArgumentError ("tensor without name/data"));
      m->names.emplace_back (tensors[i].name);
      gguf_tensor t = {};
      t.name = m->names.back ().c_str ();
      t.namelen = m->names.back ().size ();
      t.type = tensors[i].type;
      t.ndim = tensors[i].dim1 > 1 ? 2 : 1;
      t.dim[0] = tensors[i].dim0;
      t.dim[1] = tensors[i].dim1 ? tensors[i].dim1 : 1;
      t.bsize = tensors[i].bsize;
      t.num_weights = t.dim[0] * t.dim[1];
      t.weights_data = (uint8_t *)tensors[i].data;
      ts[m->names.back ()] = t;
    }
  m->model = new vkllama::Model (dev);
  try
    {
      auto s = m->model->init (kv, ts);
      if (!s.ok ())
        return fail (m, s);
    }
  catch (const std::exception &e)
    {
      return fail (m, absl::InternalError (e.what ()));
    }
  return 0;
}

extern "C" int
vkl_model_load_gguf (int dev, const char *path, vkl_model **out)
{
  if (!path || !out)
    return (int)absl::StatusCode::kInvalidArgument;
  auto *m = new vkl_model ();
  *out = m;
  gguf_ctx *g = gguf_open (path);
  if (!g)
    return fail (m, absl::NotFoundError (std::string ("not a readable GGUF file: ") + path));
  std::map<std::string, gguf_key> kv;
  std::map<std::string, gguf_tensor> ts;
  gguf_key key;
  while (gguf_get_key (g, &key))
    kv[std::string (key.name, key.namelen)] = key;
  gguf_tensor t;
  while (gguf_get_tensor (g, &t))
    ts[std::string (t.name, t.namelen)] = t;
  m->model = new vkllama::Model (dev);
  absl::Status s = absl::OkStatus ();
  try
    {
      s = m->model->init (kv, ts);
    }
  catch (const std::exception &e)
    {
      s = absl::InternalError (e.what ());
    }
  gguf_close (g); // every weight has been copied to the device by now
  return s.ok () ? 0 : fail (m, s);
}

extern "C" void
vkl_model_destroy (vkl_model *m)
{
  if (!m)
    return;
  delete m->model;
  delete m;
}

extern "C" const char *
vkl_model_last_error (const vkl_model *m)
{
  return m ? m->last_error.c_str () : "null model";
}

extern "C" size_t
vkl_model_vocab (const vkl_model *m)
{
  return m && m->model ? m->model->vocab_size () : 0;
}

extern "C" int
vkl_model_forward (vkl_model *m, const uint32_t *toks, size_t n_toks,
                   size_t offset, float *logits)
{
  if (!m || !m->model || !toks || !logits)
    return (int)absl::StatusCode::kInvalidArgument;
  try
    {
      std::vector<uint32_t> v (toks, toks + n_toks);
      auto r = (*m->model) (v, offset);
      if (!r.ok ())
        return fail (m, r.status ());
      const size_t V = m->model->vocab_size ();
      std::copy (r->end () - V, r->end (), logits);
    }
  catch (const std::exception &e)
    {
      return fail (m, absl::InternalError (e.what ()));
    }
  return 0;
}

extern "C" int
vkl_model_generate_greedy (vkl_model *m, const uint32_t *prompt,
                           size_t n_prompt, size_t n_gen, uint32_t *out_ids,
                           double *prefill_ms, double *decode_ms)
{
  if (!m || !m->model || !prompt || !out_ids)
    return (int)absl::StatusCode::kInvalidArgument;
  try
    {
      std::vector<uint32_t> p (prompt, prompt + n_prompt), out;
      auto s = m->model->generate_greedy (p, n_gen, out, prefill_ms,
                                          decode_ms);
      if (!s.ok ())
        return fail (m, s);
      std::copy (out.begin (), out.end (), out_ids);
    }
  catch (const std::exception &e)
    {
      return fail (m, absl::InternalError (e.what ()));
    }
  return 0;
}

extern "C" int
vkl_model_generate_sampled (vkl_model *m, const uint32_t *prompt,
                            size_t n_prompt, size_t n_gen, int topk,
                            float topp, uint64_t seed, uint32_t *out_ids,
                            double *prefill_ms, double *decode_ms)
{
  if (!m || !m->model || !prompt || !out_ids)
    return (int)absl::StatusCode::kInvalidArgument;
  try
    {
      std::vector<uint32_t> p (prompt, prompt + n_prompt), out;
      auto s = m->model->generate_sampled (p, n_gen, topk, topp, seed, out,
                                           prefill_ms, decode_ms);
      if (!s.ok ())
        return fail (m, s);
      std::copy (out.begin (), out.end (), out_ids);
    }
  catch (const std::exception &e)
    {
      return fail (m, absl::InternalError (e.what ()));
    }
  return 0;
}

extern "C" int
vkl_model_set_option (vkl_model *m, const char *name, int value)
{
  if (!m || !m->model || !name)
    return (int)absl::StatusCode::kInvalidArgument;
  const std::string n (name);
  if (n == "fused_decode")
    m->model->set_fused_decode (value != 0);
  else if (n == "lastblock_rope_quirk")
    m->model->set_lastblock_rope_quirk (value != 0);
  else if (n == "operator_attention")
    m->model->set_operator_attention (value != 0);
  else if (n == "decode_mode")
    m->model->set_decode_mode (value);
  else if (n == "decode_graph")
    m->model->set_decode_graph (value != 0);
  else if (n == "phase_timing")
    vkl_decode_phase_timing (value);
  else if (n == "fuse_attn_wo" || n == "wait_test" || n == "attn_split_min")
    {
      // options of this model's fused decode steps (fields of vkl_decode_model)
      if (!m->model->set_decode_option (name, value))
        return fail (m, absl::InvalidArgumentError ("option " + n + ": value out of range"));
    }
  else
    return fail (m, absl::InvalidArgumentError ("unknown option " + n));
  return 0;
}

extern "C" int
vkl_model_read_kv_cache (vkl_model *m, size_t layer, int value, uint16_t *out,
                         size_t n)
{
  if (!m || !m->model || !out)
    return (int)absl::StatusCode::kInvalidArgument;
  std::vector<uint16_t> buf;
  auto s = m->model->read_kv_cache (layer, value != 0, buf);
  if (!s.ok ())
    return fail (m, s);
  if (n < buf.size ())
    return fail (m, absl::OutOfRangeError ("output buffer too small"));
  std::copy (buf.begin (), buf.end (), out);
  return 0;
}

extern "C" int
vkl_model_write_kv_cache (vkl_model *m, size_t layer, int value, const uint16_t *rows,
                          size_t n)
{
  if (!m || !m->model || !rows)
    return (int)absl::StatusCode::kInvalidArgument;
  auto s = m->model->write_kv_cache (layer, value != 0, rows, n);
  return s.ok () ? 0 : fail (m, s);
}

extern "C" size_t
vkl_model_decode_recoveries (const vkl_model *m)
{
  return m && m->model ? m->model->decode_recoveries () : 0;
}

extern "C" size_t
vkl_model_decode_step_bytes (const vkl_model *m, size_t L)
{
  return m && m->model ? m->model->decode_step_bytes (L) : 0;
}

extern "C" int
vkl_model_phase_times (vkl_model *m, double ms_sum[VKL_DECODE_PHASES],
                       uint64_t launches[VKL_DECODE_PHASES])
{
  if (!m || !ms_sum || !launches)
    return (int)absl::StatusCode::kInvalidArgument;
  return vkl_decode_phase_times (ms_sum, launches) == 0
             ? 0
             : (int)absl::StatusCode::kInternal;
}

extern "C" int
vkl_model_phase_replay (vkl_model *m, int kind, size_t pos, int rounds,
                        double *avg_ms, uint64_t *launches)
{
  if (!m || !m->model || !avg_ms)
    return (int)absl::StatusCode::kInvalidArgument;
  auto s = m->model->decode_phase_replay (kind, pos, rounds, avg_ms, launches);
  return s.ok () ? 0 : fail (m, s);
}

extern "C" size_t
vkl_model_phase_bytes (const vkl_model *m, int kind, size_t L)
{
  return m && m->model ? m->model->decode_phase_bytes (kind, L) : 0;
}

// ---------------------------------------------------------------------------
// synthetic weights
// ---------------------------------------------------------------------------
namespace
{
inline uint64_t
splitmix64 (uint64_t x)
{
  x += 0x9e3779b97f4a7c15ull;
  x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
  x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
  return x ^ (x >> 31);
}

// pair j of stream `seed`: Box-Muller on two 24-bit uniforms
inline void
normal_pair (uint64_t seed, uint64_t j, float std, float &a, float &b)
{
  const uint64_t r = splitmix64 (seed * 0x2545f4914f6cdd1dull + j);
  const float u1 = ((float)((r >> 40) & 0xffffff) + 1.0f) * (1.0f / 16777216.0f);
  const float u2 = (float)((r >> 8) & 0xffffff) * (1.0f / 16777216.0f);
  const float rad = std * sqrtf (-2.0f * logf (u1));
  const float ang = 6.283185307179586f * u2;
  a = rad * cosf (ang);
  b = rad * sinf (ang);
}

inline float
normal_at (uint64_t seed, uint64_t i, float std)
{
  float a, b;
  normal_pair (seed, i >> 1, std, a, b);
  return (i & 1) ? b : a;
}
}

extern "C" void
vkl_synth_normal_f32 (uint64_t seed, size_t n, float std, float *out)
{
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i)
    out[i] = normal_at (seed, i, std);
}

extern "C" void
vkl_synth_normal_f16 (uint64_t seed, size_t n, float std, uint16_t *out)
{
#pragma omp parallel for schedule(static)
  for (size_t i = 0; i < n; ++i)
    out[i] = __fp32_to_fp16_rne (normal_at (seed, i, std)).u16;
}

extern "C" void
vkl_synth_normal_q8_0 (uint64_t seed, size_t rows, size_t K, float std,
                       uint8_t *out)
{
  const size_t rb = vkl_q8_0_row_bytes (K);
#pragma omp parallel
  {
    std::vector<float> row (K);
#pragma omp for schedule(static)
    for (size_t r = 0; r < rows; ++r)
      {
        // element i of the stream comes from pair i/2; rows start on an even
        // index when K is even, then one pair fills two neighbours
        const size_t base = r * K;
        size_t k = 0;
        if (base & 1)
          row[k] = normal_at (seed, base, std), ++k;
        for (; k + 1 < K; k += 2)
          normal_pair (seed, (base + k) >> 1, std, row[k], row[k + 1]);
        if (k < K)
          row[k] = normal_at (seed, base + k, std);
        vkl_quantize_q8_0_h (row.data (), K, out + r * rb);
      }
  }
}

// ---- host samplers -----------------------------------------------------------
#include "models/samplers.h"
#include <memory>

struct vkl_sampler
{
  std::unique_ptr<Sampler> impl;
};

extern "C" int
vkl_sampler_create (int kind, float param, int seeded, uint64_t seed,
                    vkl_sampler **out)
{
  if (!out || (kind != 0 && kind != 1))
    return 1;
  if (kind == 0 && !(param >= 1.0f))
    return 1;
  auto *s = new vkl_sampler;
  if (kind == 0)
    s->impl.reset (seeded ? new TopkSampler ((size_t)param, seed)
                          : new TopkSampler ((size_t)param));
  else
    s->impl.reset (seeded ? new TopPSampler (param, seed) : new TopPSampler (param));
  *out = s;
  return 0;
}

extern "C" void
vkl_sampler_destroy (vkl_sampler *s)
{
  delete s;
}

extern "C" int
vkl_sampler_sample (vkl_sampler *s, const float *logits, size_t n)
{
  if (!s || !logits)
    return -1;
  return s->impl->sample (logits, n);
}

extern "C" size_t
vkl_sampler_candidates (const vkl_sampler *s, int32_t *ids, float *probs,
                        size_t cap)
{
  if (!s)
    return 0;
  const auto &c = s->impl->candidates ();
  for (size_t i = 0; i < c.size () && i < cap; ++i)
    {
      if (ids)
        ids[i] = c[i].second;
      if (probs)
        probs[i] = c[i].first;
    }
  return c.size ();
}
