/*
 * C ABI of libvkllama_host.so around the C++ drop-in classes
 * (vkllama_amd/src/ops, vkllama_amd/models/llama2.h): what a binding in
 * another language needs to drive the llama2 token loop of the reference's
 * app/llama2_infer.cpp:120-218 (model.init, model(toks, offset), greedy
 * sampling) without touching C++ types.
 *
 * All functions return 0 on success, otherwise an absl::StatusCode value
 * (3 = invalid argument, 11 = out of range, 13 = internal, ...);
 * vkl_model_last_error() gives the message.
 */
#ifndef VKL_MODEL_H
#define VKL_MODEL_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct vkl_model vkl_model;

/* one GGUF tensor as models/llama2.h:401-431,486-646 reads it:
 * type 0 = F32, 1 = F16, 8 = Q8_0 (34-byte blocks); dim0 = columns (input
 * features), dim1 = rows; data/bsize = the raw GGUF bytes. */
typedef struct
{
  const char *name;
  uint32_t type;
  uint64_t dim0, dim1;
  const void *data;
  uint64_t bsize;
} vkl_tensor_desc;

/* GGUF hyper-parameters models/llama2.h:367-370 reads */
typedef struct
{
  uint32_t head_count;    /* llama.attention.head_count */
  uint32_t block_count;   /* llama.block_count */
  uint32_t context_length; /* llama.context_length */
  float rms_eps;          /* llama.attention.layer_norm_rms_epsilon */
} vkl_model_hparams;

/* Model::Model(dev) + Model::init(kv, tensors) */
int vkl_model_create (int dev, const vkl_model_hparams *hp,
                      const vkl_tensor_desc *tensors, size_t n_tensors,
                      vkl_model **out);
/* The same from a GGUF file, the way app/llama2_infer.cpp:46-75,120-121 of
 * the reference loads a model: the file is mapped, its keys and tensors are
 * collected into the maps Model::init takes, the weights are uploaded, and
 * the mapping is released before this returns. */
int vkl_model_load_gguf (int dev, const char *path_h, vkl_model **out);
void vkl_model_destroy (vkl_model *m);
const char *vkl_model_last_error (const vkl_model *m);
size_t vkl_model_vocab (const vkl_model *m);

/* Model::operator()(toks, offset): fp32 logits of the last row -> logits_h
 * (vocab floats) */
int vkl_model_forward (vkl_model *m, const uint32_t *toks_h, size_t n_toks,
                       size_t offset, float *logits_h);
/* the greedy loop of app/llama2_infer.cpp:140-218; times in milliseconds */
int vkl_model_generate_greedy (vkl_model *m, const uint32_t *prompt_h,
                               size_t n_prompt, size_t n_gen,
                               uint32_t *out_ids_h, double *prefill_ms,
                               double *decode_ms);
/* the same loop with every token drawn on the device (vkl_sample_f32) from
 * the topk largest logits (topp < 0) or the top-p set; position pos uses the
 * uniform number of (seed, pos), so a seed reproduces the sequence */
int vkl_model_generate_sampled (vkl_model *m, const uint32_t *prompt_h,
                                size_t n_prompt, size_t n_gen, int topk,
                                float topp, uint64_t seed,
                                uint32_t *out_ids_h, double *prefill_ms,
                                double *decode_ms);
/* options, all per model: "fused_decode" (fused one-token decode on/off),
 * "decode_mode" (0 = one launch per phase, 1 = one launch per layer; the
 * default is what vkl_decode_default_mode says for the model's shape),
 * "decode_graph" (replay of the greedy loop from a HIP graph on/off),
 * "attn_split_min" (the context length from which attention is split over
 * several workgroups per head), "fuse_attn_wo" (mode 0: attention and the Wo
 * projection in one launch on/off), "lastblock_rope_quirk" (the reference's
 * last-block RoPE position), "operator_attention" (prompt pass: scores,
 * softmax and P V as the reference's three operators with probabilities
 * rounded to fp16 one by one, instead of the one-launch attention), "wait_test" (a testing aid: waits between
 * workgroups inside a launch give up after that many polls and are never
 * answered; 0 = normal), "phase_timing" (process-wide measuring aid) */
int vkl_model_set_option (vkl_model *m, const char *name, int value);
/* how often a decode step or a generation of this model was repeated, on the
 * launches that wait for nothing, because a wait between workgroups inside a
 * launch had given up (a shared GPU); 0 in normal operation */
size_t vkl_model_decode_recoveries (const vkl_model *m);
/* one layer's K (value = 0) or V (value = 1) cache, [heads, maxlen, hd] fp16 */
int vkl_model_read_kv_cache (vkl_model *m, size_t layer, int value,
                             uint16_t *out_h, size_t n);
/* A testing aid, the mirror of vkl_model_read_kv_cache (no counterpart in the
 * reference, which fills its caches only through
 * src/ops/update_kv_cache.cpp): replaces one layer's K (value = 0) or V cache
 * with n = heads * maxlen * head_dim fp16 values from host memory, so that a
 * test can put a model at a late position without the prompt pass that leads
 * there. */
int vkl_model_write_kv_cache (vkl_model *m, size_t layer, int value,
                              const uint16_t *rows_h, size_t n);
/* algorithmic bytes of one decode step at context length L */
size_t vkl_model_decode_step_bytes (const vkl_model *m, size_t L);
/* per-phase measurements of the fused decode step: option "phase_timing"
 * switches them on; see vkl_decode_phase_times / vkl_decode_phase_bytes */
int vkl_model_phase_times (vkl_model *m, double ms_sum[9], uint64_t launches[9]);
size_t vkl_model_phase_bytes (const vkl_model *m, int kind, size_t L);
/* vkl_decode_phase_replay on this model's stream; overwrites decode scratch */
int vkl_model_phase_replay (vkl_model *m, int kind, size_t pos, int rounds,
                            double *avg_ms, uint64_t *launches);

/* ---- synthetic weights (seeded, host) ----------------------------------
 * N(0, std) values from a counter-based generator: element i of stream
 * `seed` is a pure function of (seed, i), so tensors can be produced in
 * parallel and in any order. */
void vkl_synth_normal_f32 (uint64_t seed, size_t n, float std, float *out_h);
void vkl_synth_normal_f16 (uint64_t seed, size_t n, float std,
                           uint16_t *out_h);
/* rows x K matrix of N(0, std) quantised to Q8_0 GGUF blocks */
void vkl_synth_normal_q8_0 (uint64_t seed, size_t rows, size_t K, float std,
                            uint8_t *out_h);

/* ---- host samplers (models/samplers.h:8-43) ------------------------------
 * kind 0: TopkSampler (param = k), kind 1: TopPSampler (param = p).  seeded:
 * 0 seeds from std::random_device as the reference does, else from `seed`. */
typedef struct vkl_sampler vkl_sampler;
int vkl_sampler_create (int kind, float param, int seeded, uint64_t seed,
                        vkl_sampler **out);
void vkl_sampler_destroy (vkl_sampler *s);
/* a token id drawn for one row of n logits (host memory); -1 if n == 0 */
int vkl_sampler_sample (vkl_sampler *s, const float *logits_h, size_t n);
/* candidates of the last draw, most likely first: up to cap (id, probability)
 * pairs are written; returns how many candidates there were */
size_t vkl_sampler_candidates (const vkl_sampler *s, int32_t *ids_h,
                               float *probs_h, size_t cap);

#ifdef __cplusplus
}
#endif
#endif
