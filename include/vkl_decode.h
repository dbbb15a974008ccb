/*
 * C ABI of the fused one-token decode step (libvkllama_hip.so).  It replaces,
 * for a forward pass over ONE token, the chain of about 19 dispatches per
 * block that the reference records in models/llama2.h:160-213 +
 * src/ops/multiheadattention_v2.cpp:190-324 + src/ops/feed_forward.cpp:106-128
 * and the output layer of models/llama2.h:283-298, with five phases per block:
 *   1. RMSNorm + fused K/Q/V projection
 *   2. RoPE + KV-cache write + attention over the cache (fp16 scores and
 *      probabilities, as the reference materialises them)
 *   3. Wo projection + residual add
 *   4. RMSNorm + fused up/gate projection with SiLU
 *   5. down projection + residual add
 * then RMSNorm(eps 1e-6) + lm_head + fp32 widening + arg-max.  Every fp16
 * rounding point of the operator chain is kept.
 */
#ifndef VKL_DECODE_H
#define VKL_DECODE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct
{
  /* matrices [out, in]: planar Q8_0 (see vkl_hip.h) or dense fp16 */
  const void *wk, *wq, *wv, *wo, *w_gate, *w_up, *w_down;
  const float *attn_norm, *ffn_norm; /* [dim] fp32 */
  void *kcache, *vcache;             /* [heads, maxlen, head_dim] fp16 */
} vkl_layer_weights;

typedef struct
{
  int dim, n_layers, n_heads, head_dim, ffn, vocab, maxlen;
  int wtype; /* GGML type of the matrices: 8 = Q8_0, 1 = FP16 */
  float eps;       /* block RMSNorm eps */
  float final_eps; /* output RMSNorm eps (1e-6 in the reference) */
  const vkl_layer_weights *layers;   /* DEVICE array [n_layers] */
  const vkl_layer_weights *layers_h; /* the same table in HOST memory */
  const void *tok_embd;            /* [vocab, dim] */
  const void *output;              /* [vocab, dim] */
  const float *output_norm;        /* [dim] */
  const float *freqc, *freqs;      /* RoPE tables fp32 [maxlen, head_dim/2] */
  void *scratch; /* device, vkl_decode_scratch_bytes() bytes, zeroed once */
  /* Options of this model's decode steps; all zero = the defaults.  They are
   * part of the model, not of the process: two models in one process do not
   * share them, and the graphs vkl_decode_loop caches are keyed by them. */
  int attn_split_min;  /* context length from which the attention phase runs in
                          its split form (each head's rows over several
                          workgroups of one launch); 0 = 1024, the measured
                          break-even; a value beyond maxlen never splits.  The
                          split form weights the V rows with fp32
                          probabilities, the one-workgroup form with
                          probabilities rounded to fp16 as the reference's
                          softmax stores them: outputs differ by at most one
                          fp16 step */
  int separate_attn_wo; /* mode 0: attention (one workgroup per head) and the Wo
                          projection as two launches instead of one */
  int wait_polls;      /* polls after which a wait between workgroups inside a
                          launch gives up; 0 = the default (some 10 ms) */
  int wait_test;       /* testing aid: the workgroups that others wait for
                          never raise their flags, so every such wait gives
                          up */
  void *flags;         /* from vkl_decode_flags_acquire: the flags that
                          workgroups poll inside a launch.  Null: no launch
                          waits (mode 1 and the attention + Wo launch run as
                          the launches per phase) */
} vkl_decode_model;

/* The flags that the workgroups of a launch raise for one another live in
 * device memory that no cache holds: they are polled through the scalar memory
 * path, which the weight requests of a compute unit do not queue in, and a
 * cached copy in the poller's L2 would hide the store of another XCD.  Such
 * memory must never be freed once a kernel has read it (allocations made after
 * the free have held wrong values on this GPU), so the library keeps a pool:
 * acquire hands out a zeroed area of the current device (a new one only if
 * none is free), release returns it to the pool.  One area per model.
 * No counterpart in the reference. */
int vkl_decode_flags_acquire (void **flags);
void vkl_decode_flags_release (void *flags);

/* The launch form (the `mode` of vkl_decode_step and vkl_decode_loop) that
 * measured faster for this model's shape on the MI355X: 1, one launch per
 * layer, for rows of at most 4096 (dim) and 12288 (ffn) values when the model
 * has its flag area (7B shape: 8 % faster with Q8_0 weights, 3 % with FP16);
 * 0, one launch per phase, for wider rows (13B shape: the layer launch keeps
 * twice the row in registers, spills, and runs 7 % slower) and without flags.
 * Either value may be passed for any model that the form supports.
 * No counterpart in the reference. */
int vkl_decode_default_mode (const vkl_decode_model *m);

/* bytes of device scratch a model of these dimensions needs */
size_t vkl_decode_scratch_bytes (const vkl_decode_model *m);

/* One token at KV position `pos` (context length becomes pos + 1).
 *  tok      device-visible uint32: the input token id (ids >= vocab -> 0)
 *  mode     0 = one launch per phase (attention and Wo share one below the
 *           split length); 1 = one launch per layer: all workgroups stay
 *           resident through the five phases, hand activations over through
 *           memory with bounded waits for one another, and have the next
 *           phase's weights on the way meanwhile.  Results are bit for bit
 *           those of mode 0.  Positions at or above the split length (the
 *           attention then takes more than one workgroup per head) and
 *           models whose rows the one-launch form does not cover run as
 *           mode 0.  The GPU must not be shared while such a launch runs:
 *           see vkl_decode_status
 *  logits32 optional device fp32 [vocab]: widened fp16 logits
 *  next_tok optional device-visible uint32: arg-max id, lowest index on ties
 * Returns 0 or a hipError_t; hipErrorInvalidValue for shapes the kernels do
 * not cover (dim % 32, head_dim not 64/128, ffn % 32, pos >= maxlen, ...). */
int vkl_decode_step (const vkl_decode_model *m, const uint32_t *tok,
                     uint32_t pos, int mode, float *logits32,
                     uint32_t *next_tok, void *stream);

/* Launches in which workgroups wait for one another (mode 1; the attention +
 * Wo launch of mode 0) need every workgroup resident at once and the
 * same number of them on each XCD; where that does not hold (a GPU shared
 * with other work, another way of dealing workgroups to XCDs) a bounded wait
 * inside the kernel gives up or the kernel notices the placement, the launch
 * still ends,
 * the workgroup concerned drops its results instead of storing them, and the
 * step's results are invalid.  This call synchronises the stream and returns
 * 0 if nothing of the kind happened since the last call,
 * hipErrorLaunchFailure otherwise (the mark is cleared); the caller then
 * repeats the step with mode 0 and separate_attn_wo = 1, which wait for
 * nothing.  No counterpart in the reference, which has no such kernels. */
int vkl_decode_status (const vkl_decode_model *m, void *stream);

/* n_steps greedy tokens without a host round trip per token: step i reads
 * ids[i] (device memory) at position pos0 + i and writes its arg-max id to
 * ids[i + 1], the loop of app/llama2_infer.cpp:140-177 with the sampler on the
 * device.  The launches of one step are captured once in a HIP graph (per
 * model / buffers / attention form) and replayed; results are identical to
 * n_steps calls of vkl_decode_step in the same mode.  logits32 (optional)
 * receives the logits of the last step.  The stream must not be capturing. */
int vkl_decode_loop (const vkl_decode_model *m, uint32_t *ids, uint32_t pos0,
                     int n_steps, int mode, float *logits32, void *stream);

/* The same loop with the sampler of models/samplers.cpp:37-101 instead of the
 * arg-max as the last launch of every captured step (vkl_sample_f32's kernel:
 * topp < 0 keeps the topk largest logits, else the top-p set): the token of
 * position pos0 + i + 1 is drawn with the uniform number of (seed, that
 * position).  topk, topp and seed live in device memory, so one captured
 * graph serves every request; results are those of n_steps calls of
 * vkl_decode_step, each followed by vkl_sample_f32 with counter = position. */
int vkl_decode_loop_sampled (const vkl_decode_model *m, uint32_t *ids,
                             uint32_t pos0, int n_steps, int mode,
                             float *logits32, int topk, float topp,
                             uint64_t seed, void *stream);

/* device pointer to the fp16 logits [vocab] of the last step inside scratch */
const void *vkl_decode_logits_f16 (const vkl_decode_model *m);
/* arg-max over fp32 values (first maximum); out is device-visible */
int vkl_argmax_f32 (const float *x, int n, uint32_t *out, void *stream);

/* ------------------------------------------------------------------------
 * Measuring and testing aids.  None has a counterpart in the reference; the
 * product path (vkl_decode_step / vkl_decode_loop above) does not need them.
 * ------------------------------------------------------------------------ */

/* Phase timing (a measuring aid without counterpart in the
 * reference, whose GPUDevice timestamps play this role in
 * src/core/gpu_device.cpp).  While enabled, vkl_decode_step brackets every
 * phase launch with a pair of HIP events on the launch stream and
 * synchronises the stream before it returns.  vkl_decode_phase_times adds up,
 * per phase kind (0 K/Q/V, 1 attention, 2 Wo, 3 up/gate, 4 down, 5 lm_head
 * with the arg-max its last workgroup forms, 8 a whole layer in one launch as
 * mode 1 runs it; 6 and 7 are not used), the elapsed milliseconds and the
 * number of launches since the last call, and clears both.  The timer is one
 * per process: use it from one host thread, with no other decode call in
 * flight. */
#define VKL_DECODE_PHASES 9
#define VKL_DECODE_PHASE_LAYER 8
int vkl_decode_phase_timing (int enable);
int vkl_decode_phase_times (double ms_sum[VKL_DECODE_PHASES],
                            uint64_t launches[VKL_DECODE_PHASES]);
/* Launches phase `kind` (0..4 and 8: of every layer in turn; 5: lm_head) `rounds`
 * times back to back on `stream` between ONE pair of events and returns the
 * average milliseconds per launch: the kernel's duration without the cost of
 * an event pair per launch.  The phase's outputs in scratch are overwritten
 * (a following vkl_decode_step recomputes them); the KV cache is not touched
 * for kinds other than 1, and kind 1 rewrites the rows of position `pos` with
 * what scratch currently holds, so call it before, not between, real steps of
 * a sequence you still need. */
int vkl_decode_phase_replay (const vkl_decode_model *m, int kind, uint32_t pos,
                             int rounds, void *stream, double *avg_ms,
                             uint64_t *launches);
/* algorithmic bytes one launch of phase `kind` moves at context length L
 * (weights + scales read once; activations, KV rows and results once) */
size_t vkl_decode_phase_bytes (const vkl_decode_model *m, int kind, size_t L);

#ifdef __cplusplus
}
#endif
#endif
