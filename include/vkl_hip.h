/*
 * C ABI of libvkllama_hip.so: the HIP/gfx950 layer that replaces the
 * reference's Vulkan device, command-buffer, pipeline and shader layer
 * (src/core/gpu_device.*, src/core/command.h, src/core/pipeline.*,
 * every compute shader under src/shaders/).  The C++ operator classes in vkllama_amd/src/ops call
 * nothing else.
 *
 * Conventions
 *  - every function returns 0 on success or a hipError_t value;
 *    vkl_error_string() turns it into text.  Shape violations return
 *    hipErrorInvalidValue (1) before anything is launched.
 *  - pointers are device pointers unless the name ends in _h.
 *  - `stream` is a hipStream_t passed as void*; launches are asynchronous.
 *  - fp16 data is IEEE binary16 (uint16_t bit patterns on the host side).
 *  - strides are in ELEMENTS, not bytes.
 *  - Q8_0 tensors live on the device in the PLANAR layout: for a matrix of
 *    `rows` rows and K columns, nb = ceil(K/32):
 *        int8  q[rows][nb*32]   at byte offset 0
 *        fp16  d[rows][nb]      at byte offset rows*nb*32
 *    (34*nb bytes per row in total, the same count as the GGUF block layout
 *    { fp16 d; int8 q[32]; } of src/shaders/common.h:8-10).  vkl_q8_0_pack /
 *    vkl_q8_0_unpack convert between the two on the device.
 */
#ifndef VKL_HIP_H
#define VKL_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- device, streams, memory: replaces src/core/gpu_device.h:13-37 and the
 * submit/wait/upload/download half of src/core/command.h:26-483 ---------- */
typedef struct
{
  int device;
  int compute_units;
  int wavefront_size;
  int max_lds_bytes;
  size_t total_mem;
  char name[128];
  char arch[64];
} vkl_device_info;

int vkl_device_count (int *n);
int vkl_device_open (int dev, vkl_device_info *info);
const char *vkl_error_string (int err);
int vkl_stream_create (void **stream);
int vkl_stream_destroy (void *stream);
int vkl_stream_sync (void *stream);
int vkl_device_sync (void);
int vkl_malloc (void **p, size_t bytes);
int vkl_free (void *p);
int vkl_host_malloc_h (void **p, size_t bytes); /* pinned */
int vkl_host_free_h (void *p);
int vkl_memcpy_h2d (void *dst, const void *src_h, size_t bytes, void *stream);
int vkl_memcpy_d2h (void *dst_h, const void *src, size_t bytes, void *stream);
int vkl_memcpy_d2d (void *dst, const void *src, size_t bytes, void *stream);
int vkl_memset (void *dst, int value, size_t bytes, void *stream);
/* free and total device memory in bytes (the budget query of the reference's
 * allocator, src/core/allocator.cpp, as far as callers need it) */
int vkl_mem_info (size_t *free_bytes, size_t *total_bytes);
/* device-to-device copy by a plain streaming kernel (bytes % 16 == 0, both
 * pointers 16-byte aligned): the known-size launch that hardware traffic
 * counters are calibrated against; no counterpart in the reference */
int vkl_copy_kernel (void *dst, const void *src, size_t bytes, void *stream);
/* timing: replaces the timestamp queries of src/core/pipeline.cpp:425-445 */
int vkl_event_create (void **ev);
int vkl_event_destroy (void *ev);
int vkl_event_record (void *ev, void *stream);
int vkl_event_sync (void *ev);
int vkl_event_elapsed_ms (void *start, void *stop, float *ms);

/* ---- Q8_0: src/core/quants.h:35-139 ------------------------------------ */
/* host quantiser, 34-byte blocks, fp16 (RNE) scale */
void vkl_quantize_q8_0_h (const float *src_h, size_t n, uint8_t *dst_h);
void vkl_dequantize_q8_0_h (const uint8_t *src_h, size_t n, float *dst_h);
size_t vkl_q8_0_row_bytes (size_t K);
/* GGUF 34-byte blocks (device) <-> planar (device) */
int vkl_q8_0_pack (const void *raw, void *planar, size_t rows, size_t K,
                   void *stream);
int vkl_q8_0_unpack (const void *planar, void *raw, size_t rows, size_t K,
                     void *stream);

/* ---- operators -------------------------------------------------------- */
/* src/ops/embedding.cpp:58-114, src/shaders/embedding_q8_0.comp,
 * embedding_fp16.comp.  toks: device uint32 [n]; out fp16 [n, VW]. */
int vkl_embed_q8_0 (const void *table_planar, uint32_t VH, uint32_t VW,
                    const uint32_t *toks, uint32_t n, uint32_t unk, void *out,
                    void *stream);
int vkl_embed_f16 (const void *table, uint32_t VH, uint32_t VW,
                   const uint32_t *toks, uint32_t n, uint32_t unk, void *out,
                   void *stream);
/* src/ops/rms_norm.cpp:60-91, src/shaders/rms_norm_fp16.comp */
int vkl_rmsnorm_f16 (const void *x, const float *w, int rows, int W,
                     float eps, void *out, void *stream);
/* src/ops/mat_mul.cpp:159-228 with FP16 x Q8_0, transpose_b:
 * src/shaders/matmul_b0_fp16_x_q8_0.comp.  y[m,n] = act(scale * sum_k
 * x[m,k] W[n,k] + bias), act 1 = SiLU.  x [M,K] row stride xs; y [M,N] row
 * stride ys.  If residual != NULL: y = fp16(fp32(fp16(v)) + residual[m,n])
 * (the ElementWise add of models/llama2.h:193-196,209 folded in); residual may
 * alias y.  If y32 != NULL the fp16 result is also widened to fp32 there
 * (the Cast of models/llama2.h:294). */
int vkl_matmul_q8_0 (const void *x, const void *w_planar, int M, int N,
                     int K, size_t xs, size_t ys, float scale, float bias,
                     int act, const void *residual, void *y, float *y32,
                     void *stream);
/* vkl_matmul_q8_0 for callers that cannot allocate device memory (code under
 * HIP graph capture, serving loops and harnesses that forbid it); it has no
 * counterpart in the reference.  Same arguments, same kernels and bit-identical
 * results, but it calls no hipMalloc / hipFree: the fp32 partial sums that the
 * few-row and k-split kernels exchange (M from 2 up to a few hundred rows) go
 * through a static device array of 8 MiB that every GPU the library runs on
 * holds until the process ends (its address on a device is looked up once, at
 * vkl_device_open or at the first call there).  A problem whose partial sums
 * do not fit (e.g. 2..32 rows: 128 * N * ceil(K / 1024) bytes) is refused with
 * hipErrorInvalidValue.  All calls on one GPU share the array: calls that
 * overlap in time on one GPU (different streams) race. */
int vkl_matmul_q8_0_noalloc (const void *x, const void *w_planar, int M,
                             int N, int K, size_t xs, size_t ys, float scale,
                             float bias, int act, const void *residual,
                             void *y, float *y32, void *stream);
/* A testing aid without counterpart in the reference: the address (on the
 * current device) and size of the static device array that
 * vkl_matmul_q8_0_noalloc uses as scratch, so that a test can mark it and see
 * that a call wrote there and nowhere else. */
int vkl_debug_static_scratch (void **ptr, size_t *bytes);
/* Which kernel family a matrix product with M token rows takes, and how (no
 * counterpart in the reference, whose one shader serves every row count): the
 * launchers of this header decide it in one host function, and this query
 * returns that decision without touching the GPU, so that tests can pin the
 * kernel a workload runs on.  wtype 8 = Q8_0, 1 = FP16 weights; nmat 3 = the
 * fused K/Q/V product; upgate 1 = the fused up/gate pair; workspace_bytes 0 =
 * the launcher's own scratch, else a caller's (the no-allocation entry point
 * passes 8 MiB).  Operands are taken to be dense and 16-byte aligned.
 * family: 0 none, 1 whole-K workgroups (<= 128 rows), 2 / 3 / 4 K slices + a
 * reduction launch (<= 32 rows), 5 direct-to-LDS tiles, 6 the general tile
 * kernel, 7 one weight-streaming pass per token row. */
typedef struct
{
  int family, tile_rows, ksplit, groups, launches;
  size_t workspace_bytes;
} vkl_gemm_plan_t;
int vkl_gemm_plan (int M, int N, int K, int wtype, int nmat, int upgate,
                   size_t workspace_bytes, vkl_gemm_plan_t *out);
/* src/ops/multiheadattention_v2.cpp:190-202, src/shaders/kqv_fp16_x_q8_0.comp */
int vkl_kqv_q8_0 (const void *x, const void *wk, const void *wq,
                  const void *wv, int M, int N, int K, void *k, void *q,
                  void *v, void *stream);
/* src/ops/feed_forward.cpp:106-120, src/shaders/ffn_up_and_gate_q8_0.comp:
 * out = fp16(silu(x Wgate^T) * (x Wup^T)) */
int vkl_ffn_upgate_q8_0 (const void *x, const void *wup, const void *wgate,
                         int M, int N, int K, void *out, void *stream);
/* src/shaders/matmul_b0_tb_fp16_v2.comp: Y[c,m,n] = act(scale * sum_k
 * A[c,m,k] B[c,n,k] + bias); A strides (acs, ahs), B (bcs, bhs), Y (ycs, yhs).
 * residual / y32 as for vkl_matmul_q8_0 (dense [C*M, N]). */
int vkl_matmul_f16_tb (const void *a, const void *b, int C, int M, int N,
                       int K, size_t acs, size_t ahs, size_t bcs, size_t bhs,
                       size_t ycs, size_t yhs, float scale, float bias,
                       int act, const void *residual, void *y, float *y32,
                       void *stream);
/* src/shaders/matmul_broadcast0_fp16_v2.comp, transpose_b = 0:
 * Y[c,m,n] = act(scale * sum_k A[c,m,k] B[c,k,n] + bias) */
int vkl_matmul_f16_nn (const void *a, const void *b, int C, int M, int N,
                       int K, size_t acs, size_t ahs, size_t bcs, size_t bhs,
                       size_t ycs, size_t yhs, float scale, float bias,
                       int act, void *y, void *stream);
/* src/shaders/ffn_up_and_gate_fp16.comp */
int vkl_ffn_upgate_f16 (const void *x, const void *wup, const void *wgate,
                        int M, int N, int K, void *out, void *stream);
/* src/ops/rope.cpp:112-150, src/shaders/rope_fp16.comp: in place on x
 * [C,H,W]; tables fp32 [rows, W/2]; row y uses table row y + offset. */
int vkl_rope_f16 (void *x, int C, int H, int W, const float *freqc,
                  const float *freqs, uint32_t offset, void *stream);
/* src/ops/update_kv_cache.cpp:36-76, src/shaders/update_kvcache_fp16.comp:
 * cache[c, (offset+y) % HO, :] = kv[c, y, :] */
int vkl_kv_update_f16 (void *cache, const void *kv, int C, int HO, int H,
                       int W, uint32_t offset, void *stream);
/* src/ops/softmax.cpp:52-92, src/shaders/softmax_fp16.comp */
int vkl_softmax_f16 (const void *x, int C, int H, int W, int seq_mask,
                     uint32_t offset, void *out, void *stream);
/* src/ops/multiheadattention_v2.cpp:205-287 in one launch, on the [S, H*hd]
 * outputs of the K/Q/V projections (row stride row_stride): the reshape and
 * Transpose of K, Q, V become index arithmetic, Rope (rope_fp16.comp) rotates
 * q rows [q_row0, q_row0 + q_rows) in place at positions q_pos0 + i and every
 * k row s at position k_pos0 + s, and UpdateKVCache (update_kvcache_fp16.comp)
 * writes the rotated k and v to rows (k_pos0 + s) % maxlen of [H, maxlen, hd]
 * caches.  freqc / freqs: fp32 [table_rows, hd/2]. */
int vkl_rope_kvwrite_f16 (void *q, const void *k, const void *v, int S, int H,
                          int hd, size_t row_stride, int q_row0, int q_rows,
                          uint32_t q_pos0, uint32_t k_pos0,
                          const float *freqc, const float *freqs,
                          int table_rows, void *kcache, void *vcache,
                          int maxlen, void *stream);
/* The attention core of src/ops/multiheadattention_v2.cpp:290-309 in one
 * launch for many query rows: matmul_b0_tb_fp16_v2.comp (scores = fp16(scale
 * q.k)), softmax_fp16.comp with seq_mask (key l is masked iff l > s + (L - S))
 * and matmul_broadcast0_fp16_v2.comp (P V), with neither scores nor
 * probabilities stored.  Scores and output are rounded to fp16 where the
 * shaders round them; the softmax runs with a running maximum and the
 * division by the sum of exponentials last, so the fp16 weights of the second
 * product are exp(score - max) instead of the normalised probabilities and
 * the sum adds them as rounded
 * (outputs within 5e-3 of the three shaders' relative to the size of the terms
 * summed; the operators' bar is 1e-2).  q [H,S,hd] with strides (qcs,
 * qhs); k, v [H,L,hd] views with strides (kcs, khs), (vcs, vhs), e.g. the
 * first L rows of a [H,maxlen,hd] cache; out[s*ors + h*ohs + d] (ors = H*hd,
 * ohs = hd gives the [S, H*hd] layout the output projection reads; ors = hd,
 * ohs = S*hd gives [H,S,hd]).  hd 64 or 128; strides in elements. */
int vkl_attn_prefill_causal_f16 (const void *q, const void *k, const void *v,
                                 int H, int S, int L, int hd, size_t qcs,
                                 size_t qhs, size_t kcs, size_t khs,
                                 size_t vcs, size_t vhs, float scale,
                                 void *out, size_t ors, size_t ohs,
                                 void *stream);
/* src/ops/elementwise.cpp:60-101, src/shaders/element_wise_fp16.comp:
 * y = fp16(x op y), in place into y; op 0..3 = add, sub, mul, div */
int vkl_elementwise_f16 (const void *x, void *y, size_t n, int op,
                         void *stream);
/* src/ops/elementwise.cpp:104-133, element_wise_constant_fp16.comp:
 * out = fp16(x op alpha) */
int vkl_elementwise_const_f16 (const void *x, float alpha, size_t n, int op,
                               void *out, void *stream);
/* src/ops/cast.cpp:40-77 */
int vkl_cast_f16_f32 (const void *x, float *out, size_t n, void *stream);
int vkl_cast_f32_f16 (const float *x, void *out, size_t n, void *stream);
/* src/ops/argop.h:72-140, argmax_stage0_fp16.comp + argmax_stage1.comp:
 * first index of the maximum (op 0) / minimum (op 1) of each row */
int vkl_argop_f16 (const void *x, int rows, int W, int op, uint32_t *out,
                   void *stream);
/* src/ops/slice.cpp:30-77, src/shaders/slice_fp16.comp */
int vkl_slice_f16 (const void *x, int C, int H, int W, int c0, int h0, int w0,
                   int CE, int HE, int WE, void *out, void *stream);
/* models/samplers.cpp:37-101 on the device: the next token drawn from one row
 * of V fp32 logits without the logits leaving device memory.  p < 0: the k
 * largest logits (TopkSampler; k = 1 is the arg-max); p in [0, 1]: the most
 * likely tokens until their mass reaches p (TopPSampler; at most 1024
 * candidates).  Candidates rank by logit, ties toward the lower id; their
 * probabilities are the softmax of the kept logits.  The draw inverts the
 * cumulative distribution at one uniform number per (seed, counter +
 * *counter_dev); counter_dev (device, optional) lets a position that lives
 * on the device advance the generator.  tok: device; cand_ids / cand_probs /
 * cand_n (device, optional, 1024 entries) receive the candidate set. */
int vkl_sample_f32 (const float *logits, int V, int k, float p, uint64_t seed,
                    uint32_t counter, const uint32_t *counter_dev,
                    uint32_t *tok, uint32_t *cand_ids, float *cand_probs,
                    uint32_t *cand_n, void *stream);
/* src/ops/concat.cpp:68-188, src/shaders/concat_fp16.comp: one input of a
 * Concat copied into the output: out[c*ocs + y*ohs + x + out_offset] =
 * x[c*xcs + y*xhs + x] (element strides; the operator gives each input the
 * offset of its position along the concatenation axis). */
int vkl_concat_part_f16 (const void *x, int C, int H, int W, size_t xcs,
                         size_t xhs, void *out, size_t ocs, size_t ohs,
                         size_t out_offset, void *stream);
/* src/ops/read_kvcache_op.cpp:31-70, src/shaders/read_kvcache_fp16.comp:
 * out[c, y, :] = cache[c, (y + offset) % H, :] for y < len; cache [C,H,W]. */
int vkl_read_kvcache_f16 (const void *cache, int C, int H, int W,
                          uint32_t offset, uint32_t len, void *out,
                          void *stream);
/* src/ops/reduce.h:17-120, src/shaders/reduce_fp16.comp: over the last axis of
 * [C,H,W], op 0 sum, 1 max, 2 min, 3 mean (sum * (1/W)); fp32 accumulation,
 * out [C,H] fp16. */
int vkl_reduce_f16 (const void *x, int C, int H, int W, int op, void *out,
                    void *stream);
/* src/ops/transpose.cpp:36-80 type 0, transpose_type0_fp16.comp:
 * [C,H,W] -> [H,C,W] */
int vkl_transpose102_f16 (const void *x, int C, int H, int W, void *out,
                          void *stream);

#ifdef __cplusplus
}
#endif
#endif
