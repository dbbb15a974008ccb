/*
 * CPU oracle for the llama2 token loop.  TEST INFRASTRUCTURE ONLY: nothing in
 * the shipped library may link, load or call this file.  It restates, in
 * plain C, the arithmetic of the reference's compute shaders and host code
 * (each function cites the reference file:line it follows) so that the HIP
 * kernels can be checked against it on the same seeded inputs.
 *
 * fp16 values are carried as uint16_t bit patterns.  Every function rounds to
 * fp16 (round-to-nearest-even) exactly where the reference stores a
 * float16_t and keeps fp32 in between.
 *
 * Q8_0 rows use the GGUF block the reference shaders read:
 * { fp16 d; int8 q[32]; } = 34 bytes (src/shaders/common.h:8-10).
 */
#ifndef VKL_ORACLE_H
#define VKL_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VKO_Q8_0_BLOCK 32
#define VKO_Q8_0_BYTES 34

/* ---- fp16 <-> fp32 ---------------------------------------------------- */
uint16_t vko_f32_to_f16 (float f);      /* RNE, software            */
uint16_t vko_f32_to_f16_hw (float f);   /* F16C when compiled in    */
float vko_f16_to_f32 (uint16_t h);
/* src/core/float.h:31-144: the reference's HOST helper (truncating). */
uint16_t vko_ref_host_f32_to_f16 (float f);

/* ---- Q8_0 ------------------------------------------------------------- */
/* src/core/quants.h:35-96.  scale_bytes = 2 -> 34-byte blocks with an fp16
 * (RNE) scale; scale_bytes = 4 -> the reference host format, 36-byte blocks
 * with the fp32 scale. */
void vko_q8_0_quantize_row (const float *src, size_t n, uint8_t *dst,
                            int scale_bytes);
/* src/core/quants.h:98-139 */
void vko_q8_0_dequantize_row (const uint8_t *src, size_t n, float *dst,
                              int scale_bytes);

/* ---- single ops -------------------------------------------------------- */
/* src/shaders/embedding_q8_0.comp:39-85 / embedding_fp16.comp */
void vko_embedding_q8_0 (const uint8_t *table, uint32_t VH, uint32_t VW,
                         const uint32_t *toks, uint32_t n, uint32_t unk,
                         uint16_t *out);
void vko_embedding_f16 (const uint16_t *table, uint32_t VH, uint32_t VW,
                        const uint32_t *toks, uint32_t n, uint32_t unk,
                        uint16_t *out);
/* src/shaders/rms_norm_fp16.comp:36-78 */
void vko_rmsnorm_f16 (const uint16_t *x, const float *w, int rows, int W,
                      float eps, uint16_t *out);
/* src/shaders/matmul_b0_fp16_x_q8_0.comp:52-139: y[m,n] = act(scale *
 * sum_k x[m,k] deq(W[n,k]) + bias) */
/* order in which the dot-product kernels add the 32 lanes of a subgroup
 * (subgroupAdd, implementation-defined in Vulkan): 0 pairwise halving (the
 * default), 1 sequential, 2 neighbours first, 3 sequential from the last
 * lane, 4 groups of eight then the groups.  Process-wide; for tests. */
void vko_set_lane_order (int order);
void vko_matmul_q8_0 (const uint16_t *x, const uint8_t *w, int M, int N,
                      int K, float scale, float bias, int act, uint16_t *y);
/* src/shaders/kqv_fp16_x_q8_0.comp:42-139 */
void vko_kqv_q8_0 (const uint16_t *x, const uint8_t *wk, const uint8_t *wq,
                   const uint8_t *wv, int M, int N, int K, uint16_t *k,
                   uint16_t *q, uint16_t *v);
/* src/shaders/ffn_up_and_gate_q8_0.comp:42-139: silu(x Wgate^T) * (x Wup^T) */
void vko_ffn_upgate_q8_0 (const uint16_t *x, const uint8_t *wup,
                          const uint8_t *wgate, int M, int N, int K,
                          uint16_t *out);
/* src/shaders/matmul_b0_tb_fp16_v2.comp:36-130: C channels, A [C,M,K] with
 * element strides (acs,ahs), B [C,N,K] with (bcs,bhs), Y [C,M,N] dense. */
void vko_matmul_f16_tb (const uint16_t *a, const uint16_t *b, int C, int M,
                        int N, int K, size_t acs, size_t ahs, size_t bcs,
                        size_t bhs, float scale, float bias, int act,
                        uint16_t *y);
/* src/shaders/matmul_broadcast0_fp16_v2.comp:36-104 with transpose_b = 0:
 * Y[c,m,n] = sum_k A[c,m,k] B[c,k,n]. */
void vko_matmul_f16_nn (const uint16_t *a, const uint16_t *b, int C, int M,
                        int N, int K, size_t acs, size_t ahs, size_t bcs,
                        size_t bhs, float scale, float bias, int act,
                        uint16_t *y);
/* src/shaders/ffn_up_and_gate_fp16.comp */
void vko_ffn_upgate_f16 (const uint16_t *x, const uint16_t *wup,
                         const uint16_t *wgate, int M, int N, int K,
                         uint16_t *out);
/* src/ops/rope.cpp:19-47: tables [maxlen, dim/2] */
void vko_rope_tables (int maxlen, int dim, float *freqc, float *freqs);
/* src/shaders/rope_fp16.comp:18-49: x [C,H,W] in place, row y uses table
 * row y + offset */
void vko_rope_f16 (uint16_t *x, int C, int H, int W, const float *freqc,
                   const float *freqs, uint32_t offset);
/* src/shaders/update_kvcache_fp16.comp:21-39 */
void vko_update_kvcache_f16 (uint16_t *cache, const uint16_t *kv, int C,
                             int HO, int H, int W, uint32_t offset);
/* src/shaders/softmax_fp16.comp:21-76 */
void vko_softmax_f16 (const uint16_t *x, int C, int H, int W, int seq_mask,
                      uint32_t offset, uint16_t *out);
/* src/shaders/element_wise_fp16.comp:13-50: out = fp16(x op y), op 0..3 =
 * add, sub, mul, div */
void vko_elementwise_f16 (const uint16_t *x, const uint16_t *y, size_t n,
                          int op, uint16_t *out);
/* src/shaders/argmax_stage0_fp16.comp + argmax_stage1.comp: first index of
 * the row maximum */
void vko_argmax_f16 (const uint16_t *x, int rows, int W, uint32_t *out);
uint32_t vko_argmax_f32 (const float *x, int n);
/* src/shaders/transpose_type0_fp16.comp: [C,H,W] -> [H,C,W] */
void vko_transpose102_f16 (const uint16_t *x, int C, int H, int W,
                           uint16_t *out);

/* ---- model -------------------------------------------------------------- */
typedef struct
{
  int dim, n_layers, n_heads, head_dim, ffn, vocab, maxlen;
  float eps;       /* per-block RMSNorm eps (GGUF kv)               */
  float final_eps; /* models/llama2.h:268 hard-codes 1e-6           */
  int wtype;       /* GGML type of the matrices: 8 = Q8_0, 1 = FP16 */
  int lastblock_rope_quirk; /* 1 = reference behaviour (last block's query
                               row is rotated at position `offset`)  */
  const void *tok_embd; /* [vocab, dim]  */
  const void *output;   /* [vocab, dim]  */
  const float *output_norm;
  const void *const *wq, *const *wk, *const *wv, *const *wo;
  const void *const *w_gate, *const *w_up, *const *w_down;
  const float *const *attn_norm, *const *ffn_norm;
} vko_model;

typedef struct vko_state vko_state;
vko_state *vko_state_create (const vko_model *m);
void vko_state_destroy (vko_state *s);
/* models/llama2.h:683-843: one forward over n_toks tokens at `offset`;
 * writes vocab fp32 logits of the last token. Returns 0 on success. */
int vko_forward (const vko_model *m, vko_state *s, const uint32_t *toks,
                 int n_toks, size_t offset, float *logits);
/* app/llama2_infer.cpp:140-218: prompt pass at offset 0, then one token at a
 * time; greedy = first index of the maximum logit. out_ids gets n_gen ids. */
int vko_generate_greedy (const vko_model *m, vko_state *s,
                         const uint32_t *prompt, int n_prompt, int n_gen,
                         uint32_t *out_ids, float *first_logits);
/* read access to a layer's caches, [heads, maxlen, head_dim] fp16 */
const uint16_t *vko_state_kcache (const vko_state *s, int layer);
const uint16_t *vko_state_vcache (const vko_state *s, int layer);
/* hidden state after block `layer` of the most recent forward, [rows, dim] */
const uint16_t *vko_state_hidden (const vko_state *s, int *rows);

#ifdef __cplusplus
}
#endif
#endif
