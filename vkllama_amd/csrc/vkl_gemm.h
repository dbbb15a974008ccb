// Internal interface of the MFMA GEMM used for prompt passes (many token
// rows): y[M,N] = x[M,K] W[N,K]^T with fp16 activations and either planar
// Q8_0 or dense fp16 weights.  Called by the extern "C" launchers in
// vkl_gemv_q8.hip and vkl_matmul_f16.hip when M is large enough.
#ifndef VKL_GEMM_H
#define VKL_GEMM_H
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace vkl
{
struct GemmArgs
{
  const uint16_t *x; // [M, K] fp16, row stride xs (elements)
  size_t xs;
  int M, N, K;       // K: valid columns of x
  int Kp;            // K rounded up to 32 (rows of the int8 plane)
  int wtype;         // 8 = planar Q8_0, 1 = fp16 [N, K], 2 = fp16 [K, N]
  int batch;         // independent problems (grid y); 0 means 1
  size_t xbs, wbs, ybs; // element strides between the problems of a batch
  int nmat;          // 1, or 3 independent matrices/outputs (grid z)
  int upgate;        // 1: w[0] = up, w[1] = gate, y = silu(x gate^T) * (x up^T)
  const uint8_t *wq[3];  // Q8_0: int8 planes [N, Kp]
  const uint16_t *wd[3]; // Q8_0: fp16 scale planes [N, Kp/32]
  const uint16_t *wh[3]; // fp16: [N, K] (or [K, N] for wtype 2), row stride ws
  size_t ws;
  uint16_t *y[3]; // [M, N] fp16, row stride ys
  size_t ys;
  float scale, bias;
  int act;                  // 1: SiLU
  const uint16_t *residual; // y = fp16(fp16(v) + residual), stride ys
  float *y32;               // dense [M, N] widened copy
  // fp32 scratch for partial sums (k-split forms); null: the launcher's own
  // per-stream buffer, allocated on first use
  float *workspace;
  size_t workspace_bytes; // size of `workspace` (checked before every use)
};

// smallest M for which the matrix-core kernels beat one weight-streaming pass
// per token row (measured on the 7B shapes): Q8_0 weights, fp16 weights, and
// batched fp16 products (one small matrix per head)
constexpr int kGemmMinRows = 2;
constexpr int kGemmMinRowsF16 = 3;
constexpr int kGemmMinRowsBatched = 9;

// true if the shapes/alignments are ones the kernel covers
bool gemm_mfma_supported (const GemmArgs &a);
// Which kernel family gemm_mfma_launch takes for a problem, and how: decided
// in ONE place (gemm_plan), which the launcher follows and the workspace
// query reads, so the two cannot disagree.  Pure host arithmetic: no GPU call.
enum GemmFamily
{
  GEMM_NONE = 0,     // not covered (the caller falls back to one pass per token row)
  GEMM_ROWSFULL = 1, // <= 128 rows, workgroups over the whole of K (vkl_gemm_rowsfull.hip)
  GEMM_ROWS128 = 2,  // <= 32 rows, K sliced, four independent waves, whole-line loads
  GEMM_ROWS64 = 3,   // <= 32 rows, K sliced, 64 weight rows per workgroup
  GEMM_SLICES = 4,   // <= 32 rows, K sliced, 32 weight rows per workgroup (fp16 weights)
  GEMM_WIDE = 5,     // many rows, direct-to-LDS tiles (vkl_gemm_wide.hip)
  GEMM_TILE = 6      // the general tile kernel
};
struct GemmPlan
{
  int family;
  int tile_rows; // token rows of a tile / of a launch's row block
  int ksplit;    // parts of the k range whose fp32 sums go through the workspace (1: none)
  int groups;    // rowsfull: 16-row groups per workgroup
  int launches;  // kernel launches, the reduction included
  size_t workspace_bytes;
};
GemmPlan gemm_plan (const GemmArgs &a);
int gemm_mfma_launch (const GemmArgs &a, hipStream_t s);
// bytes of fp32 scratch gemm_mfma_launch will use for this problem (0: none)
size_t gemm_mfma_workspace_bytes (const GemmArgs &a);
// Many token rows against dense fp16 weights: 256-row tiles staged by
// direct-to-LDS loads (vkl_gemm_wide.hip).  gemm_mfma_launch takes this form
// where it applies.
bool gemm_wide_supported (const GemmArgs &a);
void gemm_wide_choice (const GemmArgs &a, int *tile_rows, int *ksplit); // tile_rows 0: another form
int gemm_wide_launch (const GemmArgs &a, hipStream_t s);
size_t gemm_wide_workspace_bytes (const GemmArgs &a); // fp32 scratch of its k-split (0: none)
// At most 96 token rows against many rows of Q8_0 weights, each workgroup over
// the whole of K: no partial sums (vkl_gemm_rowsfull.hip).
bool gemm_rowsfull_supported (const GemmArgs &a);
int gemm_rowsfull_groups (const GemmArgs &a);  // 16-row groups per workgroup, 0: another form
int gemm_rowsfull_launch_rows (const GemmArgs &a); // token rows of one launch
int gemm_rowsfull_launch (const GemmArgs &a, hipStream_t s);
// The k-split forms' fp32 scratch of a stream (allocated on first use; null if
// that fails), its size, and the kernel that adds `parts` partial results of
// `rows` rows each in order and applies the epilogue.
float *gemm_stream_workspace (hipStream_t s);
size_t gemm_stream_workspace_bytes ();
int gemm_reduce_parts (const GemmArgs &a, const float *ws, int parts, int rows, hipStream_t s);
// frees the scratch buffer that launches on this stream allocated (the
// stream must be idle); called when a stream is destroyed
void gemm_release_workspace (hipStream_t s);
// this GPU's copy of the library's static scratch array and its size in bytes
// (resolved once per device); null if the address cannot be resolved
float *gemm_static_scratch (size_t *bytes);

// One token row: y[N] = W[N, K] x[K] (+ residual) on the weight-streaming
// kernel of the decode step (vkl_decode.hip); W planar Q8_0 (wtype 8) or
// dense fp16 [N, K] (wtype 1).
bool decode_gemv_supported (int N, int K, int wtype);
int decode_gemv_launch (const void *x, const void *w, int wtype, int N, int K,
                        const void *residual, void *y, hipStream_t s);
}
#endif
