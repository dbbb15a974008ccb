// MultiHeadAttentionV2: interface of the reference's
// src/ops/multiheadattention_v2.h:25-83.  `dim` is the per-head width.
#ifndef __VKLLAMA_MULTIHEADATTENTIONV2_H__
#define __VKLLAMA_MULTIHEADATTENTIONV2_H__
#include "src/core/tensor.h"
#include "src/ops/elementwise.h"
#include "src/ops/feed_forward.h"
#include "src/ops/mat_mul.h"
#include "src/ops/op.h"
#include "src/ops/rope.h"
#include "src/ops/slice.h"
#include "src/ops/softmax.h"
#include "src/ops/transpose.h"
#include "src/ops/update_kv_cache.h"
#include <memory>
#include <vector>

namespace vkllama
{
class MultiHeadAttentionV2 : public Op
{
public:
  MultiHeadAttentionV2 (GPUDevice *dev, Command *command, Tensor wk, Tensor wq,
                        Tensor wv, Tensor wo, const int maxlen, const int dim,
                        const bool transposed_weight = false,
                        Tensor::DType dtype = FP16,
                        const bool use_kvcache = false,
                        const bool clip_output = false);

  absl::StatusOr<Tensor> operator() (Tensor X,
                                     const size_t offset = 0) noexcept;
  absl::Status init () noexcept override;
  uint64_t time () noexcept override;

  // The reference rotates the clipped (last-block) query at position
  // `offset` instead of offset + rows - 1 (multiheadattention_v2.cpp:222-233,
  // 251 with rope_fp16.comp:34).  true (default) reproduces that.
  void set_lastblock_rope_quirk (bool on) { rope_quirk_ = on; }
  // true: scores, softmax and P V run as the three operators of the reference
  // (probabilities rounded to fp16 one by one, multiheadattention_v2.cpp:272-317)
  // instead of the one-launch attention with its running maximum
  void set_operator_attention (bool on) { operator_attention_ = on; }

  // the next call only: the residual is added in the output projection's launch
  void set_residual (const Tensor *r) noexcept { residual_ = r; }

  Tensor &wk () { return wk_; }
  Tensor &wq () { return wq_; }
  Tensor &wv () { return wv_; }
  Tensor &wo () { return wo_; }
  Tensor &kcache () { return kcache_; }
  Tensor &vcache () { return vcache_; }
  Rope *rope () { return rope_q_.get (); }

private:
  const Tensor *residual_ = nullptr;
  Tensor wk_, wq_, wv_, wo_;
  Tensor kcache_, vcache_;
  const int maxlen_;
  const int dim_;
  const bool transposed_weight_;
  Tensor::DType dtype_;
  const bool use_kvcache_;
  const bool clip_output_;
  bool rope_quirk_;

  std::unique_ptr<MatMul> matmul_o_;
  std::unique_ptr<MatMul> matmul_qk_;
  std::unique_ptr<MatMul> matmul_weighted_;
  std::unique_ptr<MatMul> matmul_k_, matmul_q_, matmul_v_; // FP16 weights
  std::unique_ptr<Softmax> softmax_;
  std::unique_ptr<Rope> rope_q_;
  std::unique_ptr<Rope> rope_k_;
  std::unique_ptr<Transpose> transpose_k_;
  std::unique_ptr<Transpose> transpose_q_;
  std::unique_ptr<Transpose> transpose_v_;
  std::unique_ptr<Transpose> transpose_heads_;
  std::unique_ptr<UpdateKVCache> update_kcache_op_;
  std::unique_ptr<UpdateKVCache> update_vcache_op_;
  std::unique_ptr<Slice> clip_output_op_;
  Tensor k_, q_, v_;
  Tensor attn_out_;     // [1, S, heads*dim] of the one-launch attention
  OpTimer attn_timer_;
  bool attn_fused_last_ = false;
  bool operator_attention_ = false;
};
}
#endif
