// Multi-head attention over a KV cache, operator by operator, following the
// control flow of the reference's src/ops/multiheadattention_v2.cpp:140-325:
//   K,Q,V = X Wk^T, X Wq^T, X Wv^T            (one fused launch for Q8_0)
//   [S, H, hd] -> (clip: last query row) -> [H, S, hd]
//   RoPE(Q), RoPE(K); cache[:, offset + y] = K, V
//   scores = fp16(Q K^T / sqrt(hd)) over the first L cache rows
//   P = softmax(scores, masked iff l > s + (L - S)); O = P V
//   [H, S, hd] -> [1, S, H*hd]; out = O Wo^T
// This is the general path (any S, used for prefill and by callers of the
// class); the model's one-token decode step runs the fused kernels instead.
#include "src/ops/multiheadattention_v2.h"
#include "src/core/command.h"
#include "vkl_hip.h"
#include <algorithm>
#include <cmath>

namespace vkllama
{
MultiHeadAttentionV2::MultiHeadAttentionV2 (
    GPUDevice *dev, Command *command, Tensor wk, Tensor wq, Tensor wv,
    Tensor wo, const int maxlen, const int dim, const bool transposed_weight,
    Tensor::DType dtype, const bool use_kvcache, const bool clip_output)
    : Op (dev, command), wk_ (wk), wq_ (wq), wv_ (wv), wo_ (wo),
      maxlen_ (maxlen), dim_ (dim), transposed_weight_ (transposed_weight),
      dtype_ (dtype), use_kvcache_ (use_kvcache), clip_output_ (clip_output),
      rope_quirk_ (true)
{
}

absl::Status
MultiHeadAttentionV2::init () noexcept
{
  if (dtype_ != FP16)
    return absl::InvalidArgumentError (
        "MultiHeadAttentionV2: only fp16 dtype is supported.");
  if (wk_.channels () != wq_.channels () || wk_.height () != wq_.height ()
      || wk_.width () != wq_.width () || wq_.channels () != wv_.channels ()
      || wq_.width () != wv_.width () || wq_.height () != wv_.height ())
    return absl::InvalidArgumentError (absl::StrFormat (
        "shape of weights error"
        "wk.shape = (%zu, %zu, %zu), wq.shape = (%zu, %zu, %zu), wv.shape = "
        "(%zu, %zu, %zu), wo.shape = (%zu, %zu, %zu)",
        wk_.channels (), wk_.height (), wk_.width (), wq_.channels (),
        wq_.height (), wq_.width (), wv_.channels (), wv_.height (),
        wv_.width (), wo_.channels (), wo_.height (), wo_.width ()));
  if (!transposed_weight_)
    return absl::InvalidArgumentError (
        "MultiHeadAttentionV2: only transposed ([out, in]) weights are "
        "supported");
  if (wk_.dtype () != wq_.dtype () || wk_.dtype () != wv_.dtype ()
      || (wk_.dtype () != Q8_0 && wk_.dtype () != FP16))
    return absl::InvalidArgumentError (
        "MultiHeadAttentionV2: Wk/Wq/Wv must share one of Q8_0 or FP16");
  if (dim_ <= 0 || maxlen_ <= 0 || wk_.height () % dim_ != 0
      || wk_.channels () != 1)
    return absl::InvalidArgumentError (absl::StrFormat (
        "MultiHeadAttentionV2: head dim %d does not divide %zu", dim_,
        wk_.height ()));

  matmul_o_ = std::make_unique<MatMul> (dev_, command_, wo_, 1.0, 0, 0, 0,
                                        transposed_weight_, FP16,
                                        wo_.dtype ());
  const float attn_score_scale = 1.0f / std::sqrt (static_cast<float> (dim_));
  matmul_qk_ = std::make_unique<MatMul> (dev_, command_, attn_score_scale, 0,
                                         0, 0, 1, FP16, FP16);
  matmul_weighted_
      = std::make_unique<MatMul> (dev_, command_, 1.0, 0, 0, 0, 0, FP16, FP16);
  rope_q_ = std::make_unique<Rope> (dev_, command_, maxlen_, dim_, dtype_);
  softmax_ = std::make_unique<Softmax> (dev_, command_, true, 1.0, dtype_);
  transpose_k_ = std::make_unique<Transpose> (dev_, command_, 0, dtype_);
  transpose_q_ = std::make_unique<Transpose> (dev_, command_, 0, dtype_);
  transpose_v_ = std::make_unique<Transpose> (dev_, command_, 0, dtype_);
  transpose_heads_ = std::make_unique<Transpose> (dev_, command_, 0, dtype_);
  VKLLAMA_STATUS_OK (matmul_o_->init ());
  VKLLAMA_STATUS_OK (matmul_qk_->init ());
  VKLLAMA_STATUS_OK (matmul_weighted_->init ());
  VKLLAMA_STATUS_OK (rope_q_->init ());
  VKLLAMA_STATUS_OK (softmax_->init ());
  VKLLAMA_STATUS_OK (transpose_k_->init ());
  VKLLAMA_STATUS_OK (transpose_q_->init ());
  VKLLAMA_STATUS_OK (transpose_v_->init ());
  VKLLAMA_STATUS_OK (transpose_heads_->init ());
  if (wk_.dtype () == FP16)
    {
      // The reference has no FP16 projection here (it always runs its Q8_0
      // shader); defined as three fp32-accumulating FP16 products.
      matmul_k_ = std::make_unique<MatMul> (dev_, command_, wk_, 1.0, 0, 0, 0,
                                            true, FP16, FP16);
      matmul_q_ = std::make_unique<MatMul> (dev_, command_, wq_, 1.0, 0, 0, 0,
                                            true, FP16, FP16);
      matmul_v_ = std::make_unique<MatMul> (dev_, command_, wv_, 1.0, 0, 0, 0,
                                            true, FP16, FP16);
      VKLLAMA_STATUS_OK (matmul_k_->init ());
      VKLLAMA_STATUS_OK (matmul_q_->init ());
      VKLLAMA_STATUS_OK (matmul_v_->init ());
    }
  if (use_kvcache_)
    {
      kcache_ = Tensor (wk_.height () / dim_, maxlen_, dim_, dev_, dtype_,
                        false);
      vcache_ = Tensor (wv_.height () / dim_, maxlen_, dim_, dev_, dtype_,
                        false);
      VKLLAMA_STATUS_OK (kcache_.create ());
      VKLLAMA_STATUS_OK (vcache_.create ());
      if (int e = vkl_memset (kcache_.data (), 0, kcache_.bytes (),
                              dev_->stream ()))
        return launch_status ("clearing the K cache", e);
      if (int e = vkl_memset (vcache_.data (), 0, vcache_.bytes (),
                              dev_->stream ()))
        return launch_status ("clearing the V cache", e);
      update_kcache_op_
          = std::make_unique<UpdateKVCache> (dev_, command_, dtype_);
      update_vcache_op_
          = std::make_unique<UpdateKVCache> (dev_, command_, dtype_);
      VKLLAMA_STATUS_OK (update_kcache_op_->init ());
      VKLLAMA_STATUS_OK (update_vcache_op_->init ());
    }
  if (clip_output_)
    {
      clip_output_op_.reset (new Slice (dev_, command_, dtype_));
      VKLLAMA_STATUS_OK (clip_output_op_->init ());
    }
  return absl::OkStatus ();
}

absl::StatusOr<Tensor>
MultiHeadAttentionV2::operator() (Tensor X, const size_t offset) noexcept
{
  if (X.dtype () != dtype_)
    return absl::InvalidArgumentError (
        absl::StrFormat ("multiheadattention op defined with %d dtype but "
                         "input0's dtype = %d",
                         int (dtype_), int (X.dtype ())));
  if (wv_.width () != X.width () || X.channels () != 1)
    return absl::InvalidArgumentError (
        absl::StrFormat ("shape error. wv.shape = (%zu, %zu, %zu), "
                         "input0.shape = (%zu, %zu, %zu)",
                         wv_.channels (), wv_.height (), wv_.width (),
                         X.channels (), X.height (), X.width ()));
  if (!matmul_o_)
    return absl::InternalError ("multiheadattention op used before init()");
  const size_t S = X.height (), N = wk_.height (), heads = N / dim_;
  if (use_kvcache_ && offset + S > (size_t)maxlen_)
    return absl::OutOfRangeError (absl::StrFormat (
        "multiheadattention: positions [%zu, %zu) exceed the cache length %d",
        offset, offset + S, maxlen_));

  Tensor k, q, v;
  if (wk_.dtype () == Q8_0)
    {
      if (!(k_.channels () == 1 && k_.height () == S && k_.width () == N))
        {
          k_ = Tensor (1, S, N, dev_, FP16, false);
          q_ = Tensor::like (k_);
          v_ = Tensor::like (k_);
          VKLLAMA_STATUS_OK (k_.create ());
          VKLLAMA_STATUS_OK (q_.create ());
          VKLLAMA_STATUS_OK (v_.create ());
        }
      VKLLAMA_STATUS_OK (k_.reshape (1, S, N));
      VKLLAMA_STATUS_OK (q_.reshape (1, S, N));
      VKLLAMA_STATUS_OK (v_.reshape (1, S, N));
      timer_.start (dev_);
      const int err = vkl_kqv_q8_0 (X.data (), wk_.data (), wq_.data (),
                                    wv_.data (), (int)S, (int)N,
                                    (int)X.width (), k_.data (), q_.data (),
                                    v_.data (), dev_->stream ());
      timer_.stop (dev_);
      VKLLAMA_STATUS_OK (launch_status ("kqv", err));
      k = k_, q = q_, v = v_;
    }
  else
    {
      auto rk = (*matmul_k_) (X);
      VKLLAMA_STATUS_OK (rk);
      auto rq = (*matmul_q_) (X);
      VKLLAMA_STATUS_OK (rq);
      auto rv = (*matmul_v_) (X);
      VKLLAMA_STATUS_OK (rv);
      k = *rk, q = *rq, v = *rv;
    }

  // With a cache and fp16 activations the rest of the operator is two
  // launches on the projection outputs as they lie ([S, heads*dim]): RoPE of
  // Q and K + cache write, then scores / masked softmax / P V.  Reshapes,
  // transposes, the clip of Q to its last row and the cache views of the
  // operator-by-operator form below become index arithmetic.  RoPE and the
  // cache rows are bit-identical to that form; the attention kernel rounds
  // scores and outputs where the operators do but forms its softmax with a
  // running maximum (see vkl_attn_prefill_causal_f16).
  attn_fused_last_ = false;
  if (!operator_attention_ && use_kvcache_ && dtype_ == FP16 && (dim_ == 64 || dim_ == 128)
      && k.dtype () == FP16 && q.dtype () == FP16 && v.dtype () == FP16)
    {
      const int q_row0 = clip_output_ ? (int)S - 1 : 0;
      const int q_rows = clip_output_ ? 1 : (int)S;
      const size_t q_pos0
          = clip_output_ && !rope_quirk_ ? offset + S - 1 : offset;
      if (!(attn_out_.channels () == 1 && attn_out_.height () == (size_t)q_rows
            && attn_out_.width () == N))
        {
          attn_out_ = Tensor (1, q_rows, N, dev_, FP16, false);
          VKLLAMA_STATUS_OK (attn_out_.create ());
        }
      attn_timer_.start (dev_);
      int err = vkl_rope_kvwrite_f16 (
          q.data (), k.data (), v.data (), (int)S, (int)heads, dim_, N, q_row0,
          q_rows, (uint32_t)q_pos0, (uint32_t)offset,
          (const float *)rope_q_->freqc ().data (),
          (const float *)rope_q_->freqs ().data (), maxlen_, kcache_.data (),
          vcache_.data (), maxlen_, dev_->stream ());
      if (err == 0)
        err = vkl_attn_prefill_causal_f16 (
            (const uint16_t *)q.data () + (size_t)q_row0 * N, kcache_.data (),
            vcache_.data (), (int)heads, q_rows, (int)(offset + S), dim_,
            (size_t)dim_, N, (size_t)maxlen_ * dim_, (size_t)dim_,
            (size_t)maxlen_ * dim_, (size_t)dim_,
            1.0f / std::sqrt ((float)dim_), attn_out_.data (), N,
            (size_t)dim_, dev_->stream ());
      attn_timer_.stop (dev_);
      VKLLAMA_STATUS_OK (launch_status ("attention", err));
      attn_fused_last_ = true;
      matmul_o_->set_residual (residual_);
      residual_ = nullptr;
      return (*matmul_o_) (attn_out_);
    }

  // [seqlen, heads, dim]
  VKLLAMA_STATUS_OK (k.reshape (S, heads, dim_));
  VKLLAMA_STATUS_OK (q.reshape (S, heads, dim_));
  VKLLAMA_STATUS_OK (v.reshape (S, heads, dim_));

  // clip to last token
  if (clip_output_)
    {
      std::array<uint32_t, 3> starts
          = { uint32_t (q.channels () - 1), uint32_t (0), uint32_t (0) };
      std::array<uint32_t, 3> sizes
          = { uint32_t (1), uint32_t (q.height ()), uint32_t (q.width ()) };
      auto ret = (*clip_output_op_) (q, starts, sizes);
      VKLLAMA_STATUS_OK (ret);
      q = *ret;
    }

  //[heads, seqlen, dim]
  auto transposed_k = (*transpose_k_) (k);
  auto transposed_q = (*transpose_q_) (q);
  auto transposed_v = (*transpose_v_) (v);
  VKLLAMA_STATUS_OK (transposed_k);
  VKLLAMA_STATUS_OK (transposed_q);
  VKLLAMA_STATUS_OK (transposed_v);

  const size_t q_offset
      = clip_output_ && !rope_quirk_ ? offset + S - 1 : offset;
  auto roped_q = (*rope_q_) (*transposed_q, q_offset);
  auto roped_k = (*rope_q_) (*transposed_k, offset);
  VKLLAMA_STATUS_OK (roped_k);
  VKLLAMA_STATUS_OK (roped_q);

  if (use_kvcache_)
    {
      VKLLAMA_STATUS_OK (
          (*update_kcache_op_) (kcache_, *roped_k, (uint32_t)offset));
      VKLLAMA_STATUS_OK (
          (*update_vcache_op_) (vcache_, *transposed_v, (uint32_t)offset));
      const uint32_t read_len = std::min (
          (uint32_t)(offset + transposed_k->height ()), (uint32_t)maxlen_);
      roped_k = kcache_.view (kcache_.channels (), read_len, kcache_.width ());
      transposed_v
          = vcache_.view (vcache_.channels (), read_len, vcache_.width ());
    }

  // scores, masked softmax and P V in one launch, written as [seqlen,
  // heads*dim]: the three operators below without the [heads, seqlen,
  // read_len] tensors in memory (online softmax: outputs within 5e-3 of
  // theirs relative to the size of the terms summed)
  if (!operator_attention_ && dtype_ == FP16 && (dim_ == 64 || dim_ == 128)
      && roped_q->dtype () == FP16 && roped_k->dtype () == FP16 && transposed_v->dtype () == FP16)
    {
      const size_t Sq = roped_q->height (), Lk = roped_k->height ();
      if (!(attn_out_.channels () == 1 && attn_out_.height () == Sq
            && attn_out_.width () == heads * (size_t)dim_))
        {
          attn_out_ = Tensor (1, Sq, heads * dim_, dev_, FP16, false);
          VKLLAMA_STATUS_OK (attn_out_.create ());
        }
      attn_timer_.start (dev_);
      const int err = vkl_attn_prefill_causal_f16 (
          roped_q->data (), roped_k->data (), transposed_v->data (),
          (int)heads, (int)Sq, (int)Lk, dim_, roped_q->cs () / 2,
          roped_q->hs () / 2, roped_k->cs () / 2, roped_k->hs () / 2,
          transposed_v->cs () / 2, transposed_v->hs () / 2,
          1.0f / std::sqrt ((float)dim_), attn_out_.data (),
          heads * (size_t)dim_, (size_t)dim_, dev_->stream ());
      attn_timer_.stop (dev_);
      VKLLAMA_STATUS_OK (launch_status ("attention", err));
      attn_fused_last_ = true;
      matmul_o_->set_residual (residual_);
      residual_ = nullptr;
      return (*matmul_o_) (attn_out_);
    }

  // [heads, seqlen, read_len]
  auto attn_scores = (*matmul_qk_) (*roped_q, *roped_k);
  VKLLAMA_STATUS_OK (attn_scores);
  const auto softmax_offset = attn_scores->width () - attn_scores->height ();
  auto softmax_attn_scores = (*softmax_) (*attn_scores, softmax_offset);
  VKLLAMA_STATUS_OK (softmax_attn_scores);

  // [heads, seqlen, dim]
  auto heads_out = (*matmul_weighted_) (*softmax_attn_scores, *transposed_v);
  VKLLAMA_STATUS_OK (heads_out);

  //[seqlen, heads, dim]
  auto concated = (*transpose_heads_) (*heads_out);
  VKLLAMA_STATUS_OK (concated);
  //[1, seqlen, heads*dim]
  VKLLAMA_STATUS_OK (concated->reshape (
      1, concated->channels (), concated->height () * concated->width ()));
  matmul_o_->set_residual (residual_);
  residual_ = nullptr;
  return (*matmul_o_) (*concated);
}

uint64_t
MultiHeadAttentionV2::time () noexcept
{
  uint64_t t = timer_.micros ();
  if (attn_fused_last_ && use_kvcache_)
    return t + attn_timer_.micros () + matmul_o_->time ();
  t += std::max ({ transpose_k_->time (), transpose_q_->time (),
                   transpose_v_->time () });
  if (use_kvcache_)
    t += std::max (update_kcache_op_->time (), update_vcache_op_->time ());
  t += rope_q_->time () + matmul_o_->time ();
  if (attn_fused_last_)
    t += attn_timer_.micros ();
  else
    t += matmul_qk_->time () + softmax_->time () + matmul_weighted_->time ()
         + transpose_heads_->time ();
  return t;
}
}
