#include "models/decode_plan.h"
#include "models/llama2.h"
#include "vkl_hip.h"
#include <string.h>
#include <string>

namespace vkllama
{
static absl::Status
hip_status (const char *what, int e)
{
  if (!e)
    return absl::OkStatus ();
  if (e == 1)
    return absl::InvalidArgumentError (
        absl::StrFormat ("%s: rejected by the HIP layer", what));
  return absl::InternalError (
      absl::StrFormat ("%s: %s", what, vkl_error_string (e)));
}

DecodePlan::DecodePlan ()
    : gpu_ (nullptr), usable_ (false), mode_ (1), adopted_valid_ (false),
      vocab_ (0)
{
  memset (&desc_, 0, sizeof (desc_));
}

DecodePlan::~DecodePlan ()
{
  // (back to the library's pool: memory of that kind is never freed)
  vkl_decode_flags_release (desc_.flags);
}

absl::Status
DecodePlan::build (Model &model, GPUDevice *gpu, InputLayer *in,
                   std::vector<Llama2Block *> &blocks, OutputLayer *out,
                   float eps)
{
  gpu_ = gpu;
  vocab_ = model.vocab_size ();
  tok_slot_ = Tensor (1, 1, 1, gpu, UINT32, true);
  VKLLAMA_STATUS_OK (tok_slot_.create ());
  logits32_ = Tensor (1, 1, (int)vocab_, gpu, FP32, false);
  VKLLAMA_STATUS_OK (logits32_.create ());

  Tensor &emb = in->embedding ()->vocab ();
  auto *attn0 = blocks[0]->attention ();
  const size_t dim = emb.width ();
  const size_t hd = attn0->kcache ().width ();
  const size_t heads = attn0->kcache ().channels ();
  const size_t ffn = blocks[0]->feed_forward ()->w1 ().height ();
  // The fused kernels index every layer with ONE set of dimensions and ONE
  // matrix type: they take models whose matrices are all Q8_0 or all FP16 and
  // whose blocks all have the shapes of block 0 (a block that is smaller or of
  // another type would be read past its end).
  const DType wt = emb.dtype ();
  bool uniform = (wt == Q8_0 || wt == FP16) && out->weight ().dtype () == wt
                 && out->weight ().width () == dim && out->weight ().height () == vocab_
                 && emb.height () == vocab_;
  auto is_mat = [wt] (Tensor &t, size_t rows, size_t cols) {
    return t.dtype () == wt && t.channels () == 1 && t.height () == rows && t.width () == cols;
  };
  for (auto *b : blocks)
    {
      auto *a = b->attention ();
      auto *f = b->feed_forward ();
      uniform = uniform && is_mat (a->wk (), dim, dim) && is_mat (a->wq (), dim, dim)
                && is_mat (a->wv (), dim, dim) && is_mat (a->wo (), dim, dim)
                && is_mat (f->w1 (), ffn, dim) && is_mat (f->w3 (), ffn, dim)
                && is_mat (f->w2 (), dim, ffn)
                && a->kcache ().channels () == heads && a->kcache ().width () == hd
                && a->kcache ().height () == attn0->kcache ().height ()
                && a->vcache ().channels () == heads && a->vcache ().width () == hd
                && a->vcache ().height () == attn0->kcache ().height ()
                && b->attn_norm ()->weight ().size () == dim
                && b->ffn_norm ()->weight ().size () == dim;
    }
  uniform = uniform && out->norm ()->weight ().size () == dim;
  // norm weights are read as fp32 by the fused kernels
  bool norms32 = out->norm ()->weight ().dtype () == FP32;
  for (auto *b : blocks)
    norms32 = norms32 && b->attn_norm ()->weight ().dtype () == FP32
              && b->ffn_norm ()->weight ().dtype () == FP32;
  if (!uniform || !norms32 || (hd != 64 && hd != 128) || heads * hd != dim || dim % 32
      || ffn % 32 || vocab_ % 2)
    {
      usable_ = false; // the operator chain serves these models
      return absl::OkStatus ();
    }

  std::vector<vkl_layer_weights> &lw = layers_h_;
  lw.assign (blocks.size (), vkl_layer_weights{});
  for (size_t i = 0; i < blocks.size (); ++i)
    {
      auto *a = blocks[i]->attention ();
      auto *f = blocks[i]->feed_forward ();
      lw[i].wk = a->wk ().data ();
      lw[i].wq = a->wq ().data ();
      lw[i].wv = a->wv ().data ();
      lw[i].wo = a->wo ().data ();
      lw[i].w_gate = f->w1 ().data ();
      lw[i].w_down = f->w2 ().data ();
      lw[i].w_up = f->w3 ().data ();
      lw[i].attn_norm = (const float *)blocks[i]->attn_norm ()->weight ().data ();
      lw[i].ffn_norm = (const float *)blocks[i]->ffn_norm ()->weight ().data ();
      lw[i].kcache = a->kcache ().data ();
      lw[i].vcache = a->vcache ().data ();
    }
  const size_t lbytes = lw.size () * sizeof (vkl_layer_weights);
  layers_ = Tensor (1, 1, (int)lbytes, gpu, INT8, false);
  VKLLAMA_STATUS_OK (layers_.create ());
  VKLLAMA_STATUS_OK (hip_status (
      "uploading layer table",
      vkl_memcpy_h2d (layers_.data (), lw.data (), lbytes, gpu->stream ())));
  VKLLAMA_STATUS_OK (
      hip_status ("uploading layer table", vkl_stream_sync (gpu->stream ())));

  desc_.dim = (int)dim;
  desc_.n_layers = (int)blocks.size ();
  desc_.n_heads = (int)heads;
  desc_.head_dim = (int)hd;
  desc_.ffn = (int)ffn;
  desc_.vocab = (int)vocab_;
  desc_.maxlen = (int)attn0->kcache ().height ();
  desc_.wtype = wt == Q8_0 ? 8 : 1; // GGML type numbers
  desc_.eps = eps;
  desc_.final_eps = out->norm ()->eps ();
  desc_.layers = (const vkl_layer_weights *)layers_.data ();
  desc_.layers_h = layers_h_.data ();
  desc_.tok_embd = emb.data ();
  desc_.output = out->weight ().data ();
  desc_.output_norm = (const float *)out->norm ()->weight ().data ();
  desc_.freqc = (const float *)attn0->rope ()->freqc ().data ();
  desc_.freqs = (const float *)attn0->rope ()->freqs ().data ();
  const size_t sbytes = vkl_decode_scratch_bytes (&desc_);
  scratch_ = Tensor (1, 1, (int)sbytes, gpu, INT8, false);
  VKLLAMA_STATUS_OK (scratch_.create ());
  VKLLAMA_STATUS_OK (hip_status (
      "clearing decode scratch",
      vkl_memset (scratch_.data (), 0, sbytes, gpu->stream ())));
  desc_.scratch = scratch_.data ();
  // (without such memory no launch waits: the step runs its launches per phase)
  if (vkl_decode_flags_acquire (&desc_.flags) != 0)
    desc_.flags = nullptr;
  // (the form that measured faster for this shape; set_mode overrides it)
  mode_ = vkl_decode_default_mode (&desc_);
  usable_ = true;
  return absl::OkStatus ();
}

absl::Status
DecodePlan::step_host_token (uint32_t tok, size_t offset)
{
  // the slot may still be read by a queued step
  VKLLAMA_STATUS_OK (
      hip_status ("waiting for the stream", vkl_stream_sync (gpu_->stream ())));
  *(uint32_t *)tok_slot_.host () = tok;
  return step_device_token ((const uint32_t *)tok_slot_.data (), offset);
}

absl::Status
DecodePlan::step_device_token (const uint32_t *tok, size_t offset,
                               uint32_t *next_tok)
{
  if (!usable_)
    return absl::FailedPreconditionError (
        "fused decode does not cover this model");
  adopted_valid_ = false;
  return hip_status ("decode step",
                     vkl_decode_step (&desc_, tok, (uint32_t)offset, mode_,
                                      (float *)logits32_.data (), next_tok,
                                      gpu_->stream ()));
}

absl::Status
DecodePlan::loop (uint32_t *ids, size_t pos0, size_t n_steps)
{
  if (!usable_)
    return absl::FailedPreconditionError (
        "fused decode does not cover this model");
  adopted_valid_ = false;
  return hip_status ("decode loop",
                     vkl_decode_loop (&desc_, ids, (uint32_t)pos0, (int)n_steps, mode_,
                                      (float *)logits32_.data (),
                                      gpu_->stream ()));
}

absl::Status
DecodePlan::loop_sampled (uint32_t *ids, size_t pos0, size_t n_steps, int topk, float topp,
                          uint64_t seed)
{
  if (!usable_)
    return absl::FailedPreconditionError (
        "fused decode does not cover this model");
  adopted_valid_ = false;
  return hip_status ("sampled decode loop",
                     vkl_decode_loop_sampled (&desc_, ids, (uint32_t)pos0, (int)n_steps, mode_,
                                              (float *)logits32_.data (), topk, topp, seed,
                                              gpu_->stream ()));
}

bool
DecodePlan::set_option (const char *name, int value)
{
  const std::string n (name);
  if (n == "attn_split_min")
    {
      if (value < 0)
        return false;
      desc_.attn_split_min = value;
    }
  else if (n == "fuse_attn_wo")
    desc_.separate_attn_wo = value ? 0 : 1;
  else if (n == "wait_test")
    {
      // value > 0: waits between workgroups give up after `value` polls and
      // the workgroups waited for never signal; 0: back to normal
      if (value < 0 || value >= (1 << 24))
        return false;
      desc_.wait_polls = value, desc_.wait_test = value > 0 ? 1 : 0;
    }
  else
    return false;
  return true;
}

absl::Status
DecodePlan::check ()
{
  // (mode 0 waits between workgroups too, in its fused attention + Wo launch)
  if (!usable_)
    return absl::OkStatus ();
  if (int e = vkl_decode_status (&desc_, gpu_->stream ()))
    {
      const bool had_waits = mode_ != 0 || !desc_.separate_attn_wo;
      mode_ = 0, desc_.separate_attn_wo = 1;
      return absl::UnavailableError (absl::StrFormat (
          "decode step: a wait between workgroups gave up (%s): the GPU is shared or "
          "deals workgroups to its XCDs in another order; %s",
          vkl_error_string (e),
          had_waits ? "switched to the launches that wait for nothing, repeat the call"
                    : "no such launch was in use"));
    }
  return absl::OkStatus ();
}

absl::Status
DecodePlan::adopt_logits (Tensor logits32)
{
  if (logits32.dtype () != FP32 || logits32.size () < vocab_)
    return absl::InvalidArgumentError ("logits tensor has the wrong type");
  adopted_ = logits32;
  adopted_valid_ = true;
  return absl::OkStatus ();
}

absl::Status
DecodePlan::read_logits (float *dst)
{
  const Tensor &src = adopted_valid_ ? adopted_ : logits32_;
  const float *p = (const float *)src.data () + (src.size () - vocab_);
  VKLLAMA_STATUS_OK (hip_status (
      "downloading logits",
      vkl_memcpy_d2h (dst, p, vocab_ * sizeof (float), gpu_->stream ())));
  VKLLAMA_STATUS_OK (hip_status ("downloading logits", vkl_stream_sync (gpu_->stream ())));
  return check ();
}

absl::Status
DecodePlan::argmax_logits (uint32_t *dst)
{
  const Tensor &src = adopted_valid_ ? adopted_ : logits32_;
  const float *p = (const float *)src.data () + (src.size () - vocab_);
  return hip_status ("argmax", vkl_argmax_f32 (p, (int)vocab_, dst,
                                               gpu_->stream ()));
}

absl::Status
DecodePlan::sample_logits (uint32_t *dst, int topk, float topp, uint64_t seed,
                           uint32_t counter)
{
  const Tensor &src = adopted_valid_ ? adopted_ : logits32_;
  const float *p = (const float *)src.data () + (src.size () - vocab_);
  return hip_status ("sample",
                     vkl_sample_f32 (p, (int)vocab_, topk, topp, seed, counter,
                                     nullptr, dst, nullptr, nullptr, nullptr,
                                     gpu_->stream ()));
}
}
