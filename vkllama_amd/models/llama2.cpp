// Llama-2 token loop on the HIP operator classes.  Control flow follows the
// reference's models/llama2.h: weight upload and block construction
// (:348-681), one forward pass (:683-843), block wiring (:160-213) and the
// output layer (:283-298).
#include "models/llama2.h"
#include "models/decode_plan.h"
#include "vkl_hip.h"
#include <chrono>
#include <stdexcept>
#include <string.h>

namespace vkllama
{
// ---------------------------------------------------------------------------
InputLayer::InputLayer (GPUDevice *gpu, Command *command, Tensor vocab,
                        uint32_t UNK)
    : gpu_ (gpu), command_ (command), vocab_ (vocab), UNK_ (UNK)
{
}

absl::Status
InputLayer::init ()
{
  embedding_op_.reset (
      new Embedding (gpu_, command_, vocab_, UNK_, vocab_.dtype ()));
  return embedding_op_->init ();
}

absl::StatusOr<Tensor>
InputLayer::operator() (Tensor toks)
{
  return embedding_op_->operator() (toks);
}

void
InputLayer::print_op_cost ()
{
  fprintf (stderr, "embedding lookup cost -- embedding cost: %llu\n",
           (unsigned long long)embedding_op_->time ());
}

// ---------------------------------------------------------------------------
Llama2Block::Llama2Block (GPUDevice *dev, Command *command,
                          TransformerParams const &transformer,
                          FeedForwardParams const &feed_forward,
                          RmsNormParams const &norm)
    : gpu_ (dev), command_ (command), transformer_params_ (transformer),
      feedforward_params_ (feed_forward), rmsnorm_params_ (norm)
{
}

absl::Status
Llama2Block::init ()
{
  attn_op_.reset (new MultiHeadAttentionV2 (
      gpu_, command_, transformer_params_.Wk, transformer_params_.Wq,
      transformer_params_.Wv, transformer_params_.Wo,
      transformer_params_.maxlen, transformer_params_.dim, true, FP16, true,
      transformer_params_.clip_output));
  feedforward_op_.reset (new FeedForward (
      gpu_, command_, feedforward_params_.w1, feedforward_params_.w2,
      feedforward_params_.w3, true, feedforward_params_.w1.dtype ()));
  norm_op_.reset (new RMSNorm (gpu_, command_, rmsnorm_params_.weight1,
                               rmsnorm_params_.eps, FP16));
  norm_op2_.reset (new RMSNorm (gpu_, command_, rmsnorm_params_.weight2,
                                feedforward_params_.eps, FP16));
  add_op_.reset (new ElementWise (gpu_, command_, 0, FP16));
  add_op2_.reset (new ElementWise (gpu_, command_, 0, FP16));
  VKLLAMA_STATUS_OK (attn_op_->init ());
  VKLLAMA_STATUS_OK (feedforward_op_->init ());
  VKLLAMA_STATUS_OK (norm_op_->init ());
  VKLLAMA_STATUS_OK (norm_op2_->init ());
  VKLLAMA_STATUS_OK (add_op_->init ());
  VKLLAMA_STATUS_OK (add_op2_->init ());
  if (transformer_params_.clip_output)
    {
      slice_op_.reset (new Slice (gpu_, command_, FP16));
      VKLLAMA_STATUS_OK (slice_op_->init ());
    }
  return absl::OkStatus ();
}

absl::StatusOr<Tensor>
Llama2Block::operator() (Tensor in, const size_t offset)
{
  // The residual additions of the reference's block (element_wise after the
  // attention and after the feed-forward part) run in the launches of the two
  // projections that precede them: the same fp16 values, two launches less.
  Tensor residual = in;
  if (transformer_params_.clip_output)
    {
      // the last block continues with the last row only
      std::array<uint32_t, 3> starts
          = { uint32_t (0), uint32_t (in.height () - 1), uint32_t (0) };
      std::array<uint32_t, 3> extents
          = { uint32_t (in.channels ()), uint32_t (1),
              uint32_t (in.width ()) };
      auto cliped = (*slice_op_) (in, starts, extents);
      VKLLAMA_STATUS_OK (cliped);
      residual = *cliped;
    }
  auto normed = norm_op_->operator() (in);
  VKLLAMA_STATUS_OK (normed);
  attn_op_->set_residual (&residual);
  auto added = attn_op_->operator() (*normed, offset);
  VKLLAMA_STATUS_OK (added);
  auto normed2 = norm_op2_->operator() (*added);
  VKLLAMA_STATUS_OK (normed2);
  feedforward_op_->set_residual (&*added);
  return feedforward_op_->operator() (*normed2);
}

void
Llama2Block::print_op_cost ()
{
  fprintf (stderr,
           "block cost -- attn norm cost: %llu, attn cost: %llu, attn add "
           "cost: %llu, ffn norm cost: %llu, ffn cost: %llu, ffn add cost: "
           "%llu\n",
           (unsigned long long)norm_op_->time (),
           (unsigned long long)attn_op_->time (),
           (unsigned long long)add_op_->time (),
           (unsigned long long)norm_op2_->time (),
           (unsigned long long)feedforward_op_->time (),
           (unsigned long long)add_op2_->time ());
}

// ---------------------------------------------------------------------------
OutputLayer::OutputLayer (GPUDevice *gpu, Command *command, Tensor wo,
                          Tensor norm_weight)
    : gpu_ (gpu), command_ (command), wo_ (wo), norm_weight_ (norm_weight)
{
}

absl::Status
OutputLayer::init ()
{
  matmul_op_.reset (new MatMul (gpu_, command_, wo_, 1.0, .0, 0, 0, true,
                                FP16, wo_.dtype ()));
  VKLLAMA_STATUS_OK (matmul_op_->init ());
  // the final norm's eps is fixed, not the GGUF value (models/llama2.h:268)
  norm_op_.reset (new RMSNorm (gpu_, command_, norm_weight_, 1e-6, FP16));
  VKLLAMA_STATUS_OK (norm_op_->init ());
  cast_op_.reset (new Cast (gpu_, command_, FP16, FP32));
  VKLLAMA_STATUS_OK (cast_op_->init ());
  argmax_op_.reset (new ArgMax (gpu_, command_, FP16));
  return argmax_op_->init ();
}

absl::StatusOr<Tensor>
OutputLayer::operator() (Tensor in)
{
  auto normed = norm_op_->operator() (in);
  VKLLAMA_STATUS_OK (normed);
  auto logits = matmul_op_->operator() (*normed);
  VKLLAMA_STATUS_OK (logits);
  return (*cast_op_) (*logits);
}

void
OutputLayer::print_op_cost ()
{
  fprintf (stderr,
           "output cost -- matmul out cost: %llu, norm cost: %llu, argmax "
           "cost: %llu\n",
           (unsigned long long)matmul_op_->time (),
           (unsigned long long)norm_op_->time (),
           (unsigned long long)argmax_op_->time ());
}

// ---------------------------------------------------------------------------
Model::Model (int dev)
    : dev_ (dev), gpu_ (nullptr), input_command_ (nullptr),
      output_command_ (nullptr), input_layer_ (nullptr),
      output_layer_ (nullptr), vocab_ (0), dim_ (0), ffn_ (0), heads_ (0),
      maxlen_ (0), wtype_ (Q8_0), fused_decode_ (true), plan_ (nullptr)
{
}

Model::~Model ()
{
  if (gpu_ && gpu_->stream ())
    vkl_stream_sync (gpu_->stream ());
  delete plan_;
  argmax_.reset ();
  vktoks_ = Tensor ();
  next_tok_ = Tensor ();
  delete input_layer_;
  delete output_layer_;
  for (auto *block : blocks_)
    delete block;
  delete input_command_;
  delete output_command_;
  for (auto c : block_commands_)
    delete c;
  delete gpu_;
}

static DType
to_dtype (const uint32_t type)
{
  // GGML tensor types (models/llama2.h:382-397 of the reference)
  if (type == 0)
    return FP32;
  if (type == 1)
    return FP16;
  if (type == 8)
    return Q8_0;
  return INT8;
}

namespace
{
absl::StatusOr<gguf_tensor>
find_tensor (std::map<std::string, gguf_tensor> &tensors,
             const std::string &name)
{
  auto it = tensors.find (name);
  if (it == tensors.end () || !it->second.weights_data)
    return absl::NotFoundError (
        absl::StrFormat ("model tensor %s is missing", name));
  return it->second;
}

// [rows = dim[1], cols = dim[0]] matrix (or [1, dim[0]] vector), uploaded raw
absl::StatusOr<Tensor>
upload_tensor (GPUDevice *gpu, Command *command, const gguf_tensor &t,
               bool vector)
{
  const DType dt = to_dtype (t.type);
  Tensor out (1, vector ? 1 : (int)t.dim[1], (int)t.dim[0], gpu, dt);
  VKLLAMA_STATUS_OK (out.create ());
  // bsize is not trusted beyond the tensor's own size (the reference passes
  // Tensor::bytes() for Wk/Wq/Wv and gguf bsize elsewhere, llama2.h:577-646)
  const size_t n = std::min<size_t> (t.bsize, out.bytes ());
  if (n < out.bytes ())
    return absl::OutOfRangeError (absl::StrFormat (
        "tensor %s holds %zu bytes, %zu needed", std::string (t.name ? t.name : "?"),
        (size_t)t.bsize, out.bytes ()));
  VKLLAMA_STATUS_OK (
      command->upload ((const uint8_t *)t.weights_data, n, out));
  return out;
}
}

absl::Status
Model::init (std::map<std::string, gguf_key> &kv,
             std::map<std::string, gguf_tensor> &tensors)
{
  gpu_ = new GPUDevice (dev_);
  VKLLAMA_STATUS_OK (gpu_->init ());
  input_command_ = new Command (gpu_);
  output_command_ = new Command (gpu_);
  VKLLAMA_STATUS_OK (input_command_->init ());
  VKLLAMA_STATUS_OK (output_command_->init ());

  for (const char *key :
       { "llama.attention.head_count", "llama.block_count",
         "llama.attention.layer_norm_rms_epsilon", "llama.context_length" })
    if (kv.find (key) == kv.end () || !kv[key].val)
      return absl::NotFoundError (
          absl::StrFormat ("model key %s is missing", key));
  const auto head_count = kv["llama.attention.head_count"].val->uint32;
  const auto block_count = kv["llama.block_count"].val->uint32;
  const auto norm_eps
      = kv["llama.attention.layer_norm_rms_epsilon"].val->float32;
  const auto maxlen = kv["llama.context_length"].val->uint32;
  if (head_count == 0 || block_count == 0 || maxlen == 0)
    return absl::InvalidArgumentError ("model hyper-parameters must be > 0");

  VKLLAMA_STATUS_OK (input_command_->begin ());
  VKLLAMA_STATUS_OK (output_command_->begin ());
  {
    auto embeddings = find_tensor (tensors, "token_embd.weight");
    VKLLAMA_STATUS_OK (embeddings);
    auto output_weight = find_tensor (tensors, "output.weight");
    VKLLAMA_STATUS_OK (output_weight);
    auto norm_weight = find_tensor (tensors, "output_norm.weight");
    VKLLAMA_STATUS_OK (norm_weight);
    auto vkembeddings
        = upload_tensor (gpu_, input_command_, *embeddings, false);
    VKLLAMA_STATUS_OK (vkembeddings);
    auto vkoutput_weight
        = upload_tensor (gpu_, output_command_, *output_weight, false);
    VKLLAMA_STATUS_OK (vkoutput_weight);
    auto vknorm_weight
        = upload_tensor (gpu_, input_command_, *norm_weight, true);
    VKLLAMA_STATUS_OK (vknorm_weight);
    vocab_ = vkembeddings->height ();
    dim_ = vkembeddings->width ();
    wtype_ = vkoutput_weight->dtype ();
    input_layer_ = new InputLayer (gpu_, input_command_, *vkembeddings, 0);
    output_layer_ = new OutputLayer (gpu_, output_command_, *vkoutput_weight,
                                     *vknorm_weight);
    VKLLAMA_STATUS_OK (input_layer_->init ());
    VKLLAMA_STATUS_OK (output_layer_->init ());
    VKLLAMA_STATUS_OK (input_command_->end ());
    VKLLAMA_STATUS_OK (output_command_->end ());
    VKLLAMA_STATUS_OK (input_command_->submit_and_wait ());
    VKLLAMA_STATUS_OK (output_command_->submit_and_wait ());
  }

  char vname[512];
  for (uint32_t b = 0; b < block_count; ++b)
    {
      auto get = [&] (const char *what) {
        ::snprintf (vname, sizeof (vname), "blk.%u.%s.weight", b, what);
        return find_tensor (tensors, vname);
      };
      auto command = new Command (gpu_);
      block_commands_.push_back (command);
      VKLLAMA_STATUS_OK (command->init ());
      VKLLAMA_STATUS_OK (command->begin ());

      Tensor w[9];
      const char *names[9]
          = { "attn_norm", "ffn_norm", "attn_k",   "attn_q",  "attn_v",
              "attn_output", "ffn_gate", "ffn_down", "ffn_up" };
      for (int i = 0; i < 9; ++i)
        {
          auto t = get (names[i]);
          VKLLAMA_STATUS_OK (t);
          auto up = upload_tensor (gpu_, command, *t, i < 2);
          VKLLAMA_STATUS_OK (up);
          w[i] = *up;
        }
      // head width = rows of Wk / head count (models/llama2.h:552,649)
      const auto dim = w[2].height () / head_count;
      if (dim == 0 || dim * head_count != w[2].height ())
        return absl::InvalidArgumentError (absl::StrFormat (
            "attention width %zu is not a multiple of %u heads",
            w[2].height (), head_count));
      heads_ = head_count;
      ffn_ = w[6].height ();
      Llama2Block::RmsNormParams rmsnorm_params = { w[0], w[1], norm_eps };
      Llama2Block::TransformerParams transformer_params
          = { w[2], w[3], w[4], w[5], (int)maxlen, (int)dim,
              b == (block_count - 1) };
      Llama2Block::FeedForwardParams feedfward_params
          = { w[6], w[7], w[8], norm_eps, false };
      auto *block = new Llama2Block (gpu_, command, transformer_params,
                                     feedfward_params, rmsnorm_params);
      blocks_.push_back (block);
      VKLLAMA_STATUS_OK (block->init ());
      VKLLAMA_STATUS_OK (command->end ());
      VKLLAMA_STATUS_OK (command->submit_and_wait ());
    }
  maxlen_ = maxlen;

  argmax_.reset (new ArgMax (gpu_, output_command_, FP16));
  VKLLAMA_STATUS_OK (argmax_->init ());
  plan_ = new DecodePlan ();
  VKLLAMA_STATUS_OK (plan_->build (*this, gpu_, input_layer_, blocks_,
                                   output_layer_, norm_eps));
  return absl::OkStatus ();
}

void
Model::set_decode_mode (int mode)
{
  if (plan_)
    plan_->set_mode (mode);
}

bool
Model::set_decode_option (const char *name, int value)
{
  return plan_ && plan_->set_option (name, value);
}

void
Model::set_operator_attention (bool on)
{
  for (auto *b : blocks_)
    b->attention ()->set_operator_attention (on);
}

void
Model::set_lastblock_rope_quirk (bool on)
{
  for (auto *b : blocks_)
    b->attention ()->set_lastblock_rope_quirk (on);
}

// One pass of the operator chain; returns the fp32 logits tensor [1, 1, V].
absl::StatusOr<Tensor>
Model::forward_ (std::vector<uint32_t> const &toks, const size_t offset)
{
  if (toks.empty ())
    return absl::InvalidArgumentError ("model called with no tokens");
  if (offset + toks.size () > maxlen_)
    return absl::OutOfRangeError (absl::StrFormat (
        "positions [%zu, %zu) exceed the context length %zu", offset,
        offset + toks.size (), maxlen_));
  if (vktoks_.width () != toks.size ())
    {
      // the previous buffer may still be read by queued work
      VKLLAMA_STATUS_OK (input_command_->wait ());
      vktoks_ = Tensor (1, 1, toks.size (), gpu_, UINT32, true);
      if (!vktoks_.create ().ok ())
        throw std::runtime_error ("failed at creating vktoks");
    }
  else
    {
      VKLLAMA_STATUS_OK (input_command_->wait ());
    }
  memcpy (vktoks_.host (), toks.data (), sizeof (uint32_t) * toks.size ());
  if (auto ret = vktoks_.flush (); !ret.ok ())
    throw std::runtime_error (ret.ToString ());

  VKLLAMA_STATUS_OK (input_command_->begin ());
  auto X = (*input_layer_) (vktoks_);
  VKLLAMA_STATUS_OK (X);
  VKLLAMA_STATUS_OK (input_command_->end ());
  VKLLAMA_STATUS_OK (input_command_->submit ());
  for (size_t i = 0; i < blocks_.size (); ++i)
    {
      auto *command = block_commands_[i];
      VKLLAMA_STATUS_OK (command->begin ());
      X = (*blocks_[i]) (*X, offset);
      if (!X.ok ())
        {
          fprintf (stderr, "infer block %zu failed: %s\n", i,
                   X.status ().message ().c_str ());
          return X.status ();
        }
      VKLLAMA_STATUS_OK (command->end ());
      VKLLAMA_STATUS_OK (command->submit ());
    }
  VKLLAMA_STATUS_OK (output_command_->begin ());
  return (*output_layer_) (*X);
}

absl::StatusOr<std::vector<float> >
Model::operator() (std::vector<uint32_t> const &toks, const size_t offset)
{
  if (!plan_)
    return absl::InternalError ("model used before init()");
  std::vector<float> buf_logits;
  if (fused_decode_ && toks.size () == 1 && plan_->usable ())
    {
      if (offset + 1 > maxlen_)
        return absl::OutOfRangeError (absl::StrFormat (
            "position %zu exceeds the context length %zu", offset, maxlen_));
      VKLLAMA_STATUS_OK (output_command_->wait ());
      VKLLAMA_STATUS_OK (plan_->step_host_token (toks[0], offset));
      buf_logits.resize (vocab_);
      auto rs = plan_->read_logits (buf_logits.data ());
      if (absl::IsUnavailable (rs))
        {
          // a wait between workgroups gave up; the plan has switched to the
          // launches that wait for nothing: the same step once more
          ++decode_recoveries_;
          VKLLAMA_STATUS_OK (plan_->step_host_token (toks[0], offset));
          rs = plan_->read_logits (buf_logits.data ());
        }
      VKLLAMA_STATUS_OK (rs);
      return buf_logits;
    }
  auto output = forward_ (toks, offset);
  VKLLAMA_STATUS_OK (output);
  buf_logits.resize (output->size ());
  VKLLAMA_STATUS_OK (output_command_->download (*output, buf_logits.data (),
                                                buf_logits.size ()));
  VKLLAMA_STATUS_OK (output_command_->end ());
  VKLLAMA_STATUS_OK (output_command_->submit ());
  VKLLAMA_STATUS_OK (input_command_->wait ());
  for (auto *c : block_commands_)
    VKLLAMA_STATUS_OK (c->wait ());
  VKLLAMA_STATUS_OK (output_command_->wait ());
#if __VKLLAMA_LOG_COST
  input_layer_->print_op_cost ();
  for (auto *b : blocks_)
    b->print_op_cost ();
  output_layer_->print_op_cost ();
#endif
  return buf_logits;
}

// the next token from the logits of the last pass: arg-max, or a draw from
// the top-k / top-p candidates with the uniform number of (seed, position)
absl::Status
Model::pick_token_ (uint32_t *dst, size_t position)
{
  if (!samp_on_)
    return plan_->argmax_logits (dst);
  return plan_->sample_logits (dst, samp_k_, samp_p_, samp_seed_,
                               (uint32_t)position);
}

absl::Status
Model::generate_sampled (std::vector<uint32_t> const &prompt, size_t n_gen,
                         int topk, float topp, uint64_t seed,
                         std::vector<uint32_t> &out, double *prefill_ms,
                         double *decode_ms)
{
  if (topp < 0.f && topk < 1)
    return absl::InvalidArgumentError ("top-k sampling needs k >= 1");
  if (topp > 1.f)
    return absl::InvalidArgumentError ("top-p sampling needs p in [0, 1]");
  samp_on_ = true, samp_k_ = topk, samp_p_ = topp, samp_seed_ = seed;
  auto s = generate_greedy (prompt, n_gen, out, prefill_ms, decode_ms);
  samp_on_ = false;
  return s;
}

absl::Status
Model::generate_greedy (std::vector<uint32_t> const &prompt, size_t n_gen,
                        std::vector<uint32_t> &out, double *prefill_ms,
                        double *decode_ms)
{
  auto s = generate_once_ (prompt, n_gen, out, prefill_ms, decode_ms);
  if (absl::IsUnavailable (s))
    {
      // a wait between workgroups gave up somewhere in the loop; the plan has
      // switched to the launches that wait for nothing.  The generation is
      // repeated from the prompt: KV rows written so far are rewritten with
      // the same values.
      ++decode_recoveries_;
      s = generate_once_ (prompt, n_gen, out, prefill_ms, decode_ms);
    }
  return s;
}

absl::Status
Model::generate_once_ (std::vector<uint32_t> const &prompt, size_t n_gen,
                       std::vector<uint32_t> &out, double *prefill_ms,
                       double *decode_ms)
{
  using clock = std::chrono::steady_clock;
  out.clear ();
  if (n_gen == 0)
    return absl::OkStatus ();
  if (prompt.empty ())
    return absl::InvalidArgumentError ("empty prompt");
  if (prompt.size () + n_gen - 1 > maxlen_)
    return absl::OutOfRangeError (absl::StrFormat (
        "prompt of %zu + %zu generated tokens exceed the context length %zu",
        prompt.size (), n_gen, maxlen_));
  if (!plan_)
    return absl::InternalError ("model used before init()");
  // generated ids stay in device memory between steps (the arg-max of step i
  // is the input token of step i + 1) and are copied out once at the end
  if (next_tok_.width () < n_gen)
    {
      VKLLAMA_STATUS_OK (output_command_->wait ());
      next_tok_ = Tensor (1, 1, n_gen, gpu_, UINT32, false);
      VKLLAMA_STATUS_OK (next_tok_.create ());
    }
  uint32_t *ids = (uint32_t *)next_tok_.data ();
  void *s = gpu_->stream ();

  const auto t0 = clock::now ();
  // prompt pass; arg-max of its fp16 logits becomes ids[0]
  if (fused_decode_ && prompt.size () == 1 && plan_->usable ())
    {
      VKLLAMA_STATUS_OK (plan_->step_host_token (prompt[0], 0));
    }
  else
    {
      auto logits32 = forward_ (prompt, 0);
      VKLLAMA_STATUS_OK (logits32);
      VKLLAMA_STATUS_OK (plan_->adopt_logits (*logits32));
    }
  VKLLAMA_STATUS_OK (pick_token_ (ids + 0, prompt.size ()));
  if (int e = vkl_stream_sync (s))
    return absl::InternalError (vkl_error_string (e));
  const auto t1 = clock::now ();
  size_t n_toks = prompt.size () + 1;
  size_t i0 = 1;
  if (fused_decode_ && plan_->usable () && decode_graph_ && n_gen > 1)
    {
      // ids[0] is at position prompt.size (); each replay appends one id
      if (samp_on_)
        {
          VKLLAMA_STATUS_OK (plan_->loop_sampled (ids, prompt.size (), n_gen - 1, samp_k_,
                                                  samp_p_, samp_seed_));
        }
      else
        {
          VKLLAMA_STATUS_OK (plan_->loop (ids, prompt.size (), n_gen - 1));
        }
      i0 = n_gen;
    }
  for (size_t i = i0; i < n_gen; ++i, ++n_toks)
    {
      if (fused_decode_ && plan_->usable ())
        {
          // the step's last launch reduces the arg-max partials into ids[i]
          VKLLAMA_STATUS_OK (plan_->step_device_token (
              ids + (i - 1), n_toks - 1, samp_on_ ? nullptr : ids + i));
          if (samp_on_)
            VKLLAMA_STATUS_OK (pick_token_ (ids + i, n_toks));
          continue;
        }
      else
        {
          uint32_t prev = 0;
          if (int e = vkl_memcpy_d2h (&prev, ids + (i - 1), sizeof (prev), s))
            return absl::InternalError (vkl_error_string (e));
          if (int e = vkl_stream_sync (s))
            return absl::InternalError (vkl_error_string (e));
          auto logits32 = forward_ ({ prev }, n_toks - 1);
          VKLLAMA_STATUS_OK (logits32);
          VKLLAMA_STATUS_OK (plan_->adopt_logits (*logits32));
        }
      VKLLAMA_STATUS_OK (pick_token_ (ids + i, n_toks));
    }
  if (int e = vkl_stream_sync (s))
    return absl::InternalError (vkl_error_string (e));
  const auto t2 = clock::now ();
  VKLLAMA_STATUS_OK (plan_->check ());
  // run deferred work the operator chain may have queued
  VKLLAMA_STATUS_OK (input_command_->wait ());
  for (auto *c : block_commands_)
    VKLLAMA_STATUS_OK (c->wait ());
  VKLLAMA_STATUS_OK (output_command_->wait ());
  out.resize (n_gen);
  if (int e = vkl_memcpy_d2h (out.data (), ids, n_gen * sizeof (uint32_t), s))
    return absl::InternalError (vkl_error_string (e));
  if (int e = vkl_stream_sync (s))
    return absl::InternalError (vkl_error_string (e));
  if (prefill_ms)
    *prefill_ms = std::chrono::duration<double, std::milli> (t1 - t0).count ();
  if (decode_ms)
    *decode_ms = std::chrono::duration<double, std::milli> (t2 - t1).count ();
  return absl::OkStatus ();
}

absl::Status
Model::read_kv_cache (size_t layer, bool value, std::vector<uint16_t> &out)
{
  if (layer >= blocks_.size ())
    return absl::OutOfRangeError ("no such layer");
  auto *attn = blocks_[layer]->attention ();
  Tensor &c = value ? attn->vcache () : attn->kcache ();
  out.resize (c.size ());
  VKLLAMA_STATUS_OK (output_command_->download (c, out.data (), out.size ()));
  return output_command_->wait ();
}

absl::Status
Model::write_kv_cache (size_t layer, bool value, const uint16_t *rows, size_t n)
{
  if (layer >= blocks_.size ())
    return absl::OutOfRangeError ("no such layer");
  auto *attn = blocks_[layer]->attention ();
  Tensor &c = value ? attn->vcache () : attn->kcache ();
  if (!rows || n != c.size ())
    return absl::InvalidArgumentError (absl::StrFormat (
        "a cache holds %zu values, %zu given", c.size (), n));
  VKLLAMA_STATUS_OK (output_command_->upload (rows, n, c));
  return output_command_->wait ();
}

size_t
Model::decode_step_bytes (size_t L) const
{
  // weights (34 B per 32 for Q8_0, 2 B each for FP16), fp32 norm weights, the
  // embedding row, K and V of L positions read, one position written
  const size_t per_layer = 4 * dim_ * dim_ + 3 * dim_ * ffn_;
  const size_t nw = blocks_.size () * per_layer + vocab_ * dim_;
  const size_t wbytes = wtype_ == Q8_0 ? nw / 32 * 34 : nw * 2;
  const size_t norm = (2 * blocks_.size () + 1) * dim_ * 4;
  const size_t emb = wtype_ == Q8_0 ? dim_ / 32 * 34 : dim_ * 2;
  const size_t kv = blocks_.size () * 2 * dim_ * 2;
  return wbytes + norm + emb + kv * L + kv;
}

size_t
Model::decode_phase_bytes (int kind, size_t L) const
{
  if (!plan_ || !plan_->usable ())
    return 0;
  return vkl_decode_phase_bytes (&plan_->desc (), kind, L);
}
}

namespace vkllama
{
absl::Status
Model::decode_phase_replay (int kind, size_t pos, int rounds, double *avg_ms,
                            uint64_t *launches)
{
  if (!plan_ || !plan_->usable ())
    return absl::FailedPreconditionError (
        "fused decode does not cover this model");
  const int e = vkl_decode_phase_replay (&plan_->desc (), kind, (uint32_t)pos,
                                         rounds, gpu_->stream (), avg_ms,
                                         launches);
  if (e)
    return absl::InternalError (
        absl::StrFormat ("phase replay failed: %s", vkl_error_string (e)));
  return absl::OkStatus ();
}
}
