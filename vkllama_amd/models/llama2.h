// Llama-2 token loop: public interface of the reference's models/llama2.h
// (InputLayer :36-79, Llama2Block :81-253, OutputLayer :255-320,
// Model :322-854).  Model::init takes the GGUF key/tensor maps, uploads the
// weights, and builds one operator chain per block; Model::operator() runs one
// forward pass over `toks` at KV-cache position `offset` and returns the fp32
// logits of the last row.
//
// Additions over the reference (all optional):
//  - a forward pass over ONE token runs the fused decode kernels
//    (set_fused_decode(false) forces the operator chain);
//  - generate_greedy() keeps the sampled token on the device (arg-max over
//    the logits, lowest index on ties) so that a decode loop needs no
//    128 KB logits download per token;
//  - set_lastblock_rope_quirk(false) rotates the last block's clipped query
//    at its true position instead of the reference's `offset`;
//  - set_operator_attention(true) runs the attention of a prompt pass as the
//    reference's three operators with their rounding points.
#ifndef __VKLLAMA_MODELS_LLAMA2_H__
#define __VKLLAMA_MODELS_LLAMA2_H__
// clang-format off
#include <stddef.h>
extern "C"{
#include "gguflib.h"
}
// clang-format on
#include "absl/status/statusor.h"
#include "src/core/command.h"
#include "src/core/common.h"
#include "src/core/tensor.h"
#include "src/ops/argop.h"
#include "src/ops/cast.h"
#include "src/ops/elementwise.h"
#include "src/ops/embedding.h"
#include "src/ops/feed_forward.h"
#include "src/ops/multiheadattention_v2.h"
#include "src/ops/rms_norm.h"
#include "src/ops/slice.h"
#include <map>
#include <memory>
#include <string>
#include <vector>

namespace vkllama
{
class InputLayer
{
public:
  InputLayer (GPUDevice *gpu, Command *command, Tensor vocab, uint32_t UNK = 0);
  absl::Status init ();
  absl::StatusOr<Tensor> operator() (Tensor toks);
  void print_op_cost ();
  Embedding *embedding () { return embedding_op_.get (); }

private:
  GPUDevice *gpu_;
  Command *command_;
  Tensor vocab_;
  uint32_t UNK_;
  std::unique_ptr<Embedding> embedding_op_;
};

class Llama2Block
{
public:
  struct TransformerParams
  {
    Tensor Wk;
    Tensor Wq;
    Tensor Wv;
    Tensor Wo;
    int maxlen;
    int dim;
    bool clip_output;
  };

  struct FeedForwardParams
  {
    Tensor w1;
    Tensor w2;
    Tensor w3;
    float eps;
    bool clip_output;
  };

  struct RmsNormParams
  {
    Tensor weight1;
    Tensor weight2;
    float eps;
  };

  Llama2Block (GPUDevice *dev, Command *command,
               TransformerParams const &transformer,
               FeedForwardParams const &feed_forward,
               RmsNormParams const &norm);
  absl::Status init ();
  absl::StatusOr<Tensor> operator() (Tensor in, const size_t offset);
  void print_op_cost ();

  MultiHeadAttentionV2 *attention () { return attn_op_.get (); }
  FeedForward *feed_forward () { return feedforward_op_.get (); }
  RMSNorm *attn_norm () { return norm_op_.get (); }
  RMSNorm *ffn_norm () { return norm_op2_.get (); }

private:
  GPUDevice *gpu_;
  Command *command_;
  std::unique_ptr<MultiHeadAttentionV2> attn_op_;
  std::unique_ptr<FeedForward> feedforward_op_;
  std::unique_ptr<RMSNorm> norm_op_;
  std::unique_ptr<RMSNorm> norm_op2_;
  std::unique_ptr<ElementWise> add_op_;
  std::unique_ptr<ElementWise> add_op2_;
  std::unique_ptr<Slice> slice_op_;

  TransformerParams transformer_params_;
  FeedForwardParams feedforward_params_;
  RmsNormParams rmsnorm_params_;
};

class OutputLayer
{
public:
  OutputLayer (GPUDevice *gpu, Command *command, Tensor wo,
               Tensor norm_weight);
  absl::Status init ();
  absl::StatusOr<Tensor> operator() (Tensor in);
  void print_op_cost ();
  Tensor &weight () { return wo_; }
  RMSNorm *norm () { return norm_op_.get (); }

private:
  GPUDevice *gpu_;
  Command *command_;
  Tensor wo_;
  Tensor norm_weight_;
  std::unique_ptr<MatMul> matmul_op_;
  std::unique_ptr<RMSNorm> norm_op_;
  std::unique_ptr<ArgMax> argmax_op_;
  std::unique_ptr<Cast> cast_op_;
};

struct DecodePlan; // device pointers of the fused one-token path

class Model
{
public:
  Model (int dev = 0);
  ~Model ();
  Model (const Model &) = delete;
  Model &operator= (const Model &) = delete;

  absl::Status init (std::map<std::string, gguf_key> &kv,
                     std::map<std::string, gguf_tensor> &tensors);

  absl::StatusOr<std::vector<float> >
  operator() (std::vector<uint32_t> const &toks, const size_t offset);

  // ---- additions -----------------------------------------------------------
  void set_fused_decode (bool on) { fused_decode_ = on; }
  void set_lastblock_rope_quirk (bool on);
  // prompt pass: attention as the reference's three operators (see
  // MultiHeadAttentionV2::set_operator_attention)
  void set_operator_attention (bool on);
  // 0 = one launch per decode phase, 1 = one launch per layer
  void set_decode_mode (int mode);
  // options of the fused decode steps: "attn_split_min", "fuse_attn_wo",
  // "wait_test" (DecodePlan::set_option)
  bool set_decode_option (const char *name, int value);
  // greedy loop replayed from a captured HIP graph (default) or launched
  // step by step
  void set_decode_graph (bool on) { decode_graph_ = on; }
  // Greedy loop of app/llama2_infer.cpp:140-218: prompt at offset 0, then one
  // token at a time at offset toks.size()-1; n_gen ids are written to out.
  // The wall-clock times of the two phases are returned in milliseconds.
  absl::Status generate_greedy (std::vector<uint32_t> const &prompt,
                                size_t n_gen, std::vector<uint32_t> &out,
                                double *prefill_ms = nullptr,
                                double *decode_ms = nullptr);
  // The same loop with the token drawn on the device from the top-k
  // (topp < 0) or top-p candidates of every step's logits
  // (models/samplers.cpp:37-101 as a kernel): logits never leave the device.
  // The draw at position pos uses the uniform number of (seed, pos).
  absl::Status generate_sampled (std::vector<uint32_t> const &prompt,
                                 size_t n_gen, int topk, float topp,
                                 uint64_t seed, std::vector<uint32_t> &out,
                                 double *prefill_ms = nullptr,
                                 double *decode_ms = nullptr);
  // copies one layer's K or V cache, [heads, maxlen, head_dim] fp16 bits
  absl::Status read_kv_cache (size_t layer, bool value,
                              std::vector<uint16_t> &out);
  // A testing aid, the mirror of read_kv_cache: replaces one layer's K or V
  // cache with n = heads * maxlen * head_dim fp16 values, so that a test can
  // put a model at a late position without running the prompt that leads
  // there (the reference fills its caches only through
  // src/ops/update_kv_cache.cpp).
  absl::Status write_kv_cache (size_t layer, bool value, const uint16_t *rows,
                               size_t n);
  GPUDevice *device () { return gpu_; }
  size_t vocab_size () const { return vocab_; }
  size_t context_length () const { return maxlen_; }
  size_t block_count () const { return blocks_.size (); }
  // algorithmic bytes one decode step at context length L reads and writes
  size_t decode_step_bytes (size_t L) const;
  // algorithmic bytes of one launch of a decode phase (see vkl_decode.h)
  size_t decode_phase_bytes (int kind, size_t L) const;
  absl::Status decode_phase_replay (int kind, size_t pos, int rounds,
                                    double *avg_ms, uint64_t *launches);
  // how often a decode step or generation was repeated because a wait between
  // workgroups inside a launch had given up (DecodePlan::check)
  size_t decode_recoveries () const { return decode_recoveries_; }

private:
  absl::StatusOr<Tensor> forward_ (std::vector<uint32_t> const &toks,
                                   const size_t offset);
  int dev_;
  GPUDevice *gpu_;
  Command *input_command_;
  std::vector<Command *> block_commands_;
  Command *output_command_;
  InputLayer *input_layer_;
  OutputLayer *output_layer_;
  std::vector<Llama2Block *> blocks_;
  size_t vocab_, dim_, ffn_, heads_, maxlen_;
  DType wtype_;
  bool fused_decode_;
  Tensor vktoks_;
  Tensor next_tok_;
  std::unique_ptr<ArgMax> argmax_;
  DecodePlan *plan_;
  bool decode_graph_ = true;
  // sampling on the device during generate_*(): off = arg-max
  bool samp_on_ = false;
  int samp_k_ = 1;
  float samp_p_ = -1.f;
  uint64_t samp_seed_ = 0;
  size_t decode_recoveries_ = 0;
  absl::Status pick_token_ (uint32_t *dst, size_t position);
  absl::Status generate_once_ (std::vector<uint32_t> const &prompt, size_t n_gen,
                               std::vector<uint32_t> &out, double *prefill_ms,
                               double *decode_ms);
};

}

#endif
