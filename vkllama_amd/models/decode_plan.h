// DecodePlan: the device-pointer view of a loaded model that the fused
// one-token decode step (include/vkl_decode.h) consumes, plus the small state
// the greedy loop keeps on the device (current logits, token slot).
#ifndef __VKLLAMA_MODELS_DECODE_PLAN_H__
#define __VKLLAMA_MODELS_DECODE_PLAN_H__
#include "absl/status/status.h"
#include "src/core/tensor.h"
#include "vkl_decode.h"
#include <vector>

namespace vkllama
{
class GPUDevice;
class InputLayer;
class OutputLayer;
class Llama2Block;
class Model;

struct DecodePlan
{
  DecodePlan ();
  ~DecodePlan ();
  absl::Status build (Model &model, GPUDevice *gpu, InputLayer *in,
                      std::vector<Llama2Block *> &blocks, OutputLayer *out,
                      float eps);
  // true when the fused kernels cover this model (Q8_0, head width 64/128)
  bool usable () const { return usable_; }
  void set_mode (int mode) { mode_ = mode; }
  // options of this model's decode steps (fields of vkl_decode_model);
  // false for a name the plan does not know or a value out of range
  bool set_option (const char *name, int value);
  const vkl_decode_model &desc () const { return desc_; }
  // token id given by the host / read from device-visible memory
  absl::Status step_host_token (uint32_t tok, size_t offset);
  // next_tok (optional, device-visible): receives the arg-max id of this step
  absl::Status step_device_token (const uint32_t *tok, size_t offset,
                                  uint32_t *next_tok = nullptr);
  // n_steps greedy tokens replayed from a captured graph (vkl_decode_loop);
  // ids is device memory, ids[0] the first input token
  absl::Status loop (uint32_t *ids, size_t pos0, size_t n_steps);
  // the same with a draw from the top-k / top-p candidates instead of the
  // arg-max at the end of every replayed step (vkl_decode_loop_sampled)
  absl::Status loop_sampled (uint32_t *ids, size_t pos0, size_t n_steps, int topk,
                             float topp, uint64_t seed);
  int mode () const { return mode_; }
  // After the stream has been synchronised: did a wait between workgroups
  // inside a launch give up (vkl_decode_status)?  If so the plan switches to
  // the launches that wait for nothing (mode 0, attention and Wo apart) and
  // the status is Unavailable: the caller repeats the generation.
  absl::Status check ();
  // copies the fp32 logits of the last step (fused or adopted) to the host
  absl::Status read_logits (float *dst);
  // remember the fp32 logits tensor of an operator-chain pass
  absl::Status adopt_logits (Tensor logits32);
  // arg-max of the current logits into device-visible memory
  absl::Status argmax_logits (uint32_t *dst);
  // a token drawn from the current logits on the device (vkl_sample_f32):
  // topp < 0 keeps the topk largest logits, else the top-p set
  absl::Status sample_logits (uint32_t *dst, int topk, float topp,
                              uint64_t seed, uint32_t counter);

private:
  GPUDevice *gpu_;
  bool usable_;
  int mode_;
  vkl_decode_model desc_;
  Tensor layers_;   // device array of vkl_layer_weights
  std::vector<vkl_layer_weights> layers_h_; // host mirror
  Tensor scratch_;
  Tensor logits32_; // fp32 [vocab] written by the fused step
  Tensor tok_slot_; // pinned uint32
  Tensor adopted_;  // logits of the operator chain, if newer
  bool adopted_valid_;
  size_t vocab_;
};
}
#endif
