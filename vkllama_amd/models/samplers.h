// Host samplers over one row of logits: the interface of the reference's
// models/samplers.h:8-43 (Sampler, TopkSampler, TopPSampler; sample(logits, n)
// returns a token id).  Differences, all additive: a sampler can be seeded
// (the reference seeds from std::random_device only), exposes the candidate
// set of its last call, and breaks ties between equal logits toward the
// lower token id (the reference leaves that to std::sort).
#ifndef __VKLLAMA_SAMPLERS_H__
#define __VKLLAMA_SAMPLERS_H__
#include <cstddef>
#include <cstdint>
#include <random>
#include <utility>
#include <vector>

class Sampler
{
public:
  typedef std::pair<float, int> Candidate; // (logit, then probability; token id)

  Sampler ();                        // seeded from std::random_device
  explicit Sampler (uint64_t seed);
  virtual ~Sampler () = default;
  virtual int sample (const float *logits, size_t n) = 0;
  void seed (uint64_t s);
  // candidates of the last sample() call, most likely first, with their
  // probabilities after renormalisation
  const std::vector<Candidate> &candidates () const { return cand_; }

protected:
  // index drawn from a discrete distribution proportional to probs[0..n)
  size_t sample_from_prob (const float *probs, size_t n);
  // in place: first -> exp(first - v[0].first) / sum; v[0] must hold the
  // largest logit (models/samplers.cpp:17-35)
  static void softmax (std::vector<Candidate> &v);
  // all (logit, id) pairs with the `keep` largest logits first, in order
  static std::vector<Candidate> ranked (const float *logits, size_t n, size_t keep);
  int draw ();
  std::vector<Candidate> cand_;

private:
  std::mt19937 g_;
};

// keeps the topk largest logits, softmax over them, draws one
// (models/samplers.cpp:37-64); topk = 1 is the greedy pick
class TopkSampler : public Sampler
{
public:
  TopkSampler (size_t topk = 40);
  TopkSampler (size_t topk, uint64_t seed);
  int sample (const float *logits, size_t n) override;

private:
  size_t topk_;
};

// keeps the most likely tokens until their probability mass reaches p,
// softmax over the kept logits, draws one (models/samplers.cpp:66-101)
class TopPSampler : public Sampler
{
public:
  TopPSampler (const float p);
  TopPSampler (const float p, uint64_t seed);
  int sample (const float *logits, size_t n) override;

private:
  const float p_;
};

#endif
