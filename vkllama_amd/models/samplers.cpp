#include "samplers.h"
#include <algorithm>
#include <cmath>
#include <numeric>

namespace
{
// larger logit first; equal logits: lower token id first
bool
before (const Sampler::Candidate &a, const Sampler::Candidate &b)
{
  return a.first > b.first || (a.first == b.first && a.second < b.second);
}
}

Sampler::Sampler () : g_ (std::random_device () ()) {}
Sampler::Sampler (uint64_t s) : g_ ((std::mt19937::result_type)s) {}

void
Sampler::seed (uint64_t s)
{
  g_.seed ((std::mt19937::result_type)s);
}

size_t
Sampler::sample_from_prob (const float *probs, size_t n)
{
  std::discrete_distribution<size_t> dist (probs, probs + n);
  return dist (g_);
}

void
Sampler::softmax (std::vector<Candidate> &v)
{
  if (v.empty ())
    return;
  const float top = v[0].first;
  float total = 0.f;
  for (auto &c : v)
    {
      c.first = std::exp (c.first - top);
      total += c.first;
    }
  for (auto &c : v)
    c.first /= total;
}

std::vector<Sampler::Candidate>
Sampler::ranked (const float *logits, size_t n, size_t keep)
{
  std::vector<Candidate> all (n);
  for (size_t i = 0; i < n; ++i)
    all[i] = Candidate (logits[i], (int)i);
  keep = std::min (keep, n);
  // only the kept prefix has to be in order: for a small top-k this is far
  // cheaper than sorting the whole vocabulary for every token
  std::partial_sort (all.begin (), all.begin () + keep, all.end (), before);
  return all;
}

int
Sampler::draw ()
{
  std::vector<float> probs (cand_.size ());
  std::transform (cand_.begin (), cand_.end (), probs.begin (),
                  [] (const Candidate &c) { return c.first; });
  return cand_[sample_from_prob (probs.data (), probs.size ())].second;
}

TopkSampler::TopkSampler (size_t topk) : topk_ (topk) {}
TopkSampler::TopkSampler (size_t topk, uint64_t s) : Sampler (s), topk_ (topk) {}

int
TopkSampler::sample (const float *logits, size_t n)
{
  if (n == 0)
    return -1;
  // the reference resizes to topk even beyond n; here the vocabulary bounds it
  const size_t k = std::max<size_t> (1, std::min (topk_, n));
  cand_ = ranked (logits, n, k);
  cand_.resize (k);
  softmax (cand_);
  return k == 1 ? cand_[0].second : draw ();
}

TopPSampler::TopPSampler (const float p) : p_ (p) {}
TopPSampler::TopPSampler (const float p, uint64_t s) : Sampler (s), p_ (p) {}

int
TopPSampler::sample (const float *logits, size_t n)
{
  if (n == 0)
    return -1;
  std::vector<Candidate> all = ranked (logits, n, n);
  std::vector<Candidate> probs (all);
  softmax (probs);
  cand_.clear ();
  float mass = 0.f;
  for (size_t i = 0; i < n && mass < p_; ++i)
    {
      cand_.push_back (all[i]);
      mass += probs[i].first;
    }
  if (cand_.empty ()) // p <= 0: the most likely token alone
    cand_.push_back (all[0]);
  softmax (cand_);
  return draw ();
}
