// Command-line generation from a GGUF file with the drop-in classes: the flow
// of the reference's app/llama2_infer.cpp (open the file, collect keys and
// tensors, Model::init, prompt pass, then one token per step picked on the
// host by a TopkSampler(1), line 138 there) without the sentencepiece
// tokenizer, which is not available to C++ in this image: the prompt is given
// as token ids.
//
//   llama2_infer [--topk K | --topp P] [--seed S] MODEL.gguf N_TOKENS ID [ID ...]
#include "models/gguflib.h"
#include "models/llama2.h"
#include "models/samplers.h"
#include <cstring>
#include <memory>
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <string>
#include <vector>

int
main (int argc, char **argv)
{
  size_t topk = 1;
  float topp = -1.f;
  bool seeded = false;
  uint64_t seed = 0;
  while (argc > 2 && argv[1][0] == '-' && argv[1][1] == '-')
    {
      if (!strcmp (argv[1], "--topk"))
        topk = (size_t)strtoul (argv[2], nullptr, 10);
      else if (!strcmp (argv[1], "--topp"))
        topp = strtof (argv[2], nullptr);
      else if (!strcmp (argv[1], "--seed"))
        seeded = true, seed = strtoull (argv[2], nullptr, 10);
      else
        break;
      argv += 2, argc -= 2;
    }
  if (argc < 4 || topk < 1)
    {
      fprintf (stderr,
               "usage: llama2_infer [--topk K | --topp P] [--seed S] <model.gguf> <predict tokens> "
               "<prompt id> [id ...]\n");
      return 2;
    }
  std::unique_ptr<Sampler> sampler;
  if (topp >= 0.f)
    sampler.reset (seeded ? new TopPSampler (topp, seed) : new TopPSampler (topp));
  else
    sampler.reset (seeded ? new TopkSampler (topk, seed) : new TopkSampler (topk));
  gguf_ctx *gguf = gguf_open (argv[1]);
  if (!gguf)
    {
      fprintf (stderr, "cannot read %s as a GGUF file\n", argv[1]);
      return 1;
    }
  std::map<std::string, gguf_key> kv;
  gguf_key key;
  while (gguf_get_key (gguf, &key))
    {
      fprintf (stderr, "%.*s: [%s]\n", (int)key.namelen, key.name,
               gguf_get_value_type_name (key.type));
      kv[std::string (key.name, key.namelen)] = key;
    }
  std::map<std::string, gguf_tensor> tensors;
  gguf_tensor tensor;
  while (gguf_get_tensor (gguf, &tensor))
    tensors[std::string (tensor.name, tensor.namelen)] = tensor;

  const int predict = atoi (argv[2]);
  std::vector<uint32_t> prompt;
  for (int i = 3; i < argc; ++i)
    prompt.push_back ((uint32_t)strtoul (argv[i], nullptr, 10));

  vkllama::Model model (0);
  auto ret = model.init (kv, tensors);
  gguf_close (gguf);
  if (!ret.ok ())
    {
      fprintf (stderr, "failed at init model: %s\n", ret.ToString ().c_str ());
      return 1;
    }
  fprintf (stderr, "all weights are uploaded to device\n");

  using clock = std::chrono::steady_clock;
  std::vector<uint32_t> toks = prompt;
  size_t offset = 0;
  const auto t0 = clock::now ();
  auto t1 = t0;
  for (int i = 0; i < predict; ++i)
    {
      auto logits = model (toks, offset);
      if (!logits.ok ())
        {
          fprintf (stderr, "failed at inferring: %s\n", logits.status ().ToString ().c_str ());
          return 1;
        }
      if (i == 0)
        t1 = clock::now ();
      // the sampler sees the last row of logits (top-1 by default; the
      // lowest index wins ties)
      const size_t V = model.vocab_size ();
      const float *row = logits->data () + (logits->size () - V);
      const uint32_t next = (uint32_t)sampler->sample (row, V);
      printf ("%u%c", next, i + 1 == predict ? '\n' : ' ');
      offset += toks.size ();
      toks = { next };
    }
  const auto t2 = clock::now ();
  fprintf (stderr, "prompt %zu tokens %.1f ms; %d tokens %.1f ms\n", prompt.size (),
           std::chrono::duration<double, std::milli> (t1 - t0).count (), predict - 1,
           std::chrono::duration<double, std::milli> (t2 - t1).count ());
  return 0;
}
