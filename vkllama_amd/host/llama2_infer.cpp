// Command-line greedy generation from a GGUF file with the drop-in classes:
// the flow of the reference's app/llama2_infer.cpp (open the file, collect
// keys and tensors, Model::init, prompt pass, then one token per step with a
// top-1 pick on the host) without the sentencepiece tokenizer, which is not
// available to C++ in this image: the prompt is given as token ids.
//
//   llama2_infer MODEL.gguf N_TOKENS ID [ID ...]
#include "models/gguflib.h"
#include "models/llama2.h"
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
  if (argc < 4)
    {
      fprintf (stderr, "usage: %s <model.gguf> <predict tokens> <prompt id> [id ...]\n", argv[0]);
      return 2;
    }
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
      // top-1 over the last row of logits; the lowest index wins ties
      const size_t V = model.vocab_size ();
      const float *row = logits->data () + (logits->size () - V);
      const uint32_t next = (uint32_t)(std::max_element (row, row + V) - row);
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
