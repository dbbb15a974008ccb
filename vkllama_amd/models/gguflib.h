/* Layout-compatible declarations of the two structures of antirez/gguf-tools'
 * gguflib.h that the model loader reads (the reference's models/llama2.h
 * takes std::map<std::string, gguf_key> and std::map<std::string,
 * gguf_tensor>).  Only the fields the loader touches are used here:
 * gguf_key::val->uint32 / float32 and gguf_tensor::type, dim[0..1],
 * weights_data, bsize.  If the real gguflib.h is on the include path first,
 * define VKLLAMA_HAVE_GGUFLIB to skip these. */
#ifndef VKLLAMA_GGUFLIB_COMPAT_H
#define VKLLAMA_GGUFLIB_COMPAT_H
#ifndef VKLLAMA_HAVE_GGUFLIB
#include <stddef.h>
#include <stdint.h>

#define GGUF_TENSOR_MAX_DIM 8

enum gguf_tensor_type
{
  GGUF_TYPE_F32 = 0,
  GGUF_TYPE_F16 = 1,
  GGUF_TYPE_Q8_0 = 8,
};

union gguf_value
{
  uint8_t uint8;
  int8_t int8;
  uint16_t uint16;
  int16_t int16;
  uint32_t uint32;
  int32_t int32;
  float float32;
  uint64_t uint64;
  int64_t int64;
  double float64;
  uint8_t boolval;
  struct
  {
    uint32_t type;
    uint64_t len;
  } __attribute__ ((packed)) array;
} __attribute__ ((packed));

typedef struct
{
  const char *name;
  size_t namelen;
  uint32_t type;
  union gguf_value *val;
} gguf_key;

typedef struct
{
  const char *name;
  size_t namelen;
  uint32_t type;
  uint32_t ndim;
  uint64_t dim[GGUF_TENSOR_MAX_DIM];
  uint64_t offset;
  uint64_t bsize;
  uint64_t num_weights;
  uint8_t *weights_data;
} gguf_tensor;
#endif
#endif
