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

/* GGUF metadata value types (the file format's numbering) */
enum gguf_value_type
{
  GGUF_VALUE_TYPE_UINT8 = 0,
  GGUF_VALUE_TYPE_INT8 = 1,
  GGUF_VALUE_TYPE_UINT16 = 2,
  GGUF_VALUE_TYPE_INT16 = 3,
  GGUF_VALUE_TYPE_UINT32 = 4,
  GGUF_VALUE_TYPE_INT32 = 5,
  GGUF_VALUE_TYPE_FLOAT32 = 6,
  GGUF_VALUE_TYPE_BOOL = 7,
  GGUF_VALUE_TYPE_STRING = 8,
  GGUF_VALUE_TYPE_ARRAY = 9,
  GGUF_VALUE_TYPE_UINT64 = 10,
  GGUF_VALUE_TYPE_INT64 = 11,
  GGUF_VALUE_TYPE_FLOAT64 = 12,
};

/* The part of gguf-tools' reader interface that app/llama2_infer.cpp:46-75 of
 * the reference uses, implemented in models/gguf_reader.cpp from the GGUF
 * file format (versions 2 and 3, little endian): the file is mapped read-only
 * and keys / tensors are handed out in file order; names and values point
 * into the mapping and stay valid until gguf_close. */
typedef struct gguf_ctx gguf_ctx;
#ifdef __cplusplus
extern "C" {
#endif
gguf_ctx *gguf_open (const char *filename);
void gguf_close (gguf_ctx *ctx);
void gguf_rewind (gguf_ctx *ctx);
/* 1 and *key filled while keys remain, then 0 */
int gguf_get_key (gguf_ctx *ctx, gguf_key *key);
/* 1 and *tensor filled while tensors remain, then 0; all keys are skipped
 * first if the caller has not read them */
int gguf_get_tensor (gguf_ctx *ctx, gguf_tensor *tensor);
const char *gguf_get_value_type_name (uint32_t type);
const char *gguf_get_tensor_type_name (uint32_t type);
uint32_t gguf_version (const gguf_ctx *ctx);
uint64_t gguf_tensor_count (const gguf_ctx *ctx);
uint64_t gguf_key_count (const gguf_ctx *ctx);
#ifdef __cplusplus
}
#endif
#endif
#endif
