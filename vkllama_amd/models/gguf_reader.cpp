// A reader for GGUF files with the calling interface the reference's
// app/llama2_infer.cpp:46-75 uses from gguf-tools (gguf_open / gguf_get_key /
// gguf_get_tensor).  Written from the file format:
//   header   magic "GGUF" u32 | version u32 | tensor_count u64 | kv_count u64
//   kv       key string (u64 length + bytes) | value type u32 | value
//            string = u64 length + bytes; array = element type u32 + count u64
//            + elements; scalars little endian
//   tensor   name string | n_dims u32 | dims u64[n_dims] | ggml type u32 |
//            offset u64 (from the start of the data section)
//   data     starts at the next multiple of general.alignment (default 32)
#include "models/gguflib.h"
#include <fcntl.h>
#include <string.h>
#include <string>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <vector>

struct gguf_ctx
{
  int fd = -1;
  uint8_t *data = nullptr;
  size_t size = 0;
  uint32_t version = 0;
  uint64_t n_tensors = 0, n_kv = 0;
  std::vector<gguf_key> keys;
  std::vector<gguf_tensor> tensors;
  size_t next_key = 0, next_tensor = 0;
};

namespace
{
struct Cursor
{
  const uint8_t *base;
  size_t size, off;
  bool ok = true;

  bool
  need (size_t n)
  {
    if (!ok || n > size - off)
      ok = false;
    return ok;
  }

  template <typename T>
  T
  get ()
  {
    T v = T ();
    if (need (sizeof (T)))
      {
        memcpy (&v, base + off, sizeof (T));
        off += sizeof (T);
      }
    return v;
  }

  // a GGUF string: returns the pointer to its bytes
  const char *
  str (uint64_t &len)
  {
    len = get<uint64_t> ();
    if (!need (len))
      return nullptr;
    const char *p = (const char *)(base + off);
    off += len;
    return p;
  }
};

size_t
scalar_bytes (uint32_t type)
{
  switch (type)
    {
    case GGUF_VALUE_TYPE_UINT8:
    case GGUF_VALUE_TYPE_INT8:
    case GGUF_VALUE_TYPE_BOOL: return 1;
    case GGUF_VALUE_TYPE_UINT16:
    case GGUF_VALUE_TYPE_INT16: return 2;
    case GGUF_VALUE_TYPE_UINT32:
    case GGUF_VALUE_TYPE_INT32:
    case GGUF_VALUE_TYPE_FLOAT32: return 4;
    case GGUF_VALUE_TYPE_UINT64:
    case GGUF_VALUE_TYPE_INT64:
    case GGUF_VALUE_TYPE_FLOAT64: return 8;
    default: return 0;
    }
}

// advances past one value of the given type
void
skip_value (Cursor &c, uint32_t type, int depth = 0)
{
  if (type == GGUF_VALUE_TYPE_STRING)
    {
      uint64_t n;
      c.str (n);
    }
  else if (type == GGUF_VALUE_TYPE_ARRAY)
    {
      const uint32_t et = c.get<uint32_t> ();
      const uint64_t n = c.get<uint64_t> ();
      if (depth > 4 || (et > GGUF_VALUE_TYPE_FLOAT64))
        {
          c.ok = false;
          return;
        }
      const size_t sb = scalar_bytes (et);
      if (sb)
        {
          if (n > (c.size - c.off) / sb)
            c.ok = false;
          else
            c.off += n * sb;
        }
      else
        for (uint64_t i = 0; i < n && c.ok; ++i)
          skip_value (c, et, depth + 1);
    }
  else
    {
      const size_t sb = scalar_bytes (type);
      if (!sb || !c.need (sb))
        c.ok = false;
      else
        c.off += sb;
    }
}

// bytes of a tensor of `n` weights: F32, F16, Q8_0 (34 bytes per 32 weights
// of a row; rows are whole blocks), 0 for types this build does not read
uint64_t
tensor_bytes (uint32_t type, const uint64_t *dim, uint32_t ndim)
{
  uint64_t rows = 1;
  for (uint32_t i = 1; i < ndim; ++i)
    rows *= dim[i];
  const uint64_t cols = ndim ? dim[0] : 0;
  switch (type)
    {
    case GGUF_TYPE_F32: return rows * cols * 4;
    case GGUF_TYPE_F16: return rows * cols * 2;
    case GGUF_TYPE_Q8_0: return rows * ((cols + 31) / 32) * 34;
    default: return 0;
    }
}

bool
parse (gguf_ctx *ctx)
{
  Cursor c{ ctx->data, ctx->size, 0 };
  if (c.get<uint32_t> () != 0x46554747u) // "GGUF"
    return false;
  ctx->version = c.get<uint32_t> ();
  if (ctx->version < 2 || ctx->version > 3)
    return false;
  ctx->n_tensors = c.get<uint64_t> ();
  ctx->n_kv = c.get<uint64_t> ();
  if (!c.ok || ctx->n_kv > (1u << 24) || ctx->n_tensors > (1u << 24))
    return false;
  uint64_t alignment = 32;
  for (uint64_t i = 0; i < ctx->n_kv; ++i)
    {
      gguf_key k = {};
      uint64_t len;
      k.name = c.str (len);
      k.namelen = len;
      k.type = c.get<uint32_t> ();
      if (!c.ok)
        return false;
      k.val = (union gguf_value *)(ctx->data + c.off);
      if (k.type == GGUF_VALUE_TYPE_UINT32 && len == 17
          && !memcmp (k.name, "general.alignment", 17) && c.need (4))
        alignment = k.val->uint32;
      skip_value (c, k.type);
      if (!c.ok)
        return false;
      ctx->keys.push_back (k);
    }
  if (alignment == 0 || (alignment & (alignment - 1)))
    return false;
  for (uint64_t i = 0; i < ctx->n_tensors; ++i)
    {
      gguf_tensor t = {};
      uint64_t len;
      t.name = c.str (len);
      t.namelen = len;
      t.ndim = c.get<uint32_t> ();
      if (!c.ok || t.ndim > GGUF_TENSOR_MAX_DIM)
        return false;
      t.num_weights = 1;
      for (uint32_t d = 0; d < GGUF_TENSOR_MAX_DIM; ++d)
        t.dim[d] = 1;
      for (uint32_t d = 0; d < t.ndim; ++d)
        {
          t.dim[d] = c.get<uint64_t> ();
          t.num_weights *= t.dim[d];
        }
      t.type = c.get<uint32_t> ();
      t.offset = c.get<uint64_t> ();
      if (!c.ok)
        return false;
      t.bsize = tensor_bytes (t.type, t.dim, t.ndim);
      ctx->tensors.push_back (t);
    }
  const uint64_t data_start = (c.off + alignment - 1) / alignment * alignment;
  for (gguf_tensor &t : ctx->tensors)
    {
      const uint64_t begin = data_start + t.offset;
      if (begin > ctx->size || t.bsize > ctx->size - begin)
        return false; // tensor data runs past the end of the file
      t.offset = begin;
      t.weights_data = ctx->data + begin;
    }
  return true;
}
}

extern "C" gguf_ctx *
gguf_open (const char *filename)
{
  if (!filename)
    return nullptr;
  gguf_ctx *ctx = new gguf_ctx ();
  ctx->fd = open (filename, O_RDONLY);
  struct stat st;
  if (ctx->fd < 0 || fstat (ctx->fd, &st) != 0 || st.st_size < 24)
    {
      gguf_close (ctx);
      return nullptr;
    }
  ctx->size = (size_t)st.st_size;
  void *m = mmap (nullptr, ctx->size, PROT_READ, MAP_PRIVATE, ctx->fd, 0);
  if (m == MAP_FAILED)
    {
      gguf_close (ctx);
      return nullptr;
    }
  ctx->data = (uint8_t *)m;
  if (!parse (ctx))
    {
      gguf_close (ctx);
      return nullptr;
    }
  return ctx;
}

extern "C" void
gguf_close (gguf_ctx *ctx)
{
  if (!ctx)
    return;
  if (ctx->data)
    munmap (ctx->data, ctx->size);
  if (ctx->fd >= 0)
    close (ctx->fd);
  delete ctx;
}

extern "C" void
gguf_rewind (gguf_ctx *ctx)
{
  if (ctx)
    ctx->next_key = ctx->next_tensor = 0;
}

extern "C" int
gguf_get_key (gguf_ctx *ctx, gguf_key *key)
{
  if (!ctx || !key || ctx->next_key >= ctx->keys.size ())
    return 0;
  *key = ctx->keys[ctx->next_key++];
  return 1;
}

extern "C" int
gguf_get_tensor (gguf_ctx *ctx, gguf_tensor *tensor)
{
  if (!ctx || !tensor)
    return 0;
  ctx->next_key = ctx->keys.size ();
  if (ctx->next_tensor >= ctx->tensors.size ())
    return 0;
  *tensor = ctx->tensors[ctx->next_tensor++];
  return 1;
}

extern "C" const char *
gguf_get_value_type_name (uint32_t type)
{
  static const char *names[] = { "uint8",  "int8",   "uint16", "int16", "uint32",
                                 "int32",  "float32", "bool",  "string", "array",
                                 "uint64", "int64",  "float64" };
  return type <= GGUF_VALUE_TYPE_FLOAT64 ? names[type] : "unknown";
}

extern "C" const char *
gguf_get_tensor_type_name (uint32_t type)
{
  switch (type)
    {
    case GGUF_TYPE_F32: return "f32";
    case GGUF_TYPE_F16: return "f16";
    case GGUF_TYPE_Q8_0: return "q8_0";
    default: return "unsupported";
    }
}

extern "C" uint32_t
gguf_version (const gguf_ctx *ctx)
{
  return ctx ? ctx->version : 0;
}

extern "C" uint64_t
gguf_tensor_count (const gguf_ctx *ctx)
{
  return ctx ? ctx->tensors.size () : 0;
}

extern "C" uint64_t
gguf_key_count (const gguf_ctx *ctx)
{
  return ctx ? ctx->keys.size () : 0;
}
