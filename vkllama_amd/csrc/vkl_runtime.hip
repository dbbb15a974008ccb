// Device, stream, memory and event entry points of the C ABI (include/vkl_hip.h).
#include "../../include/vkl_hip.h"
#include "vkl_common.h"
#include "vkl_gemm.h"
#include <string.h>

extern "C" {

int
vkl_device_count (int *n)
{
  VKL_CHECK_ARG (n != nullptr);
  VKL_HIP (hipGetDeviceCount (n));
  return 0;
}

int
vkl_device_open (int dev, vkl_device_info *info)
{
  int n = 0;
  VKL_HIP (hipGetDeviceCount (&n));
  VKL_CHECK_ARG (dev >= 0 && dev < n);
  VKL_HIP (hipSetDevice (dev));
  // this device's copy of the static scratch array (vkl_matmul_q8_0_noalloc)
  // is looked up here, once, with the device current
  (void)vkl::gemm_static_scratch (nullptr);
  if (info)
    {
      hipDeviceProp_t p;
      VKL_HIP (hipGetDeviceProperties (&p, dev));
      memset (info, 0, sizeof (*info));
      info->device = dev;
      info->compute_units = p.multiProcessorCount;
      info->wavefront_size = p.warpSize;
      info->max_lds_bytes = (int)p.sharedMemPerBlock;
      info->total_mem = p.totalGlobalMem;
      strncpy (info->name, p.name, sizeof (info->name) - 1);
      strncpy (info->arch, p.gcnArchName, sizeof (info->arch) - 1);
    }
  return 0;
}

const char *
vkl_error_string (int err)
{
  return hipGetErrorString ((hipError_t)err);
}

int
vkl_stream_create (void **stream)
{
  VKL_CHECK_ARG (stream != nullptr);
  hipStream_t s;
  VKL_HIP (hipStreamCreateWithFlags (&s, hipStreamNonBlocking));
  *stream = (void *)s;
  return 0;
}

int
vkl_stream_destroy (void *stream)
{
  // scratch that launches on this stream allocated goes with it
  VKL_HIP (hipStreamSynchronize ((hipStream_t)stream));
  vkl::gemm_release_workspace ((hipStream_t)stream);
  VKL_HIP (hipStreamDestroy ((hipStream_t)stream));
  return 0;
}

int
vkl_stream_sync (void *stream)
{
  VKL_HIP (hipStreamSynchronize ((hipStream_t)stream));
  return 0;
}

int
vkl_device_sync (void)
{
  VKL_HIP (hipDeviceSynchronize ());
  return 0;
}

int
vkl_malloc (void **p, size_t bytes)
{
  VKL_CHECK_ARG (p != nullptr);
  VKL_HIP (hipMalloc (p, bytes ? bytes : 1));
  return 0;
}

int
vkl_free (void *p)
{
  VKL_HIP (hipFree (p));
  return 0;
}

int
vkl_host_malloc_h (void **p, size_t bytes)
{
  VKL_CHECK_ARG (p != nullptr);
  VKL_HIP (hipHostMalloc (p, bytes ? bytes : 1, hipHostMallocDefault));
  return 0;
}

int
vkl_host_free_h (void *p)
{
  VKL_HIP (hipHostFree (p));
  return 0;
}

int
vkl_memcpy_h2d (void *dst, const void *src_h, size_t bytes, void *stream)
{
  if (bytes == 0)
    return 0;
  VKL_HIP (hipMemcpyAsync (dst, src_h, bytes, hipMemcpyHostToDevice,
                           (hipStream_t)stream));
  return 0;
}

int
vkl_memcpy_d2h (void *dst_h, const void *src, size_t bytes, void *stream)
{
  if (bytes == 0)
    return 0;
  VKL_HIP (hipMemcpyAsync (dst_h, src, bytes, hipMemcpyDeviceToHost,
                           (hipStream_t)stream));
  return 0;
}

int
vkl_memcpy_d2d (void *dst, const void *src, size_t bytes, void *stream)
{
  if (bytes == 0)
    return 0;
  VKL_HIP (hipMemcpyAsync (dst, src, bytes, hipMemcpyDeviceToDevice,
                           (hipStream_t)stream));
  return 0;
}

// A plain streaming copy (16 bytes per lane and iteration).  It is the unit
// against which hardware traffic counters are calibrated: one launch reads
// and writes exactly `n16` * 16 bytes.
__global__ __launch_bounds__ (512) void
copy_bytes_kernel (const uint4 *__restrict__ src, uint4 *__restrict__ dst,
                   size_t n16)
{
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n16; i += stride)
    dst[i] = src[i];
}

int
vkl_copy_kernel (void *dst, const void *src, size_t bytes, void *stream)
{
  VKL_CHECK_ARG (dst && src && (bytes % 16) == 0);
  VKL_CHECK_ARG (((uintptr_t)dst % 16) == 0 && ((uintptr_t)src % 16) == 0);
  if (bytes == 0)
    return 0;
  copy_bytes_kernel<<<dim3 (2048), dim3 (512), 0, (hipStream_t)stream>>> (
      (const uint4 *)src, (uint4 *)dst, bytes / 16);
  return vkl_launch_status ();
}

__global__ void
fill_bytes_kernel (uint8_t *dst, uint8_t v, size_t n)
{
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride)
    dst[i] = v;
}

int
vkl_mem_info (size_t *free_bytes, size_t *total_bytes)
{
  VKL_CHECK_ARG (free_bytes && total_bytes);
  VKL_HIP (hipMemGetInfo (free_bytes, total_bytes));
  return 0;
}

// A fill kernel rather than hipMemsetAsync, so that the call can be recorded
// into a HIP graph by a caller.
int
vkl_memset (void *dst, int value, size_t bytes, void *stream)
{
  if (bytes == 0)
    return 0;
  size_t blocks = (bytes + 255) / 256;
  if (blocks > 4096)
    blocks = 4096;
  fill_bytes_kernel<<<dim3 ((unsigned)blocks), dim3 (256), 0,
                      (hipStream_t)stream>>> ((uint8_t *)dst, (uint8_t)value,
                                              bytes);
  return vkl_launch_status ();
}

int
vkl_event_create (void **ev)
{
  VKL_CHECK_ARG (ev != nullptr);
  hipEvent_t e;
  VKL_HIP (hipEventCreate (&e));
  *ev = (void *)e;
  return 0;
}

int
vkl_event_destroy (void *ev)
{
  VKL_HIP (hipEventDestroy ((hipEvent_t)ev));
  return 0;
}

int
vkl_event_record (void *ev, void *stream)
{
  VKL_HIP (hipEventRecord ((hipEvent_t)ev, (hipStream_t)stream));
  return 0;
}

int
vkl_event_sync (void *ev)
{
  VKL_HIP (hipEventSynchronize ((hipEvent_t)ev));
  return 0;
}

int
vkl_event_elapsed_ms (void *start, void *stop, float *ms)
{
  VKL_CHECK_ARG (ms != nullptr);
  VKL_HIP (hipEventElapsedTime (ms, (hipEvent_t)start, (hipEvent_t)stop));
  return 0;
}
}
