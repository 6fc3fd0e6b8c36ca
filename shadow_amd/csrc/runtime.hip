// Device, stream, allocator, copy and event entry points: the part of the C ABI
// that Shadow's GPUAllocator / GPUContext sit on.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>

#include "../../include/shadow_hip.h"
#include "launch.h"

namespace {
inline int rc(hipError_t e) { return static_cast<int>(e); }
inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }
inline hipEvent_t as_event(void* e) { return static_cast<hipEvent_t>(e); }

int copy(void* dst, const void* src, size_t bytes, hipMemcpyKind kind, void* stream) {
  if (bytes == 0) return SHDW_OK;
  if (!dst || !src) return SHDW_E_INVALID_ARGUMENT;
  if (stream == nullptr) return rc(hipMemcpy(dst, src, bytes, kind));
  return rc(hipMemcpyAsync(dst, src, bytes, kind, as_stream(stream)));
}
}  // namespace

extern "C" {

int shdw_hip_device_count(int* count) {
  if (!count) return SHDW_E_INVALID_ARGUMENT;
  *count = 0;
  return rc(hipGetDeviceCount(count));
}

int shdw_hip_set_device(int device_id) {
  const hipError_t e = hipSetDevice(device_id);
  if (e != hipSuccess) return rc(e);
  // the library's own device memory is looked up here, once per device, so that
  // no later call has to do it at a time when it cannot (a stream being captured)
  return shdw::library_scratch_prepare();
}

int shdw_hip_device_info(int device_id, char* buf, size_t buf_size) {
  if (!buf || buf_size == 0) return SHDW_E_INVALID_ARGUMENT;
  hipDeviceProp_t prop;
  hipError_t e = hipGetDeviceProperties(&prop, device_id);
  if (e != hipSuccess) return rc(e);
  std::snprintf(buf, buf_size, "%s|%s|%d|%d", prop.name, prop.gcnArchName,
                prop.multiProcessorCount, prop.clockRate);
  return SHDW_OK;
}

int shdw_hip_stream_create(void** stream) {
  if (!stream) return SHDW_E_INVALID_ARGUMENT;
  hipStream_t s = nullptr;
  hipError_t e = hipStreamCreate(&s);  // default priority
  *stream = s;
  return rc(e);
}

int shdw_hip_stream_destroy(void* stream) {
  if (!stream) return SHDW_OK;
  return rc(hipStreamDestroy(as_stream(stream)));
}

int shdw_hip_stream_sync(void* stream) { return rc(hipStreamSynchronize(as_stream(stream))); }

const char* shdw_hip_error_string(int code) {
  switch (code) {
    case SHDW_OK: return "success";
    case SHDW_E_INVALID_ARGUMENT: return "shadow_hip: invalid argument";
    case SHDW_E_UNSUPPORTED: return "shadow_hip: unsupported shape";
    case SHDW_E_WORKSPACE: return "shadow_hip: workspace missing or too small";
    case SHDW_E_STATIC_SCRATCH:
      return "shadow_hip: this shape needs more scratch than the library's static buffer holds "
             "(shdw_hip_reduce_static_max_workspace_bytes); use shdw_hip_reduce with a workspace";
    default: break;
  }
  if (code < 0) return "shadow_hip: unknown error";
  return hipGetErrorString(static_cast<hipError_t>(code));
}

int shdw_hip_last_error(void) { return rc(hipGetLastError()); }

int shdw_hip_malloc(void** ptr, size_t bytes) {
  if (!ptr) return SHDW_E_INVALID_ARGUMENT;
  *ptr = nullptr;
  return rc(hipMalloc(ptr, bytes));
}

int shdw_hip_free(void* ptr) {
  if (!ptr) return SHDW_OK;
  return rc(hipFree(ptr));
}

int shdw_hip_mem_info(size_t* free_bytes, size_t* total_bytes) {
  size_t f = 0, t = 0;
  const int code = rc(hipMemGetInfo(&f, &t));
  if (free_bytes) *free_bytes = f;
  if (total_bytes) *total_bytes = t;
  return code;
}

int shdw_hip_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream) {
  return copy(dst, src, bytes, hipMemcpyHostToDevice, stream);
}
int shdw_hip_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream) {
  return copy(dst, src, bytes, hipMemcpyDeviceToHost, stream);
}
int shdw_hip_memcpy_d2d(void* dst, const void* src, size_t bytes, void* stream) {
  return copy(dst, src, bytes, hipMemcpyDeviceToDevice, stream);
}

int shdw_hip_host_malloc(void** ptr, size_t bytes) {
  if (!ptr) return SHDW_E_INVALID_ARGUMENT;
  *ptr = nullptr;
  return rc(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
}
int shdw_hip_host_free(void* ptr) {
  if (!ptr) return SHDW_OK;
  return rc(hipHostFree(ptr));
}

int shdw_hip_event_create(void** event) {
  if (!event) return SHDW_E_INVALID_ARGUMENT;
  hipEvent_t e = nullptr;
  hipError_t err = hipEventCreate(&e);
  *event = e;
  return rc(err);
}
int shdw_hip_event_destroy(void* event) {
  if (!event) return SHDW_OK;
  return rc(hipEventDestroy(as_event(event)));
}
int shdw_hip_event_record(void* event, void* stream) {
  return rc(hipEventRecord(as_event(event), as_stream(stream)));
}
int shdw_hip_event_sync(void* event) { return rc(hipEventSynchronize(as_event(event))); }
int shdw_hip_event_elapsed_ms(void* start, void* stop, float* ms) {
  if (!ms) return SHDW_E_INVALID_ARGUMENT;
  return rc(hipEventElapsedTime(ms, as_event(start), as_event(stop)));
}

}  // extern "C"
