// Runtime plumbing behind the C ABI: memory, copies, streams, events, error text.
#include <cstdarg>
#include <cstring>

#include "common.h"

namespace rwkv {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

const char* rwkv_hip_last_error(void) { return g_error; }

int rwkv_hip_device_count(int* count) {
  RWKV_REQUIRE(count != nullptr, "count is NULL");
  int n = 0;
  hipError_t err = hipGetDeviceCount(&n);
  if (err != hipSuccess) {
    (void)hipGetLastError();
    n = 0;
  }
  *count = n;
  return RWKV_OK;
}

int rwkv_hip_device_name(char* buf, size_t buf_len) {
  RWKV_REQUIRE(buf != nullptr && buf_len > 0, "bad buffer");
  hipDeviceProp_t prop;
  RWKV_HIP_TRY(hipGetDeviceProperties(&prop, 0));
  snprintf(buf, buf_len, "%s (%s, %d CUs)", prop.name, prop.gcnArchName, prop.multiProcessorCount);
  return RWKV_OK;
}

int rwkv_hip_malloc(void** ptr, size_t bytes) {
  RWKV_REQUIRE(ptr != nullptr, "ptr is NULL");
  *ptr = nullptr;
  if (bytes == 0) return RWKV_OK;
  RWKV_HIP_TRY(hipMalloc(ptr, bytes));
  return RWKV_OK;
}

int rwkv_hip_free(void* ptr) {
  if (ptr) RWKV_HIP_TRY(hipFree(ptr));
  return RWKV_OK;
}

int rwkv_hip_host_alloc(void** ptr_host, size_t bytes) {
  RWKV_REQUIRE(ptr_host != nullptr, "ptr is NULL");
  *ptr_host = nullptr;
  if (bytes == 0) return RWKV_OK;
  RWKV_HIP_TRY(hipHostMalloc(ptr_host, bytes, hipHostMallocDefault));
  return RWKV_OK;
}

int rwkv_hip_host_free(void* ptr_host) {
  if (ptr_host) RWKV_HIP_TRY(hipHostFree(ptr_host));
  return RWKV_OK;
}

int rwkv_hip_memcpy_h2d(void* dst, const void* src_host, size_t bytes) {
  if (bytes) RWKV_HIP_TRY(hipMemcpy(dst, src_host, bytes, hipMemcpyHostToDevice));
  return RWKV_OK;
}
int rwkv_hip_memcpy_d2h(void* dst_host, const void* src, size_t bytes) {
  if (bytes) RWKV_HIP_TRY(hipMemcpy(dst_host, src, bytes, hipMemcpyDeviceToHost));
  return RWKV_OK;
}
int rwkv_hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
  if (bytes) RWKV_HIP_TRY(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToDevice));
  return RWKV_OK;
}
int rwkv_hip_memcpy_h2d_async(rwkv_stream_t s, void* dst, const void* src_host, size_t bytes) {
  if (bytes) RWKV_HIP_TRY(hipMemcpyAsync(dst, src_host, bytes, hipMemcpyHostToDevice, as_stream(s)));
  return RWKV_OK;
}
int rwkv_hip_memcpy_d2h_async(rwkv_stream_t s, void* dst_host, const void* src, size_t bytes) {
  if (bytes) RWKV_HIP_TRY(hipMemcpyAsync(dst_host, src, bytes, hipMemcpyDeviceToHost, as_stream(s)));
  return RWKV_OK;
}
int rwkv_hip_memcpy_d2d_async(rwkv_stream_t s, void* dst, const void* src, size_t bytes) {
  if (bytes) RWKV_HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(s)));
  return RWKV_OK;
}
int rwkv_hip_memset(void* ptr, int value, size_t bytes) {
  if (bytes) RWKV_HIP_TRY(hipMemset(ptr, value, bytes));
  return RWKV_OK;
}
int rwkv_hip_mem_info(size_t* free_bytes, size_t* total_bytes) {
  RWKV_REQUIRE(free_bytes && total_bytes, "NULL output");
  RWKV_HIP_TRY(hipMemGetInfo(free_bytes, total_bytes));
  return RWKV_OK;
}

int rwkv_hip_stream_create(rwkv_stream_t* s) {
  RWKV_REQUIRE(s != nullptr, "stream out is NULL");
  hipStream_t st = nullptr;
  // default priority on purpose: every stream of this library runs at the same priority
  RWKV_HIP_TRY(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  *s = st;
  return RWKV_OK;
}
int rwkv_hip_stream_destroy(rwkv_stream_t s) {
  if (s) RWKV_HIP_TRY(hipStreamDestroy(as_stream(s)));
  return RWKV_OK;
}
int rwkv_hip_stream_sync(rwkv_stream_t s) {
  RWKV_HIP_TRY(hipStreamSynchronize(as_stream(s)));
  return RWKV_OK;
}
int rwkv_hip_device_sync(void) {
  RWKV_HIP_TRY(hipDeviceSynchronize());
  return RWKV_OK;
}

int rwkv_hip_event_create(void** ev) {
  RWKV_REQUIRE(ev != nullptr, "event out is NULL");
  hipEvent_t e = nullptr;
  RWKV_HIP_TRY(hipEventCreate(&e));
  *ev = e;
  return RWKV_OK;
}
int rwkv_hip_event_destroy(void* ev) {
  if (ev) RWKV_HIP_TRY(hipEventDestroy(reinterpret_cast<hipEvent_t>(ev)));
  return RWKV_OK;
}
int rwkv_hip_event_record(void* ev, rwkv_stream_t s) {
  RWKV_HIP_TRY(hipEventRecord(reinterpret_cast<hipEvent_t>(ev), as_stream(s)));
  return RWKV_OK;
}
int rwkv_hip_event_elapsed_ms(void* ev_start, void* ev_stop, float* ms) {
  RWKV_REQUIRE(ms != nullptr, "ms is NULL");
  RWKV_HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev_stop)));
  RWKV_HIP_TRY(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(ev_start), reinterpret_cast<hipEvent_t>(ev_stop)));
  return RWKV_OK;
}

}  // extern "C"
