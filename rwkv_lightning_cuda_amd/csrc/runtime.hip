// Runtime plumbing behind the C ABI: memory, copies, streams, events, error text.
#include <cstdarg>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

#include "common.h"

namespace rwkv {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int device_cu_count() {
  constexpr int kMaxDevices = 64;
  static int cached[kMaxDevices] = {0};  // racing first calls store the same value
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return 256;
  }
  if (cached[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    cached[dev] = n;
  }
  return cached[dev];
}

}  // namespace rwkv

using namespace rwkv;

namespace {

// One link of a chain of dependent launches: every block reads the counter the previous launch left, one thread
// writes it back incremented.  Next to no work: what a chain of these costs per link is the cost of a launch that
// has to wait for its predecessor.
__global__ void chain_link_kernel(unsigned* counter) {
  const unsigned seen = *counter;
  if (blockIdx.x == 0 && threadIdx.x == 0) *counter = seen + 1;
}

}  // namespace

extern "C" {

const char* rwkv_hip_last_error(void) { return g_error; }

int rwkv_hip_measure_launch_chain(int links, int blocks, int threads, int use_graph, int reps, float* us_per_link) {
  RWKV_REQUIRE(us_per_link != nullptr, "us_per_link is NULL");
  RWKV_REQUIRE(links >= 1 && links <= 4096 && blocks >= 1 && blocks <= 65536 && threads >= 1 && threads <= 1024 && reps >= 1 &&
                   reps <= 1000,
               "measure_launch_chain: argument out of range");
  hipStream_t st = nullptr;
  unsigned* counter = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  int rc = RWKV_OK;
  auto fail = [&](hipError_t err, const char* what) {
    if (err != hipSuccess && rc == RWKV_OK) {
      set_error("measure_launch_chain: %s failed: %s", what, hipGetErrorString(err));
      rc = RWKV_E_RUNTIME;
    }
    return err != hipSuccess;
  };
  auto chain = [&] {
    for (int i = 0; i < links; ++i) hipLaunchKernelGGL(chain_link_kernel, dim3(blocks), dim3(threads), 0, st, counter);
  };
  do {
    if (fail(hipStreamCreateWithFlags(&st, hipStreamNonBlocking), "stream create")) break;
    if (fail(hipMalloc(reinterpret_cast<void**>(&counter), 256), "malloc")) break;
    if (fail(hipMemsetAsync(counter, 0, 256, st), "memset")) break;
    if (fail(hipEventCreate(&e0), "event create") || fail(hipEventCreate(&e1), "event create")) break;
    if (use_graph) {
      if (fail(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal), "begin capture")) break;
      chain();
      if (fail(hipStreamEndCapture(st, &graph), "end capture")) break;
      if (fail(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "graph instantiate")) break;
    }
    auto run = [&] {
      if (use_graph) (void)hipGraphLaunch(exec, st);
      else chain();
    };
    run();  // warm
    if (fail(hipStreamSynchronize(st), "sync")) break;
    if (fail(hipEventRecord(e0, st), "event record")) break;
    for (int r = 0; r < reps; ++r) run();
    if (fail(hipEventRecord(e1, st), "event record")) break;
    if (fail(hipStreamSynchronize(st), "sync")) break;
    if (fail(hipGetLastError(), "launch")) break;
    float ms = 0.0f;
    if (fail(hipEventElapsedTime(&ms, e0, e1), "elapsed")) break;
    unsigned count = 0;
    if (fail(hipMemcpy(&count, counter, sizeof(count), hipMemcpyDeviceToHost), "copy back")) break;
    if (count != static_cast<unsigned>(links) * (reps + 1)) {
      set_error("measure_launch_chain: the chain counted %u links instead of %u", count, static_cast<unsigned>(links) * (reps + 1));
      rc = RWKV_E_RUNTIME;
      break;
    }
    *us_per_link = ms * 1e3f / (static_cast<float>(reps) * links);
  } while (false);
  if (exec) (void)hipGraphExecDestroy(exec);
  if (graph) (void)hipGraphDestroy(graph);
  if (e0) (void)hipEventDestroy(e0);
  if (e1) (void)hipEventDestroy(e1);
  if (counter) (void)hipFree(counter);
  if (st) (void)hipStreamDestroy(st);
  return rc;
}

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

// ---- recycled blocks: generation states and logits of a serving loop ----------------------------------------------
// A block given back through rwkv_hip_free_recycled is kept (per device and byte size, last in first out) and
// handed to the next rwkv_hip_malloc_recycled of that size, so the buffers of one request come back at the same
// addresses for the next one of the same shape - which is what a session's captured decode graphs are keyed by.
namespace {
struct RecycleBin {
  std::mutex lock;
  std::map<std::pair<int, size_t>, std::vector<void*>> blocks;  // (device, bytes) -> free blocks
  std::vector<std::pair<std::pair<int, size_t>, void*>> order;  // oldest first, for trimming
  size_t held = 0;
};
RecycleBin& recycle_bin() {
  static RecycleBin* bin = new RecycleBin();  // never destroyed: the runtime may be gone at exit
  return *bin;
}
constexpr size_t kRecycleMaxHeld = static_cast<size_t>(24) << 30;

// frees the oldest blocks until at most `keep` bytes are held (lock taken by the caller)
void recycle_trim_locked(RecycleBin& bin, size_t keep) {
  while (bin.held > keep && !bin.order.empty()) {
    const auto entry = bin.order.front();
    bin.order.erase(bin.order.begin());
    auto& list = bin.blocks[entry.first];
    for (size_t i = 0; i < list.size(); ++i) {
      if (list[i] == entry.second) {
        list.erase(list.begin() + static_cast<long>(i));
        break;
      }
    }
    (void)hipFree(entry.second);
    bin.held -= entry.first.second;
  }
}
}  // namespace

int rwkv_hip_malloc_recycled(void** ptr, size_t bytes) {
  RWKV_REQUIRE(ptr != nullptr, "ptr is NULL");
  *ptr = nullptr;
  if (bytes == 0) return RWKV_OK;
  int dev = 0;
  RWKV_HIP_TRY(hipGetDevice(&dev));
  RecycleBin& bin = recycle_bin();
  {
    std::lock_guard<std::mutex> guard(bin.lock);
    auto it = bin.blocks.find(std::make_pair(dev, bytes));
    if (it != bin.blocks.end() && !it->second.empty()) {
      void* p = it->second.back();
      it->second.pop_back();
      for (size_t i = bin.order.size(); i-- > 0;) {
        if (bin.order[i].second == p) {
          bin.order.erase(bin.order.begin() + static_cast<long>(i));
          break;
        }
      }
      bin.held -= bytes;
      *ptr = p;
      return RWKV_OK;
    }
  }
  hipError_t err = hipMalloc(ptr, bytes);
  if (err == hipErrorOutOfMemory) {  // give the held blocks back and try once more
    (void)hipGetLastError();
    std::lock_guard<std::mutex> guard(bin.lock);
    recycle_trim_locked(bin, 0);
    err = hipMalloc(ptr, bytes);
  }
  RWKV_HIP_TRY(err);
  return RWKV_OK;
}

int rwkv_hip_free_recycled(void* ptr, size_t bytes) {
  if (!ptr) return RWKV_OK;
  if (bytes == 0 || bytes > kRecycleMaxHeld) return rwkv_hip_free(ptr);
  // like hipFree, returns only when the device no longer uses the block
  RWKV_HIP_TRY(hipDeviceSynchronize());
  int dev = 0;
  RWKV_HIP_TRY(hipGetDevice(&dev));
  RecycleBin& bin = recycle_bin();
  std::lock_guard<std::mutex> guard(bin.lock);
  recycle_trim_locked(bin, kRecycleMaxHeld - bytes);
  const auto key = std::make_pair(dev, bytes);
  bin.blocks[key].push_back(ptr);
  bin.order.push_back(std::make_pair(key, ptr));
  bin.held += bytes;
  return RWKV_OK;
}

int rwkv_hip_recycle_trim(void) {
  RecycleBin& bin = recycle_bin();
  std::lock_guard<std::mutex> guard(bin.lock);
  recycle_trim_locked(bin, 0);
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
  {  // blocks held for recycling are free memory to the caller (an allocation that needs them gets them)
    RecycleBin& bin = recycle_bin();
    std::lock_guard<std::mutex> guard(bin.lock);
    *free_bytes += bin.held;
  }
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
int rwkv_hip_event_sync(void* ev) {
  RWKV_REQUIRE(ev != nullptr, "event is NULL");
  RWKV_HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev)));
  return RWKV_OK;
}
int rwkv_hip_stream_wait_event(rwkv_stream_t s, void* ev) {
  RWKV_REQUIRE(ev != nullptr, "event is NULL");
  RWKV_HIP_TRY(hipStreamWaitEvent(as_stream(s), reinterpret_cast<hipEvent_t>(ev), 0));
  return RWKV_OK;
}
int rwkv_hip_event_elapsed_ms(void* ev_start, void* ev_stop, float* ms) {
  RWKV_REQUIRE(ms != nullptr, "ms is NULL");
  RWKV_HIP_TRY(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev_stop)));
  RWKV_HIP_TRY(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(ev_start), reinterpret_cast<hipEvent_t>(ev_stop)));
  return RWKV_OK;
}

}  // extern "C"
