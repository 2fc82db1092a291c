// Two-tier positional store: an HBM slice followed by a pinned, device-mapped
// host slice.  World size is 1, so the peer tier and its IPC handle exchange
// (upstream src/chunk_tensor.cc:112-139) have no counterpart here.
#include <atomic>
#include <cstdarg>
#include <chrono>
#include <mutex>
#include <vector>
#include <cstring>
#include <new>

#include "common.h"

namespace dgs {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// HBM bytes held by live stores (upstream src/cuda_context.h:11-38, made atomic).
static std::atomic<int64_t> g_allocated{0};

constexpr int kDebugOptions = 5;
static std::atomic<int64_t> g_debug[kDebugOptions];
int64_t debug_option(int32_t option) {
  return option >= 0 && option < kDebugOptions ? g_debug[option].load(std::memory_order_relaxed) : 0;
}

}  // namespace dgs

struct dgs_store {
  int64_t total = 0;
  int64_t device_elems = 0;
  int64_t host_elems = 0;
  int32_t elem_bytes = 0;
  int device = -1;
  void* dev = nullptr;       // HBM slice
  void* host_cpu = nullptr;  // pinned slice, CPU address
  void* host_dev = nullptr;  // same memory, device address
};

DGS_API const char* dgs_last_error(void) { return dgs::g_error; }

DGS_API const char* dgs_status_name(dgs_status s) {
  switch (s) {
    case DGS_OK: return "DGS_OK";
    case DGS_ERR_INVALID: return "DGS_ERR_INVALID";
    case DGS_ERR_HIP: return "DGS_ERR_HIP";
    case DGS_ERR_WORKSPACE: return "DGS_ERR_WORKSPACE";
    case DGS_ERR_UNSUPPORTED: return "DGS_ERR_UNSUPPORTED";
    case DGS_ERR_RANGE: return "DGS_ERR_RANGE";
    default: return "DGS_ERR_?";
  }
}

DGS_API int dgs_abi_version(void) { return DGS_ABI_VERSION; }

DGS_API dgs_status dgs_debug_set(int32_t option, int64_t value) {
  DGS_REQUIRE(option >= 0 && option < dgs::kDebugOptions, DGS_ERR_INVALID, "debug_set: unknown option %d", option);
  dgs::g_debug[option].store(value, std::memory_order_relaxed);
  return DGS_OK;
}

namespace dgs {
namespace {
template <int OP>
__global__ __launch_bounds__(256) void probe_table_kernel(unsigned long long* __restrict__ table, uint64_t slots,
                                                          int64_t n_ops, uint64_t salt,
                                                          unsigned long long* __restrict__ sink) {
  const int64_t j = int64_t(blockIdx.x) * 256 + threadIdx.x;
  if (j >= n_ops) return;
  uint64_t x = uint64_t(j) * 0x9E3779B97F4A7C15ull + salt;
  x ^= x >> 31;
  x *= 0xBF58476D1CE4E5B9ull;
  x ^= x >> 29;
  unsigned long long* slot = table + x % slots;  // always inside the table
  unsigned long long seen = ~0ull;
  if (OP == DGS_PROBE_LOAD) seen = __builtin_nontemporal_load(slot);
  if (OP == DGS_PROBE_STORE) *slot = static_cast<unsigned long long>(j);
  if (OP == DGS_PROBE_ATOMIC_MIN) seen = atomicMin(slot, static_cast<unsigned long long>(j) | (salt << 40));
  if (OP == DGS_PROBE_ATOMIC_MIN_NO_RETURN) atomicMin(slot, static_cast<unsigned long long>(j) | (salt << 40));
  if (seen == 0x0123456789abcdefull) *sink = seen;  // keeps the value alive; practically never taken
}
}  // namespace
}  // namespace dgs

DGS_API dgs_status dgs_debug_probe_table(int32_t op, void* table, int64_t slots, int64_t n_ops, uint64_t salt,
                                         void* sink, void* stream) {
  using namespace dgs;
  DGS_REQUIRE(op >= DGS_PROBE_LOAD && op <= DGS_PROBE_ATOMIC_MIN_NO_RETURN, DGS_ERR_INVALID, "probe: unknown op %d", op);
  DGS_REQUIRE(table != nullptr && sink != nullptr && slots > 0, DGS_ERR_INVALID, "probe: null table or no slots");
  DGS_REQUIRE(n_ops >= 0 && n_ops <= (int64_t(1) << 38), DGS_ERR_INVALID, "probe: n_ops=%lld", (long long)n_ops);
  if (n_ops == 0) return DGS_OK;
  const dim3 grid(uint32_t((n_ops + 255) / 256)), block(256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto* t = static_cast<unsigned long long*>(table);
  auto* k = static_cast<unsigned long long*>(sink);
  switch (op) {
    case DGS_PROBE_LOAD: hipLaunchKernelGGL(probe_table_kernel<DGS_PROBE_LOAD>, grid, block, 0, st, t, uint64_t(slots), n_ops, salt, k); break;
    case DGS_PROBE_STORE: hipLaunchKernelGGL(probe_table_kernel<DGS_PROBE_STORE>, grid, block, 0, st, t, uint64_t(slots), n_ops, salt, k); break;
    case DGS_PROBE_ATOMIC_MIN: hipLaunchKernelGGL(probe_table_kernel<DGS_PROBE_ATOMIC_MIN>, grid, block, 0, st, t, uint64_t(slots), n_ops, salt, k); break;
    default: hipLaunchKernelGGL(probe_table_kernel<DGS_PROBE_ATOMIC_MIN_NO_RETURN>, grid, block, 0, st, t, uint64_t(slots), n_ops, salt, k); break;
  }
  DGS_LAUNCH_CHECK();
  return DGS_OK;
}

DGS_API dgs_status dgs_store_split(int64_t total_elems, int32_t elem_bytes, int64_t capacity_bytes,
                                   int64_t* device_elems, int64_t* host_elems) {
  DGS_REQUIRE(total_elems >= 0, DGS_ERR_INVALID, "store: negative element count %lld",
              (long long)total_elems);
  DGS_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4 || elem_bytes == 8,
              DGS_ERR_INVALID, "store: element width %d is not 1, 2, 4 or 8", elem_bytes);
  DGS_REQUIRE(capacity_bytes >= 0, DGS_ERR_INVALID, "store: capacity_per_gpu %lld is negative",
              (long long)capacity_bytes);
  DGS_REQUIRE(device_elems && host_elems, DGS_ERR_INVALID, "store: null output pointer");
  int64_t dev = capacity_bytes / elem_bytes;
  if (dev > total_elems) dev = total_elems;
  *device_elems = dev;
  *host_elems = total_elems - dev;
  return DGS_OK;
}

DGS_API dgs_status dgs_store_create(int64_t total_elems, int32_t elem_bytes, int64_t capacity_bytes,
                                    dgs_store** out) {
  DGS_REQUIRE(out != nullptr, DGS_ERR_INVALID, "store: null output pointer");
  *out = nullptr;
  int64_t dev_elems = 0, host_elems = 0;
  dgs_status st = dgs_store_split(total_elems, elem_bytes, capacity_bytes, &dev_elems, &host_elems);
  if (st != DGS_OK) return st;

  dgs_store* s = new (std::nothrow) dgs_store();
  DGS_REQUIRE(s != nullptr, DGS_ERR_INVALID, "store: out of host memory");
  s->total = total_elems;
  s->device_elems = dev_elems;
  s->host_elems = host_elems;
  s->elem_bytes = elem_bytes;
  hipError_t e = hipGetDevice(&s->device);
  if (e == hipSuccess && host_elems > 0) {
    e = hipHostMalloc(&s->host_cpu, size_t(host_elems) * elem_bytes,
                      hipHostMallocMapped | hipHostMallocPortable);
    if (e == hipSuccess) e = hipHostGetDevicePointer(&s->host_dev, s->host_cpu, 0);
  }
  if (e == hipSuccess && dev_elems > 0) {
    const size_t bytes = size_t(dev_elems) * elem_bytes;
    e = hipMalloc(&s->dev, bytes);
    if (e == hipSuccess) {
      dgs::g_allocated += int64_t(bytes);
      e = hipMemset(s->dev, 0xFF, bytes);
    }
  }
  if (e != hipSuccess) {
    dgs::set_error("store: allocating %lld device + %lld host elements of %d B failed: %s",
                   (long long)dev_elems, (long long)host_elems, elem_bytes, hipGetErrorString(e));
    dgs_store_destroy(s);
    return DGS_ERR_HIP;
  }
  *out = s;
  return DGS_OK;
}

DGS_API dgs_status dgs_store_destroy(dgs_store* s) {
  if (s == nullptr) return DGS_OK;
  hipError_t first = hipSuccess;
  if (s->dev) {
    hipError_t e = hipFree(s->dev);
    if (e == hipSuccess) dgs::g_allocated -= s->device_elems * int64_t(s->elem_bytes);
    else first = e;
  }
  if (s->host_cpu) {
    hipError_t e = hipHostFree(s->host_cpu);
    if (e != hipSuccess && first == hipSuccess) first = e;
  }
  delete s;
  if (first != hipSuccess) {
    dgs::set_error("store: release failed: %s", hipGetErrorString(first));
    return DGS_ERR_HIP;
  }
  return DGS_OK;
}

DGS_API dgs_status dgs_store_load(dgs_store* s, const void* src, int64_t n_elems) {
  DGS_REQUIRE(s != nullptr, DGS_ERR_INVALID, "store: null store");
  DGS_REQUIRE(n_elems == s->total, DGS_ERR_INVALID,
              "store: load of %lld elements into a store of %lld", (long long)n_elems,
              (long long)s->total);
  DGS_REQUIRE(src != nullptr || n_elems == 0, DGS_ERR_INVALID, "store: null source");
  const char* p = static_cast<const char*>(src);
  const size_t dev_bytes = size_t(s->device_elems) * s->elem_bytes;
  if (dev_bytes) DGS_HIP_TRY(hipMemcpy(s->dev, p, dev_bytes, hipMemcpyHostToDevice));
  if (s->host_elems) memcpy(s->host_cpu, p + dev_bytes, size_t(s->host_elems) * s->elem_bytes);
  return DGS_OK;
}

DGS_API dgs_status dgs_store_view(const dgs_store* s, dgs_view* v) {
  DGS_REQUIRE(s != nullptr && v != nullptr, DGS_ERR_INVALID, "store: null argument");
  v->dev = s->dev;
  v->host = s->host_dev;
  v->threshold = s->device_elems;
  v->total = s->total;
  v->elem_bytes = s->elem_bytes;
  v->reserved_ = 0;
  return DGS_OK;
}

DGS_API dgs_status dgs_store_slices(const dgs_store* s, void** dev_ptr, int64_t* device_elems,
                                    void** host_cpu_ptr, int64_t* host_elems) {
  DGS_REQUIRE(s != nullptr, DGS_ERR_INVALID, "store: null store");
  if (dev_ptr) *dev_ptr = s->dev;
  if (device_elems) *device_elems = s->device_elems;
  if (host_cpu_ptr) *host_cpu_ptr = s->host_cpu;
  if (host_elems) *host_elems = s->host_elems;
  return DGS_OK;
}

DGS_API int64_t dgs_current_allocated(void) { return dgs::g_allocated.load(); }

DGS_API dgs_status dgs_read_back(void* host_dst, const void* dev_src, size_t n_bytes, void* stream) {
  DGS_REQUIRE(host_dst != nullptr && dev_src != nullptr, DGS_ERR_INVALID, "read_back: null pointer");
  hipStream_t st = static_cast<hipStream_t>(stream);
  DGS_HIP_TRY(hipMemcpyAsync(host_dst, dev_src, n_bytes, hipMemcpyDeviceToHost, st));
  DGS_HIP_TRY(hipStreamSynchronize(st));
  return DGS_OK;
}

namespace dgs {
// Recycled events for dgs_read_back_begin/_wait (default flags plus no timing).
static std::mutex g_event_mutex;
static std::vector<hipEvent_t> g_event_pool;
}  // namespace dgs

DGS_API dgs_status dgs_ticket_record(void* stream, void** ticket) {
  DGS_REQUIRE(ticket != nullptr, DGS_ERR_INVALID, "ticket_record: null ticket");
  hipEvent_t ev = nullptr;
  {
    std::lock_guard<std::mutex> lock(dgs::g_event_mutex);
    if (!dgs::g_event_pool.empty()) {
      ev = dgs::g_event_pool.back();
      dgs::g_event_pool.pop_back();
    }
  }
  if (ev == nullptr) DGS_HIP_TRY(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
  const hipError_t e = hipEventRecord(ev, static_cast<hipStream_t>(stream));
  if (e != hipSuccess) {
    std::lock_guard<std::mutex> lock(dgs::g_event_mutex);
    dgs::g_event_pool.push_back(ev);
    dgs::set_error("ticket_record: %s", hipGetErrorString(e));
    return DGS_ERR_HIP;
  }
  *ticket = ev;
  return DGS_OK;
}

DGS_API dgs_status dgs_ticket_stream_wait(void* stream, void* ticket) {
  DGS_REQUIRE(ticket != nullptr, DGS_ERR_INVALID, "ticket_stream_wait: null ticket");
  DGS_HIP_TRY(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(ticket), 0));
  return DGS_OK;
}

DGS_API dgs_status dgs_ticket_wait(void* ticket) {
  DGS_REQUIRE(ticket != nullptr, DGS_ERR_INVALID, "ticket_wait: null ticket");
  hipEvent_t ev = static_cast<hipEvent_t>(ticket);
  const hipError_t e = hipEventSynchronize(ev);
  {
    std::lock_guard<std::mutex> lock(dgs::g_event_mutex);
    dgs::g_event_pool.push_back(ev);
  }
  if (e != hipSuccess) {
    dgs::set_error("ticket_wait: %s", hipGetErrorString(e));
    return DGS_ERR_HIP;
  }
  return DGS_OK;
}

namespace dgs {
// Polls `n_words` host words until all are non-negative.  `still_running` is asked now and then
// whether the work that writes them can still be under way (it may cost far more than a poll:
// a stream query takes tens of microseconds, so the first one comes after 200 us of polling and
// the next ones 100 us apart); when it says no, or fails, the wait ends.
template <typename StillRunning>
static hipError_t poll_words(const int64_t* words, int32_t n_words, StillRunning still_running) {
  using clock = std::chrono::steady_clock;
  int32_t seen = 0;  // words [0, seen) have turned non-negative
  clock::time_point next_ask;
  bool timing = false;
  for (uint32_t spins = 1;; ++spins) {
    while (seen < n_words && __atomic_load_n(words + seen, __ATOMIC_ACQUIRE) >= 0) ++seen;
    if (seen == n_words) return hipSuccess;
    if ((spins & 63u) == 0) {
      const clock::time_point now = clock::now();
      if (!timing) {
        timing = true;
        next_ask = now + std::chrono::microseconds(200);
      } else if (now >= next_ask) {
        const hipError_t e = still_running();
        if (e != hipErrorNotReady) return e;  // finished (the words are what they will be) or failed
        next_ask = clock::now() + std::chrono::microseconds(100);
      }
    }
    __builtin_ia32_pause();
  }
}
}  // namespace dgs

DGS_API dgs_status dgs_ticket_sync_words(void* ticket, const int64_t* words, int32_t n_words) {
  DGS_REQUIRE(ticket != nullptr, DGS_ERR_INVALID, "ticket_sync_words: null ticket");
  DGS_REQUIRE(words != nullptr && n_words >= 1, DGS_ERR_INVALID, "ticket_sync_words: no words");
  hipEvent_t ev = static_cast<hipEvent_t>(ticket);
  const hipError_t e = dgs::poll_words(words, n_words, [ev] { return hipEventQuery(ev); });
  if (e != hipSuccess) {
    dgs::set_error("ticket_sync_words: %s", hipGetErrorString(e));
    return DGS_ERR_HIP;
  }
  return DGS_OK;
}

DGS_API dgs_status dgs_ticket_wait_words(void* ticket, const int64_t* words, int32_t n_words) {
  DGS_REQUIRE(ticket != nullptr, DGS_ERR_INVALID, "ticket_wait_words: null ticket");
  DGS_REQUIRE(words != nullptr && n_words >= 1, DGS_ERR_INVALID, "ticket_wait_words: no words");
  const dgs_status s = dgs_ticket_sync_words(ticket, words, n_words);
  dgs_ticket_release(ticket);
  return s;
}

DGS_API dgs_status dgs_ticket_sync(void* ticket) {
  DGS_REQUIRE(ticket != nullptr, DGS_ERR_INVALID, "ticket_sync: null ticket");
  const hipError_t e = hipEventSynchronize(static_cast<hipEvent_t>(ticket));
  if (e != hipSuccess) {
    dgs::set_error("ticket_sync: %s", hipGetErrorString(e));
    return DGS_ERR_HIP;
  }
  return DGS_OK;
}

DGS_API dgs_status dgs_stream_wait_words(void* stream, const int64_t* words, int32_t n_words) {
  DGS_REQUIRE(words != nullptr && n_words >= 1, DGS_ERR_INVALID, "stream_wait_words: no words");
  hipStream_t st = static_cast<hipStream_t>(stream);
  const hipError_t e = dgs::poll_words(words, n_words, [st] { return hipStreamQuery(st); });
  if (e != hipSuccess) {
    dgs::set_error("stream_wait_words: %s", hipGetErrorString(e));
    return DGS_ERR_HIP;
  }
  return DGS_OK;
}

DGS_API dgs_status dgs_ticket_release(void* ticket) {
  DGS_REQUIRE(ticket != nullptr, DGS_ERR_INVALID, "ticket_release: null ticket");
  std::lock_guard<std::mutex> lock(dgs::g_event_mutex);
  dgs::g_event_pool.push_back(static_cast<hipEvent_t>(ticket));
  return DGS_OK;
}

DGS_API dgs_status dgs_stream_query(void* stream, int32_t* idle) {
  DGS_REQUIRE(idle != nullptr, DGS_ERR_INVALID, "stream_query: null output");
  *idle = 0;
  const hipError_t e = hipStreamQuery(static_cast<hipStream_t>(stream));
  if (e == hipErrorNotReady) return DGS_OK;
  if (e == hipSuccess) {
    *idle = 1;
    return DGS_OK;
  }
  if (e == hipErrorInvalidHandle || e == hipErrorInvalidResourceHandle || e == hipErrorContextIsDestroyed) {
    // the handle names no live stream: nothing can be pending on it.  Only this error is taken
    // off the runtime's last-error slot; any other one stays there and is reported.
    (void)hipGetLastError();
    *idle = 1;
    return DGS_OK;
  }
  dgs::set_error("stream_query: %s", hipGetErrorString(e));
  return DGS_ERR_HIP;
}

DGS_API dgs_status dgs_ticket_query(void* ticket, int32_t* reached) {
  DGS_REQUIRE(ticket != nullptr && reached != nullptr, DGS_ERR_INVALID, "ticket_query: null argument");
  *reached = 0;
  const hipError_t e = hipEventQuery(static_cast<hipEvent_t>(ticket));
  if (e == hipErrorNotReady) return DGS_OK;
  if (e != hipSuccess) {
    dgs::set_error("ticket_query: %s", hipGetErrorString(e));
    return DGS_ERR_HIP;
  }
  *reached = 1;
  return DGS_OK;
}

DGS_API dgs_status dgs_read_back_begin(void* host_dst, const void* dev_src, size_t n_bytes, void* stream,
                                       void** ticket) {
  DGS_REQUIRE(host_dst != nullptr && dev_src != nullptr && ticket != nullptr, DGS_ERR_INVALID,
              "read_back_begin: null pointer");
  DGS_HIP_TRY(hipMemcpyAsync(host_dst, dev_src, n_bytes, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
  return dgs_ticket_record(stream, ticket);
}

DGS_API dgs_status dgs_read_back_wait(void* ticket) { return dgs_ticket_wait(ticket); }
