// Device runtime calls of the itexhip C ABI (host only): what a TensorFlow StreamExecutor plugin needs
// from HIP - device enumeration, raw device and pinned host memory, streams, events, copies, fills,
// host callbacks.  The reference reaches its SYCL runtime through the ITEX_GPU* wrappers
// (third_party/build_option/sycl/runtime/itex_gpu_runtime.h, used by
// itex/core/devices/gpu/gpu_device_plugin.cc:27-376); these functions stand in their place.
// Every function makes `device` current on the calling thread when it takes one.
#include "common.hpp"

using namespace itexhip;

namespace {
#define ITEXHIP_RT(call, who)                                       \
  do {                                                              \
    hipError_t e_ = (call);                                         \
    if (e_ != hipSuccess) return itexhip::hip_fail(e_, who);        \
  } while (0)

__global__ void fill_u32_kernel(uint32_t* p, uint32_t pattern, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = pattern;
}
__global__ void fill_u8_kernel(uint8_t* p, uint8_t pattern, int64_t begin, int64_t n) {
  const int64_t i = begin + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) p[i] = pattern;
}
}  // namespace

extern "C" int itexhip_device_count(int* count) {
  ITEXHIP_REQUIRE(count != nullptr, "itexhip_device_count: null output");
  *count = 0;
  hipError_t e = hipGetDeviceCount(count);
  if (e == hipErrorNoDevice) {
    *count = 0;
    (void)hipGetLastError();
    return ITEXHIP_OK;
  }
  if (e != hipSuccess) return hip_fail(e, "itexhip_device_count");
  return ITEXHIP_OK;
}

extern "C" int itexhip_device_info(int device, char* name, size_t name_len, char* pci_bus_id, size_t pci_len,
                                   int64_t* total_memory, int* compute_units) {
  hipDeviceProp_t prop;
  ITEXHIP_RT(hipGetDeviceProperties(&prop, device), "itexhip_device_info");
  if (name && name_len) snprintf(name, name_len, "%s (%s)", prop.name, prop.gcnArchName);
  if (pci_bus_id && pci_len) ITEXHIP_RT(hipDeviceGetPCIBusId(pci_bus_id, static_cast<int>(pci_len), device), "itexhip_device_info");
  if (total_memory) *total_memory = static_cast<int64_t>(prop.totalGlobalMem);
  if (compute_units) *compute_units = prop.multiProcessorCount;
  return ITEXHIP_OK;
}

extern "C" int itexhip_mem_info(int device, int64_t* free_bytes, int64_t* total_bytes) {
  ITEXHIP_RT(hipSetDevice(device), "itexhip_mem_info");
  size_t f = 0, t = 0;
  ITEXHIP_RT(hipMemGetInfo(&f, &t), "itexhip_mem_info");
  if (free_bytes) *free_bytes = static_cast<int64_t>(f);
  if (total_bytes) *total_bytes = static_cast<int64_t>(t);
  return ITEXHIP_OK;
}

extern "C" int itexhip_malloc(int device, size_t bytes, void** ptr) {
  ITEXHIP_REQUIRE(ptr != nullptr, "itexhip_malloc: null output");
  *ptr = nullptr;
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_RT(hipSetDevice(device), "itexhip_malloc");
  ITEXHIP_RT(hipMalloc(ptr, bytes), "itexhip_malloc");
  return ITEXHIP_OK;
}

extern "C" int itexhip_free(int device, void* ptr) {
  if (ptr == nullptr) return ITEXHIP_OK;
  ITEXHIP_RT(hipSetDevice(device), "itexhip_free");
  ITEXHIP_RT(hipFree(ptr), "itexhip_free");
  return ITEXHIP_OK;
}

extern "C" int itexhip_host_malloc(size_t bytes, void** ptr) {
  ITEXHIP_REQUIRE(ptr != nullptr, "itexhip_host_malloc: null output");
  *ptr = nullptr;
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_RT(hipHostMalloc(ptr, bytes, hipHostMallocDefault), "itexhip_host_malloc");
  return ITEXHIP_OK;
}

extern "C" int itexhip_host_free(void* ptr) {
  if (ptr == nullptr) return ITEXHIP_OK;
  ITEXHIP_RT(hipHostFree(ptr), "itexhip_host_free");
  return ITEXHIP_OK;
}

extern "C" int itexhip_stream_create(int device, void** stream) {
  ITEXHIP_REQUIRE(stream != nullptr, "itexhip_stream_create: null output");
  ITEXHIP_RT(hipSetDevice(device), "itexhip_stream_create");
  hipStream_t s = nullptr;
  // default priority on purpose; non-blocking with respect to the legacy default stream
  ITEXHIP_RT(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "itexhip_stream_create");
  *stream = s;
  return ITEXHIP_OK;
}

extern "C" int itexhip_stream_destroy(void* stream) {
  if (stream == nullptr) return ITEXHIP_OK;
  ITEXHIP_RT(hipStreamDestroy(as_stream(stream)), "itexhip_stream_destroy");
  return ITEXHIP_OK;
}

/* 1: all work done, 0: still running */
extern "C" int itexhip_stream_query(void* stream, int* done) {
  ITEXHIP_REQUIRE(done != nullptr, "itexhip_stream_query: null output");
  hipError_t e = hipStreamQuery(as_stream(stream));
  if (e == hipErrorNotReady) {
    *done = 0;
    (void)hipGetLastError();
    return ITEXHIP_OK;
  }
  if (e != hipSuccess) return hip_fail(e, "itexhip_stream_query");
  *done = 1;
  return ITEXHIP_OK;
}

extern "C" int itexhip_event_create(int device, void** event) {
  ITEXHIP_REQUIRE(event != nullptr, "itexhip_event_create: null output");
  ITEXHIP_RT(hipSetDevice(device), "itexhip_event_create");
  hipEvent_t ev = nullptr;
  ITEXHIP_RT(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "itexhip_event_create");
  *event = ev;
  return ITEXHIP_OK;
}

extern "C" int itexhip_event_destroy(void* event) {
  if (event == nullptr) return ITEXHIP_OK;
  ITEXHIP_RT(hipEventDestroy(static_cast<hipEvent_t>(event)), "itexhip_event_destroy");
  return ITEXHIP_OK;
}

extern "C" int itexhip_event_record(void* event, void* stream) {
  ITEXHIP_REQUIRE(event != nullptr, "itexhip_event_record: null event");
  ITEXHIP_RT(hipEventRecord(static_cast<hipEvent_t>(event), as_stream(stream)), "itexhip_event_record");
  return ITEXHIP_OK;
}

/* 1: the recorded work has completed (or nothing was recorded), 0: pending */
extern "C" int itexhip_event_query(void* event, int* done) {
  ITEXHIP_REQUIRE(event != nullptr && done != nullptr, "itexhip_event_query: null argument");
  hipError_t e = hipEventQuery(static_cast<hipEvent_t>(event));
  if (e == hipErrorNotReady) {
    *done = 0;
    (void)hipGetLastError();
    return ITEXHIP_OK;
  }
  if (e != hipSuccess) return hip_fail(e, "itexhip_event_query");
  *done = 1;
  return ITEXHIP_OK;
}

extern "C" int itexhip_event_synchronize(void* event) {
  ITEXHIP_REQUIRE(event != nullptr, "itexhip_event_synchronize: null event");
  ITEXHIP_RT(hipEventSynchronize(static_cast<hipEvent_t>(event)), "itexhip_event_synchronize");
  return ITEXHIP_OK;
}

extern "C" int itexhip_stream_wait_event(void* stream, void* event) {
  ITEXHIP_REQUIRE(event != nullptr, "itexhip_stream_wait_event: null event");
  ITEXHIP_RT(hipStreamWaitEvent(as_stream(stream), static_cast<hipEvent_t>(event), 0), "itexhip_stream_wait_event");
  return ITEXHIP_OK;
}

extern "C" int itexhip_device_synchronize(int device) {
  ITEXHIP_RT(hipSetDevice(device), "itexhip_device_synchronize");
  ITEXHIP_RT(hipDeviceSynchronize(), "itexhip_device_synchronize");
  return ITEXHIP_OK;
}

extern "C" int itexhip_memcpy_d2h_async(void* dst_host, const void* src_device, size_t bytes, void* stream) {
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(dst_host && src_device, "itexhip_memcpy_d2h_async: null buffer");
  ITEXHIP_RT(hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, as_stream(stream)), "itexhip_memcpy_d2h_async");
  return ITEXHIP_OK;
}

/* Fill kernels (no memset nodes: these may be captured into HIP graphs).  bytes need not be a multiple
 * of 4 for the byte fill; the 32-bit fill takes a count of bytes that is. */
extern "C" int itexhip_memset8_async(void* dst, uint8_t pattern, size_t bytes, void* stream) {
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(dst != nullptr, "itexhip_memset8_async: null buffer");
  hipStream_t st = as_stream(stream);
  const uintptr_t addr = reinterpret_cast<uintptr_t>(dst);
  const int64_t n = static_cast<int64_t>(bytes);
  int64_t head = static_cast<int64_t>((4 - (addr & 3)) & 3);
  if (head > n) head = n;
  const int64_t words = (n - head) / 4;
  if (head > 0) fill_u8_kernel<<<1, 64, 0, st>>>(static_cast<uint8_t*>(dst), pattern, 0, head);
  if (words > 0) {
    const uint32_t p32 = 0x01010101u * pattern;
    fill_u32_kernel<<<static_cast<unsigned>((words + 255) / 256), 256, 0, st>>>(
        reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(dst) + head), p32, words);
  }
  const int64_t done = head + words * 4;
  if (done < n) fill_u8_kernel<<<1, 64, 0, st>>>(static_cast<uint8_t*>(dst), pattern, done, n);
  ITEXHIP_CHECK_LAUNCH("itexhip_memset8_async");
  return ITEXHIP_OK;
}

extern "C" int itexhip_memset32_async(void* dst, uint32_t pattern, size_t bytes, void* stream) {
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(dst != nullptr, "itexhip_memset32_async: null buffer");
  ITEXHIP_REQUIRE((bytes & 3) == 0 && (reinterpret_cast<uintptr_t>(dst) & 3) == 0,
                  "itexhip_memset32_async: address and size must be multiples of 4");
  const int64_t words = static_cast<int64_t>(bytes / 4);
  fill_u32_kernel<<<static_cast<unsigned>((words + 255) / 256), 256, 0, as_stream(stream)>>>(
      static_cast<uint32_t*>(dst), pattern, words);
  ITEXHIP_CHECK_LAUNCH("itexhip_memset32_async");
  return ITEXHIP_OK;
}

/* fn(arg) runs on a runtime thread once the work already on `stream` has completed */
extern "C" int itexhip_launch_host_func(void* stream, void (*fn)(void*), void* arg) {
  ITEXHIP_REQUIRE(fn != nullptr, "itexhip_launch_host_func: null function");
  ITEXHIP_RT(hipLaunchHostFunc(as_stream(stream), fn, arg), "itexhip_launch_host_func");
  return ITEXHIP_OK;
}
