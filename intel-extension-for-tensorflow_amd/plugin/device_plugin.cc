// StreamExecutor side of the PluggableDevice plugin: SE_InitPlugin and the platform / device / stream
// executor callbacks over the HIP runtime calls of the itexhip C ABI.  TensorFlow calls SE_InitPlugin
// once after dlopen and from then on drives the device through the function tables filled here
// (the reference: itex/core/devices/xpu_device.cc:656-693, 772-812 and
// itex/core/devices/gpu/gpu_device_plugin.cc:27-376).
//
// Device memory comes from one ArenaAllocator per device (the reference puts its BFCAllocator there,
// gpu_device_plugin.cc:57-83); use_bfc_allocator stays off so that TensorFlow does not stack a second
// sub-allocator on top.  Streams are created at the default priority.  Timers are not implemented, as
// in the reference (:209-231).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "arena_allocator.h"
#include "itexhip.h"
#include "tf_stream_executor_subset.h"

struct SP_Event_st {
  void* event_handle;  // hipEvent_t
};
struct SP_Timer_st {
  uint64_t nanoseconds;
};

namespace itex_amd {
namespace {

const char* DeviceType() {
  const char* dev = std::getenv("ITEX_AMD_DEVICE_TYPE");
  return dev && dev[0] ? dev : "XPU";
}

struct DeviceState {
  int ordinal = 0;
  std::string name, pci;
  std::unique_ptr<ArenaAllocator> arena;
};

std::mutex g_mu;
std::vector<std::unique_ptr<DeviceState>> g_devices;

void Fail(TF_Status* status, const char* what) {
  if (status) TF_SetStatus(status, TF_INTERNAL, (std::string(what) + ": " + itexhip_last_error()).c_str());
}
void Ok(TF_Status* status) {
  if (status) TF_SetStatus(status, TF_OK, "");
}

DeviceState* StateOf(const SP_Device* device) { return static_cast<DeviceState*>(device->device_handle); }

size_t MemoryLimitFromEnv() {
  // same switch as the reference's allocator (bfc_allocator.cc:253-267)
  const char* v = std::getenv("ITEX_LIMIT_MEMORY_SIZE_IN_MB");
  if (!v || !v[0]) return 0;
  const long long mb = std::atoll(v);
  return mb > 0 ? static_cast<size_t>(mb) << 20 : 0;
}

// ---- platform ---------------------------------------------------------------------------------
void get_device_count(const SP_Platform*, int* device_count, TF_Status* status) {
  if (itexhip_device_count(device_count) != ITEXHIP_OK) return Fail(status, "get_device_count");
  Ok(status);
}

void create_device(const SP_Platform*, SE_CreateDeviceParams* params, TF_Status* status) {
  int count = 0;
  if (itexhip_device_count(&count) != ITEXHIP_OK) return Fail(status, "create_device");
  if (params->ordinal < 0 || params->ordinal >= count) {
    TF_SetStatus(status, TF_INVALID_ARGUMENT, "create_device: no such device ordinal");
    return;
  }
  std::lock_guard<std::mutex> lock(g_mu);
  if (static_cast<int>(g_devices.size()) <= params->ordinal) g_devices.resize(params->ordinal + 1);
  if (!g_devices[params->ordinal]) {
    auto st = std::make_unique<DeviceState>();
    st->ordinal = params->ordinal;
    char name[256] = "", pci[64] = "";
    if (itexhip_device_info(params->ordinal, name, sizeof(name), pci, sizeof(pci), nullptr, nullptr) != ITEXHIP_OK)
      return Fail(status, "create_device");
    st->name = name;
    st->pci = pci;
    const int ordinal = params->ordinal;
    st->arena = std::make_unique<ArenaAllocator>(
        [ordinal](size_t bytes) -> void* {
          void* p = nullptr;
          return itexhip_malloc(ordinal, bytes, &p) == ITEXHIP_OK ? p : nullptr;
        },
        [ordinal](void* p) { itexhip_free(ordinal, p); }, MemoryLimitFromEnv());
    g_devices[params->ordinal] = std::move(st);
  }
  DeviceState* st = g_devices[params->ordinal].get();
  params->device->struct_size = SP_DEVICE_STRUCT_SIZE;
  params->device->ordinal = params->ordinal;
  params->device->device_handle = st;
  params->device->hardware_name = st->name.c_str();
  params->device->device_vendor = "AMD";
  params->device->pci_bus_id = st->pci.c_str();
  Ok(status);
}

void destroy_device(const SP_Platform*, SP_Device* device) {
  // the arena (and its device memory) lives until the process ends: tensors may outlive the SP_Device
  device->device_handle = nullptr;
  device->ordinal = -1;
}

int32_t get_numa_node(const SP_Device*) { return -1; }
int64_t get_memory_bandwidth(const SP_Device*) { return 8000LL * 1000 * 1000 * 1000; }  // HBM3E, bytes/s
double get_gflops(const SP_Device*) { return 157300.0; }                                // fp32 vector, GFLOP/s

void create_device_fns(const SP_Platform*, SE_CreateDeviceFnsParams* params, TF_Status* status) {
  params->device_fns->struct_size = SP_DEVICE_FNS_STRUCT_SIZE;
  params->device_fns->get_numa_node = get_numa_node;
  params->device_fns->get_memory_bandwidth = get_memory_bandwidth;
  params->device_fns->get_gflops = get_gflops;
  Ok(status);
}
void destroy_device_fns(const SP_Platform*, SP_DeviceFns*) {}

// ---- memory -----------------------------------------------------------------------------------
void allocate(const SP_Device* device, uint64_t size, int64_t /*memory_space*/, SP_DeviceMemoryBase* mem) {
  mem->struct_size = SP_DEVICE_MEMORY_BASE_STRUCT_SIZE;
  mem->opaque = size ? StateOf(device)->arena->Allocate(size) : nullptr;
  mem->size = mem->opaque ? size : 0;
  mem->payload = 0;
}
void deallocate(const SP_Device* device, SP_DeviceMemoryBase* mem) {
  if (mem->opaque && !StateOf(device)->arena->Deallocate(mem->opaque))
    std::fprintf(stderr, "itex_amd: deallocate of an address this device did not allocate: %p\n", mem->opaque);
  mem->opaque = nullptr;
  mem->size = 0;
}
void* host_memory_allocate(const SP_Device*, uint64_t size) {
  void* p = nullptr;
  return itexhip_host_malloc(size, &p) == ITEXHIP_OK ? p : nullptr;
}
void host_memory_deallocate(const SP_Device*, void* mem) { itexhip_host_free(mem); }

TF_Bool get_allocator_stats(const SP_Device* device, SP_AllocatorStats* stats) {
  const ArenaStats s = StateOf(device)->arena->stats();
  stats->struct_size = SP_ALLOCATORSTATS_STRUCT_SIZE;
  stats->num_allocs = s.num_allocs;
  stats->bytes_in_use = s.bytes_in_use;
  stats->peak_bytes_in_use = s.peak_bytes_in_use;
  stats->largest_alloc_size = s.largest_alloc_size;
  stats->has_bytes_limit = s.bytes_limit != 0;
  stats->bytes_limit = s.bytes_limit;
  stats->bytes_reserved = s.bytes_reserved;
  stats->peak_bytes_reserved = s.peak_bytes_reserved;
  stats->has_bytes_reservable_limit = 0;
  stats->bytes_reservable_limit = 0;
  stats->largest_free_block_bytes = s.largest_free_block_bytes;
  return 1;
}
TF_Bool device_memory_usage(const SP_Device* device, int64_t* free, int64_t* total) {
  return itexhip_mem_info(StateOf(device)->ordinal, free, total) == ITEXHIP_OK;
}

// ---- streams and events ------------------------------------------------------------------------
void create_stream(const SP_Device* device, SP_Stream* stream, TF_Status* status) {
  void* h = nullptr;
  if (itexhip_stream_create(StateOf(device)->ordinal, &h) != ITEXHIP_OK) return Fail(status, "create_stream");
  *stream = new SP_Stream_st{h};
  Ok(status);
}
void destroy_stream(const SP_Device*, SP_Stream stream) {
  if (!stream) return;
  itexhip_stream_destroy(stream->stream_handle);
  delete stream;
}
void create_stream_dependency(const SP_Device* device, SP_Stream dependent, SP_Stream other, TF_Status* status) {
  // `dependent` waits for everything already enqueued on `other`
  void* ev = nullptr;
  if (itexhip_event_create(StateOf(device)->ordinal, &ev) != ITEXHIP_OK) return Fail(status, "create_stream_dependency");
  const bool ok = itexhip_event_record(ev, other->stream_handle) == ITEXHIP_OK &&
                  itexhip_stream_wait_event(dependent->stream_handle, ev) == ITEXHIP_OK;
  itexhip_event_destroy(ev);  // the runtime keeps the event alive until the wait has been resolved
  if (!ok) return Fail(status, "create_stream_dependency");
  Ok(status);
}
void get_stream_status(const SP_Device*, SP_Stream stream, TF_Status* status) {
  int done = 0;
  if (itexhip_stream_query(stream->stream_handle, &done) != ITEXHIP_OK) return Fail(status, "get_stream_status");
  Ok(status);
}
void create_event(const SP_Device* device, SP_Event* event, TF_Status* status) {
  void* h = nullptr;
  if (itexhip_event_create(StateOf(device)->ordinal, &h) != ITEXHIP_OK) return Fail(status, "create_event");
  *event = new SP_Event_st{h};
  Ok(status);
}
void destroy_event(const SP_Device*, SP_Event event) {
  if (!event) return;
  itexhip_event_destroy(event->event_handle);
  delete event;
}
SE_EventStatus get_event_status(const SP_Device*, SP_Event event) {
  int done = 0;
  if (itexhip_event_query(event->event_handle, &done) != ITEXHIP_OK) return SE_EVENT_ERROR;
  return done ? SE_EVENT_COMPLETE : SE_EVENT_PENDING;
}
void record_event(const SP_Device*, SP_Stream stream, SP_Event event, TF_Status* status) {
  if (itexhip_event_record(event->event_handle, stream->stream_handle) != ITEXHIP_OK) return Fail(status, "record_event");
  Ok(status);
}
void wait_for_event(const SP_Device* const, SP_Stream stream, SP_Event event, TF_Status* const status) {
  if (itexhip_stream_wait_event(stream->stream_handle, event->event_handle) != ITEXHIP_OK)
    return Fail(status, "wait_for_event");
  Ok(status);
}

void create_timer(const SP_Device*, SP_Timer* timer, TF_Status* status) {
  *timer = nullptr;
  TF_SetStatus(status, TF_UNIMPLEMENTED, "timers are not implemented");
}
void destroy_timer(const SP_Device*, SP_Timer) {}
void start_timer(const SP_Device*, SP_Stream, SP_Timer, TF_Status* status) {
  TF_SetStatus(status, TF_UNIMPLEMENTED, "timers are not implemented");
}
void stop_timer(const SP_Device*, SP_Stream, SP_Timer, TF_Status* status) {
  TF_SetStatus(status, TF_UNIMPLEMENTED, "timers are not implemented");
}
uint64_t timer_nanoseconds(SP_Timer timer) { return timer ? timer->nanoseconds : 0; }

// ---- copies, fills, synchronisation --------------------------------------------------------------
void memcpy_dtoh(const SP_Device*, SP_Stream stream, void* host_dst, const SP_DeviceMemoryBase* device_src, uint64_t size,
                 TF_Status* status) {
  if (itexhip_memcpy_d2h_async(host_dst, device_src->opaque, size, stream->stream_handle) != ITEXHIP_OK)
    return Fail(status, "memcpy_dtoh");
  Ok(status);
}
void memcpy_htod(const SP_Device*, SP_Stream stream, SP_DeviceMemoryBase* device_dst, const void* host_src, uint64_t size,
                 TF_Status* status) {
  if (itexhip_memcpy_h2d_async(device_dst->opaque, host_src, size, stream->stream_handle) != ITEXHIP_OK)
    return Fail(status, "memcpy_htod");
  Ok(status);
}
void memcpy_dtod(const SP_Device*, SP_Stream stream, SP_DeviceMemoryBase* device_dst, const SP_DeviceMemoryBase* device_src,
                 uint64_t size, TF_Status* status) {
  if (itexhip_memcpy_d2d_async(device_dst->opaque, device_src->opaque, size, stream->stream_handle) != ITEXHIP_OK)
    return Fail(status, "memcpy_dtod");
  Ok(status);
}
void sync_memcpy_dtoh(const SP_Device*, void* host_dst, const SP_DeviceMemoryBase* device_src, uint64_t size,
                      TF_Status* status) {
  if (itexhip_memcpy_d2h(host_dst, device_src->opaque, size, nullptr) != ITEXHIP_OK) return Fail(status, "sync_memcpy_dtoh");
  Ok(status);
}
void sync_memcpy_htod(const SP_Device*, SP_DeviceMemoryBase* device_dst, const void* host_src, uint64_t size,
                      TF_Status* status) {
  if (itexhip_memcpy_h2d_async(device_dst->opaque, host_src, size, nullptr) != ITEXHIP_OK ||
      itexhip_stream_synchronize(nullptr) != ITEXHIP_OK)
    return Fail(status, "sync_memcpy_htod");
  Ok(status);
}
void sync_memcpy_dtod(const SP_Device*, SP_DeviceMemoryBase* device_dst, const SP_DeviceMemoryBase* device_src,
                      uint64_t size, TF_Status* status) {
  if (itexhip_memcpy_d2d_async(device_dst->opaque, device_src->opaque, size, nullptr) != ITEXHIP_OK ||
      itexhip_stream_synchronize(nullptr) != ITEXHIP_OK)
    return Fail(status, "sync_memcpy_dtod");
  Ok(status);
}
void block_host_for_event(const SP_Device*, SP_Event event, TF_Status* status) {
  if (itexhip_event_synchronize(event->event_handle) != ITEXHIP_OK) return Fail(status, "block_host_for_event");
  Ok(status);
}
void block_host_until_done(const SP_Device*, SP_Stream stream, TF_Status* status) {
  if (itexhip_stream_synchronize(stream->stream_handle) != ITEXHIP_OK) return Fail(status, "block_host_until_done");
  Ok(status);
}
void synchronize_all_activity(const SP_Device* device, TF_Status* status) {
  if (itexhip_device_synchronize(StateOf(device)->ordinal) != ITEXHIP_OK) return Fail(status, "synchronize_all_activity");
  Ok(status);
}
void mem_zero(const SP_Device*, SP_Stream stream, SP_DeviceMemoryBase* location, uint64_t size, TF_Status* status) {
  if (itexhip_memset8_async(location->opaque, 0, size, stream->stream_handle) != ITEXHIP_OK) return Fail(status, "mem_zero");
  Ok(status);
}
void memset8(const SP_Device*, SP_Stream stream, SP_DeviceMemoryBase* location, uint8_t pattern, uint64_t size,
             TF_Status* status) {
  if (itexhip_memset8_async(location->opaque, pattern, size, stream->stream_handle) != ITEXHIP_OK)
    return Fail(status, "memset");
  Ok(status);
}
void memset32(const SP_Device*, SP_Stream stream, SP_DeviceMemoryBase* location, uint32_t pattern, uint64_t size,
              TF_Status* status) {
  if (itexhip_memset32_async(location->opaque, pattern, size, stream->stream_handle) != ITEXHIP_OK)
    return Fail(status, "memset32");
  Ok(status);
}

struct HostCallback {
  SE_StatusCallbackFn fn;
  void* arg;
};
void RunHostCallback(void* p) {
  std::unique_ptr<HostCallback> cb(static_cast<HostCallback*>(p));
  TF_Status* st = TF_NewStatus();
  cb->fn(cb->arg, st);
  if (TF_GetCode(st) != TF_OK) std::fprintf(stderr, "itex_amd: host callback failed: %s\n", TF_Message(st));
  TF_DeleteStatus(st);
}
TF_Bool host_callback(const SP_Device*, SP_Stream stream, SE_StatusCallbackFn callback_fn, void* callback_arg) {
  auto* cb = new HostCallback{callback_fn, callback_arg};
  if (itexhip_launch_host_func(stream->stream_handle, RunHostCallback, cb) != ITEXHIP_OK) {
    delete cb;
    return 0;
  }
  return 1;
}

void create_stream_executor(const SP_Platform*, SE_CreateStreamExecutorParams* params, TF_Status* status) {
  SP_StreamExecutor* se = params->stream_executor;
  se->struct_size = SP_STREAMEXECUTOR_STRUCT_SIZE;
  se->allocate = allocate;
  se->deallocate = deallocate;
  se->host_memory_allocate = host_memory_allocate;
  se->host_memory_deallocate = host_memory_deallocate;
  se->unified_memory_allocate = nullptr;
  se->unified_memory_deallocate = nullptr;
  se->get_allocator_stats = get_allocator_stats;
  se->device_memory_usage = device_memory_usage;
  se->create_stream = create_stream;
  se->destroy_stream = destroy_stream;
  se->create_stream_dependency = create_stream_dependency;
  se->get_stream_status = get_stream_status;
  se->create_event = create_event;
  se->destroy_event = destroy_event;
  se->get_event_status = get_event_status;
  se->record_event = record_event;
  se->wait_for_event = wait_for_event;
  se->create_timer = create_timer;
  se->destroy_timer = destroy_timer;
  se->start_timer = start_timer;
  se->stop_timer = stop_timer;
  se->memcpy_dtoh = memcpy_dtoh;
  se->memcpy_htod = memcpy_htod;
  se->memcpy_dtod = memcpy_dtod;
  se->sync_memcpy_dtoh = sync_memcpy_dtoh;
  se->sync_memcpy_htod = sync_memcpy_htod;
  se->sync_memcpy_dtod = sync_memcpy_dtod;
  se->block_host_for_event = block_host_for_event;
  se->block_host_until_done = block_host_until_done;
  se->synchronize_all_activity = synchronize_all_activity;
  se->mem_zero = mem_zero;
  se->memset = memset8;
  se->memset32 = memset32;
  se->host_callback = host_callback;
  Ok(status);
}
void destroy_stream_executor(const SP_Platform*, SP_StreamExecutor*) {}

void create_timer_fns(const SP_Platform*, SP_TimerFns* timer_fns, TF_Status* status) {
  timer_fns->struct_size = SP_TIMER_FNS_STRUCT_SIZE;
  timer_fns->nanoseconds = timer_nanoseconds;
  Ok(status);
}
void destroy_timer_fns(const SP_Platform*, SP_TimerFns*) {}
void destroy_platform(SP_Platform*) {}
void destroy_platform_fns(SP_PlatformFns*) {}

}  // namespace
}  // namespace itex_amd

extern "C" void SE_InitPlugin(SE_PlatformRegistrationParams* params, TF_Status* status) {
  using namespace itex_amd;
  params->struct_size = SE_PLATFORM_REGISTRATION_PARAMS_STRUCT_SIZE;
  params->major_version = SE_MAJOR;
  params->minor_version = SE_MINOR;
  params->patch_version = SE_PATCH;
  params->platform->struct_size = SP_PLATFORM_STRUCT_SIZE;
  params->platform->name = DeviceType();
  params->platform->type = DeviceType();
  params->platform->supports_unified_memory = 0;
  params->platform->use_bfc_allocator = 0;
  params->platform->force_memory_growth = 0;
  SP_PlatformFns* fns = params->platform_fns;
  fns->struct_size = SP_PLATFORM_FNS_STRUCT_SIZE;
  fns->get_device_count = get_device_count;
  fns->create_device = create_device;
  fns->destroy_device = destroy_device;
  fns->create_device_fns = create_device_fns;
  fns->destroy_device_fns = destroy_device_fns;
  fns->create_stream_executor = create_stream_executor;
  fns->destroy_stream_executor = destroy_stream_executor;
  fns->create_timer_fns = create_timer_fns;
  fns->destroy_timer_fns = destroy_timer_fns;
  params->destroy_platform = destroy_platform;
  params->destroy_platform_fns = destroy_platform_fns;
  if (status) TF_SetStatus(status, TF_OK, "");
}
