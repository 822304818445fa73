/*
 * tf_stream_executor_subset.h - TensorFlow 2.15's StreamExecutor C API for PluggableDevice plugins
 * (tensorflow/c/experimental/stream_executor/stream_executor.h), declared here because TensorFlow's
 * headers are not available to this build.  Field order and types follow that public header; every
 * struct starts with struct_size (+ ext) and is versioned through the *_STRUCT_SIZE macros below, which
 * name the last field like the original.  The reference fills these tables in
 * itex/core/devices/xpu_device.cc:656-693 (SP_StreamExecutor), :772-812 (platform, SE_InitPlugin) and
 * itex/core/devices/gpu/gpu_device_plugin.cc:27-376 (the callbacks).
 * Layout not verified against a real TensorFlow build (none is available here).
 */
#ifndef ITEX_AMD_TF_STREAM_EXECUTOR_SUBSET_H_
#define ITEX_AMD_TF_STREAM_EXECUTOR_SUBSET_H_

#include <stddef.h>
#include <stdint.h>

#include "tf_c_api_subset.h"

#define SE_MAJOR 0
#define SE_MINOR 0
#define SE_PATCH 1

#ifdef __cplusplus
extern "C" {
#endif

typedef unsigned char TF_Bool;

/* SP_Stream is declared in tf_c_api_subset.h (the struct body belongs to the plugin) */
typedef struct SP_Event_st* SP_Event;
typedef struct SP_Timer_st* SP_Timer;
typedef void (*SE_StatusCallbackFn)(void* const arg, TF_Status* const status);

typedef struct SP_TimerFns {
  size_t struct_size;
  void* ext;
  uint64_t (*nanoseconds)(SP_Timer timer);
} SP_TimerFns;
#define SP_TIMER_FNS_STRUCT_SIZE (offsetof(SP_TimerFns, nanoseconds) + sizeof(void*))

typedef struct SP_AllocatorStats {
  size_t struct_size;
  int64_t num_allocs;
  int64_t bytes_in_use;
  int64_t peak_bytes_in_use;
  int64_t largest_alloc_size;
  int8_t has_bytes_limit;
  int64_t bytes_limit;
  int64_t bytes_reserved;
  int64_t peak_bytes_reserved;
  int8_t has_bytes_reservable_limit;
  int64_t bytes_reservable_limit;
  int64_t largest_free_block_bytes;
} SP_AllocatorStats;
#define SP_ALLOCATORSTATS_STRUCT_SIZE (offsetof(SP_AllocatorStats, largest_free_block_bytes) + sizeof(int64_t))

typedef enum SE_EventStatus {
  SE_EVENT_UNKNOWN,
  SE_EVENT_ERROR,
  SE_EVENT_PENDING,
  SE_EVENT_COMPLETE,
} SE_EventStatus;

typedef struct SP_DeviceMemoryBase {
  size_t struct_size;
  void* ext;
  void* opaque; /* device address */
  uint64_t size;
  uint64_t payload;
} SP_DeviceMemoryBase;
#define SP_DEVICE_MEMORY_BASE_STRUCT_SIZE (offsetof(SP_DeviceMemoryBase, payload) + sizeof(uint64_t))

typedef struct SP_Device {
  size_t struct_size;
  void* ext;
  int32_t ordinal;
  void* device_handle;
  const char* hardware_name;
  const char* device_vendor;
  const char* pci_bus_id;
} SP_Device;
#define SP_DEVICE_STRUCT_SIZE (offsetof(SP_Device, pci_bus_id) + sizeof(const char*))

typedef struct SE_CreateDeviceParams {
  size_t struct_size;
  void* ext;
  int32_t ordinal;
  SP_Device* device;
} SE_CreateDeviceParams;
#define SE_CREATE_DEVICE_PARAMS_STRUCT_SIZE (offsetof(SE_CreateDeviceParams, device) + sizeof(SP_Device*))

typedef struct SP_DeviceFns {
  size_t struct_size;
  void* ext;
  int32_t (*get_numa_node)(const SP_Device* device);
  int64_t (*get_memory_bandwidth)(const SP_Device* device);
  double (*get_gflops)(const SP_Device* device);
} SP_DeviceFns;
#define SP_DEVICE_FNS_STRUCT_SIZE (offsetof(SP_DeviceFns, get_gflops) + sizeof(void*))

typedef struct SE_CreateDeviceFnsParams {
  size_t struct_size;
  void* ext;
  SP_DeviceFns* device_fns;
} SE_CreateDeviceFnsParams;
#define SE_CREATE_DEVICE_FNS_PARAMS_STRUCT_SIZE (offsetof(SE_CreateDeviceFnsParams, device_fns) + sizeof(SP_DeviceFns*))

typedef struct SP_StreamExecutor {
  size_t struct_size;
  void* ext;
  void (*allocate)(const SP_Device* device, uint64_t size, int64_t memory_space, SP_DeviceMemoryBase* mem);
  void (*deallocate)(const SP_Device* device, SP_DeviceMemoryBase* memory);
  void* (*host_memory_allocate)(const SP_Device* device, uint64_t size);
  void (*host_memory_deallocate)(const SP_Device* device, void* mem);
  void* (*unified_memory_allocate)(const SP_Device* device, uint64_t bytes);
  void (*unified_memory_deallocate)(const SP_Device* device, void* location);
  TF_Bool (*get_allocator_stats)(const SP_Device* device, SP_AllocatorStats* stats);
  TF_Bool (*device_memory_usage)(const SP_Device* device, int64_t* free, int64_t* total);
  void (*create_stream)(const SP_Device* device, SP_Stream* stream, TF_Status* status);
  void (*destroy_stream)(const SP_Device* device, SP_Stream stream);
  void (*create_stream_dependency)(const SP_Device* device, SP_Stream dependent, SP_Stream other, TF_Status* status);
  void (*get_stream_status)(const SP_Device* device, SP_Stream stream, TF_Status* status);
  void (*create_event)(const SP_Device* device, SP_Event* event, TF_Status* status);
  void (*destroy_event)(const SP_Device* device, SP_Event event);
  SE_EventStatus (*get_event_status)(const SP_Device* device, SP_Event event);
  void (*record_event)(const SP_Device* device, SP_Stream stream, SP_Event event, TF_Status* status);
  void (*wait_for_event)(const SP_Device* const device, SP_Stream stream, SP_Event event, TF_Status* const status);
  void (*create_timer)(const SP_Device* device, SP_Timer* timer, TF_Status* status);
  void (*destroy_timer)(const SP_Device* device, SP_Timer timer);
  void (*start_timer)(const SP_Device* device, SP_Stream stream, SP_Timer timer, TF_Status* status);
  void (*stop_timer)(const SP_Device* device, SP_Stream stream, SP_Timer timer, TF_Status* status);
  void (*memcpy_dtoh)(const SP_Device* device, SP_Stream stream, void* host_dst, const SP_DeviceMemoryBase* device_src,
                      uint64_t size, TF_Status* status);
  void (*memcpy_htod)(const SP_Device* device, SP_Stream stream, SP_DeviceMemoryBase* device_dst, const void* host_src,
                      uint64_t size, TF_Status* status);
  void (*memcpy_dtod)(const SP_Device* device, SP_Stream stream, SP_DeviceMemoryBase* device_dst,
                      const SP_DeviceMemoryBase* device_src, uint64_t size, TF_Status* status);
  void (*sync_memcpy_dtoh)(const SP_Device* device, void* host_dst, const SP_DeviceMemoryBase* device_src, uint64_t size,
                           TF_Status* status);
  void (*sync_memcpy_htod)(const SP_Device* device, SP_DeviceMemoryBase* device_dst, const void* host_src, uint64_t size,
                           TF_Status* status);
  void (*sync_memcpy_dtod)(const SP_Device* device, SP_DeviceMemoryBase* device_dst, const SP_DeviceMemoryBase* device_src,
                           uint64_t size, TF_Status* status);
  void (*block_host_for_event)(const SP_Device* device, SP_Event event, TF_Status* status);
  void (*block_host_until_done)(const SP_Device* device, SP_Stream stream, TF_Status* status);
  void (*synchronize_all_activity)(const SP_Device* device, TF_Status* status);
  void (*mem_zero)(const SP_Device* device, SP_Stream stream, SP_DeviceMemoryBase* location, uint64_t size,
                   TF_Status* status);
  void (*memset)(const SP_Device* device, SP_Stream stream, SP_DeviceMemoryBase* location, uint8_t pattern, uint64_t size,
                 TF_Status* status);
  void (*memset32)(const SP_Device* device, SP_Stream stream, SP_DeviceMemoryBase* location, uint32_t pattern,
                   uint64_t size, TF_Status* status);
  TF_Bool (*host_callback)(const SP_Device* device, SP_Stream stream, SE_StatusCallbackFn callback_fn, void* callback_arg);
} SP_StreamExecutor;
#define SP_STREAMEXECUTOR_STRUCT_SIZE (offsetof(SP_StreamExecutor, host_callback) + sizeof(void*))

typedef struct SE_CreateStreamExecutorParams {
  size_t struct_size;
  void* ext;
  SP_StreamExecutor* stream_executor;
} SE_CreateStreamExecutorParams;
#define SE_CREATE_STREAM_EXECUTOR_PARAMS_STRUCT_SIZE \
  (offsetof(SE_CreateStreamExecutorParams, stream_executor) + sizeof(SP_StreamExecutor*))

typedef struct SP_Platform {
  size_t struct_size;
  void* ext;
  const char* name; /* e.g. "XPU" */
  const char* type; /* device type string used in kernel registration */
  TF_Bool supports_unified_memory;
  TF_Bool use_bfc_allocator; /* let TensorFlow put its own BFC allocator on top of allocate() */
  TF_Bool force_memory_growth;
} SP_Platform;
#define SP_PLATFORM_STRUCT_SIZE (offsetof(SP_Platform, force_memory_growth) + sizeof(TF_Bool))

typedef struct SP_PlatformFns {
  size_t struct_size;
  void* ext;
  void (*get_device_count)(const SP_Platform* platform, int* device_count, TF_Status* status);
  void (*create_device)(const SP_Platform* platform, SE_CreateDeviceParams* params, TF_Status* status);
  void (*destroy_device)(const SP_Platform* platform, SP_Device* device);
  void (*create_device_fns)(const SP_Platform* platform, SE_CreateDeviceFnsParams* params, TF_Status* status);
  void (*destroy_device_fns)(const SP_Platform* platform, SP_DeviceFns* device_fns);
  void (*create_stream_executor)(const SP_Platform* platform, SE_CreateStreamExecutorParams* params, TF_Status* status);
  void (*destroy_stream_executor)(const SP_Platform* platform, SP_StreamExecutor* stream_executor);
  void (*create_timer_fns)(const SP_Platform* platform, SP_TimerFns* timer, TF_Status* status);
  void (*destroy_timer_fns)(const SP_Platform* platform, SP_TimerFns* timer_fns);
} SP_PlatformFns;
#define SP_PLATFORM_FNS_STRUCT_SIZE (offsetof(SP_PlatformFns, destroy_timer_fns) + sizeof(void*))

typedef struct SE_PlatformRegistrationParams {
  size_t struct_size;
  void* ext;
  int32_t major_version;
  int32_t minor_version;
  int32_t patch_version;
  SP_Platform* platform;
  SP_PlatformFns* platform_fns;
  void (*destroy_platform)(SP_Platform* platform);
  void (*destroy_platform_fns)(SP_PlatformFns* platform_fns);
} SE_PlatformRegistrationParams;
#define SE_PLATFORM_REGISTRATION_PARAMS_STRUCT_SIZE \
  (offsetof(SE_PlatformRegistrationParams, destroy_platform_fns) + sizeof(void*))

/* The plugin's entry point, looked up by TensorFlow after dlopen (itex/core/devices/xpu_device.cc:793-812). */
void SE_InitPlugin(SE_PlatformRegistrationParams* params, TF_Status* status);

#ifdef __cplusplus
}
#endif
#endif /* ITEX_AMD_TF_STREAM_EXECUTOR_SUBSET_H_ */
