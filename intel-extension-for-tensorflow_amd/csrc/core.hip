// Error reporting and build information of the itexhip C ABI (host only).
#include <stdarg.h>

#include "common.hpp"

namespace itexhip {
namespace {
thread_local char g_error[512] = "";
}

int g_forced_tile_shape[2] = {-1, -1};

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace itexhip

extern "C" const char* itexhip_last_error(void) { return itexhip::g_error; }

extern "C" void itexhip_test_force_tile_shape(int matmul_shape, int conv_shape) {
  __atomic_store_n(&itexhip::g_forced_tile_shape[0], matmul_shape, __ATOMIC_RELAXED);
  __atomic_store_n(&itexhip::g_forced_tile_shape[1], conv_shape, __ATOMIC_RELAXED);
}

extern "C" const char* itexhip_build_info(void) { return "itexhip 0.1 gfx950"; }

extern "C" int itexhip_memcpy_h2d_async(void* dst_device, const void* src_host, size_t bytes, void* stream) {
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(dst_device && src_host, "itexhip_memcpy_h2d_async: null buffer");
  hipError_t e = hipMemcpyAsync(dst_device, src_host, bytes, hipMemcpyHostToDevice, itexhip::as_stream(stream));
  if (e != hipSuccess) return itexhip::hip_fail(e, "itexhip_memcpy_h2d_async");
  return ITEXHIP_OK;
}

extern "C" int itexhip_stream_synchronize(void* stream) {
  hipError_t e = hipStreamSynchronize(itexhip::as_stream(stream));
  if (e != hipSuccess) return itexhip::hip_fail(e, "itexhip_stream_synchronize");
  return ITEXHIP_OK;
}

extern "C" int itexhip_memcpy_d2h(void* dst_host, const void* src_device, size_t bytes, void* stream) {
  if (bytes == 0) return ITEXHIP_OK;
  ITEXHIP_REQUIRE(dst_host && src_device, "itexhip_memcpy_d2h: null buffer");
  hipError_t e = hipMemcpyAsync(dst_host, src_device, bytes, hipMemcpyDeviceToHost, itexhip::as_stream(stream));
  if (e == hipSuccess) e = hipStreamSynchronize(itexhip::as_stream(stream));
  if (e != hipSuccess) return itexhip::hip_fail(e, "itexhip_memcpy_d2h");
  return ITEXHIP_OK;
}
