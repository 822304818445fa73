// Keeps a small host vector mirrored in device memory: the device copy is refreshed (stream-ordered
// copy, no host wait) only when the host values change or grow.  Counterpart of the reference's
// HostDataCache (itex/core/kernels/common/host_data_cache.h:35-95), which blocks on the copy.
#ifndef ITEX_AMD_PLUGIN_DEVICE_VECTOR_CACHE_H_
#define ITEX_AMD_PLUGIN_DEVICE_VECTOR_CACHE_H_

#include <cstring>
#include <vector>

#include "itexhip.h"
#include "op_kernel.h"

namespace itex_amd {

template <typename T>
class DeviceVectorCache {
 public:
  // Returns the device pointer holding `n` values equal to host[0..n); nullptr after a failure
  // (already reported on ctx).
  T* Get(OpKernelContext* ctx, const T* host, size_t n, TF_DataType dtype) {
    const bool same = device_.valid() && host_.size() == n && std::memcmp(host_.data(), host, n * sizeof(T)) == 0;
    changed_ = !same;
    if (same) return device_.flat<T>();
    if (!device_.valid() || capacity_ < n) {
      device_ = ctx->allocate_temp(dtype, {static_cast<int64_t>(n)});
      if (!device_.valid()) return nullptr;
      capacity_ = n;
    }
    // the staging copy must outlive the asynchronous transfer: keep every generation until replaced twice
    retired_.swap(host_);
    host_.assign(host, host + n);
    const int st = itexhip_memcpy_h2d_async(device_.data(), host_.data(), n * sizeof(T), ctx->stream());
    if (st != ITEXHIP_OK) {
      ctx->CtxFailure(static_cast<TF_Code>(st), std::string("Operation received an exception: ") + itexhip_last_error());
      device_.reset();
      host_.clear();
      return nullptr;
    }
    return device_.flat<T>();
  }

  // whether the last Get() had to refresh the device copy
  bool changed() const { return changed_; }

 private:
  bool changed_ = true;
  std::vector<T> host_, retired_;
  Tensor device_;
  size_t capacity_ = 0;
};

}  // namespace itex_amd
#endif  // ITEX_AMD_PLUGIN_DEVICE_VECTOR_CACHE_H_
