// RequantizePerChannel and RequantizationRangePerChannel op kernels
// (itex/core/kernels/onednn/block/requantize_per_channel_op.cc:34-191,
//  itex/core/kernels/onednn/block/requantization_range_per_channel_op.cc:32-184).
#include <cmath>
#include <cstdlib>
#include <limits>
#include <mutex>
#include <string>
#include <vector>

#include "device_vector_cache.h"
#include "itexhip.h"
#include "op_kernel.h"

namespace itex_amd {
namespace {

class RequantizePerChannelOp : public OpKernel {
 public:
  RequantizePerChannelOp(OpKernelConstruction* ctx, TF_DataType out) : out_type_(out) {
    TF_DataType t = out;
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("out_type", &t));
    ITEX_REQUIRES(ctx, t == TF_QINT8 || t == TF_QUINT8, TF_INVALID_ARGUMENT,
                  "out_type must be qint8 or quint8, but got: " + std::to_string(static_cast<int>(t)));
    out_type_ = t;
  }
  void Compute(OpKernelContext* ctx) override {
    // one Compute at a time per node: the cached scale vector is reassigned in place
    std::lock_guard<std::mutex> lock(mu_);
    Tensor input = ctx->input(0), in_min = ctx->input(1), in_max = ctx->input(2);
    Tensor req_min = ctx->input(3), req_max = ctx->input(4);
    if (!ctx->ok()) return;
    const int64_t depth = in_min.NumElements();
    ITEX_REQUIRES(ctx, input.dims() == 4, TF_INVALID_ARGUMENT, "Current RequantizePerChannel operatorsupports 4D tensors only.");
    ITEX_REQUIRES(ctx, in_max.NumElements() == depth, TF_INVALID_ARGUMENT,
                  "input_max has incorrect size, expected " + std::to_string(depth) + " was " + std::to_string(in_max.NumElements()));
    ITEX_REQUIRES(ctx, input.dim_size(3) == depth, TF_INVALID_ARGUMENT,
                  "input_min has incorrect size, expected " + std::to_string(input.dim_size(3)) + " was " + std::to_string(depth));
    const float rmin = req_min.flat<float>()[0], rmax = req_max.flat<float>()[0];
    const float factor = (out_type_ == TF_QINT8) ? 127.0f : 255.0f;
    const float requested_min_max = std::max(std::fabs(rmin), std::fabs(rmax));
    std::vector<float> scales(depth);
    for (int64_t i = 0; i < depth; ++i) {
      const float min_max_from_vec = std::max(std::fabs(in_min.flat<float>()[i]), std::fabs(in_max.flat<float>()[i]));
      scales[i] = factor * (min_max_from_vec / requested_min_max / 2147483648.0f);
    }
    Tensor out = ctx->allocate_output(0, out_type_, input.shape());
    if (!ctx->ok()) return;
    float* sc_dev = scales_.Get(ctx, scales.data(), scales.size(), TF_FLOAT);
    if (sc_dev == nullptr) return;
    const int st = itexhip_requantize_per_channel(input.flat<int32_t>(), out.data(), input.NumElements() / std::max<int64_t>(depth, 1),
                                                  depth, out_type_, sc_dev, ctx->stream());
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
    Tensor omin = ctx->allocate_output(1, TF_FLOAT, {});
    Tensor omax = ctx->allocate_output(2, TF_FLOAT, {});
    if (!ctx->ok()) return;
    omin.flat<float>()[0] = rmin;
    omax.flat<float>()[0] = rmax;
  }

 private:
  TF_DataType out_type_;
  std::mutex mu_;
  DeviceVectorCache<float> scales_;
};
struct RequantizeS8 : RequantizePerChannelOp { explicit RequantizeS8(OpKernelConstruction* c) : RequantizePerChannelOp(c, TF_QINT8) {} };
struct RequantizeU8 : RequantizePerChannelOp { explicit RequantizeU8(OpKernelConstruction* c) : RequantizePerChannelOp(c, TF_QUINT8) {} };

class RequantizationRangePerChannelOp : public OpKernel {
 public:
  explicit RequantizationRangePerChannelOp(OpKernelConstruction* ctx) {
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("clip_value_max", &clip_value_max_));
  }
  void Compute(OpKernelContext* ctx) override {
    Tensor input = ctx->input(0), in_min = ctx->input(1), in_max = ctx->input(2);
    if (!ctx->ok()) return;
    const int64_t depth = in_max.NumElements();
    ITEX_REQUIRES(ctx, in_min.NumElements() == depth, TF_INVALID_ARGUMENT,
                  "input_min has incorrect size, expected " + std::to_string(depth) + " was " + std::to_string(in_min.NumElements()));
    ITEX_REQUIRES(ctx, input.dims() >= 1 && input.dim_size(input.dims() - 1) == depth, TF_INVALID_ARGUMENT,
                  "input_max has incorrect size, expected " + std::to_string(input.dims() ? input.dim_size(input.dims() - 1) : 0) +
                      " was " + std::to_string(depth));
    // The per-channel extrema are reduced on the device in one pass; the 2*depth integers then cross to
    // the host once (the reference copies two scalars per channel, waiting each time, :110-127).
    Tensor mm_dev = ctx->allocate_temp(TF_INT32, {2 * depth});
    if (!ctx->ok()) return;
    int32_t* mn_dev = mm_dev.flat<int32_t>();
    int st = itexhip_minmax_i32_per_channel(input.flat<int32_t>(), input.NumElements() / std::max<int64_t>(depth, 1), depth,
                                            mn_dev, mn_dev + depth, ctx->stream());
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
    std::vector<int32_t> mm(2 * depth);
    st = itexhip_memcpy_d2h(mm.data(), mn_dev, mm.size() * sizeof(int32_t), ctx->stream());
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());

    float out_min_max = std::numeric_limits<float>::min();
    bool is_non_negative = true;
    for (int64_t i = 0; i < depth; ++i) {
      const int32_t mn = mm[i], mx = mm[depth + i];
      // |INT32_MIN| is not representable; the reference's std::abs wraps to INT32_MIN there
      const int32_t amn = mn == std::numeric_limits<int32_t>::min() ? mn : std::abs(mn);
      const int32_t amx = mx == std::numeric_limits<int32_t>::min() ? mx : std::abs(mx);
      const int32_t abs_max = std::max(amn, amx);
      const float scale = std::max(std::fabs(in_min.flat<float>()[i]), std::fabs(in_max.flat<float>()[i]));
      const float range = scale * static_cast<float>(abs_max) / 2147483648.0f;
      if (mn < 0) is_non_negative = false;
      out_min_max = std::max(out_min_max, range);
    }
    if (out_min_max > clip_value_max_) out_min_max = clip_value_max_;
    Tensor omin = ctx->allocate_output(0, TF_FLOAT, {});
    Tensor omax = ctx->allocate_output(1, TF_FLOAT, {});
    if (!ctx->ok()) return;
    omin.flat<float>()[0] = is_non_negative ? 0.0f : -out_min_max;
    omax.flat<float>()[0] = out_min_max;
  }

 private:
  float clip_value_max_ = std::numeric_limits<float>::infinity();
};

}  // namespace

void AddRequantizeKernels() {
  KernelDefBuilder s8("RequantizePerChannel", "OneDnnRequantizePerChannelOp");
  s8.TypeConstraint("T", TF_QINT32).TypeConstraint("out_type", TF_QINT8);
  for (const char* h : {"input_min", "input_max", "requested_output_min", "requested_output_max", "output_min", "output_max"})
    s8.HostMemory(h);
  s8.Register<RequantizeS8>();
  KernelDefBuilder u8("RequantizePerChannel", "OneDnnRequantizePerChannelOp");
  u8.TypeConstraint("T", TF_QINT32).TypeConstraint("out_type", TF_QUINT8);
  for (const char* h : {"input_min", "input_max", "requested_output_min", "requested_output_max", "output_min", "output_max"})
    u8.HostMemory(h);
  u8.Register<RequantizeU8>();
  KernelDefBuilder r("RequantizationRangePerChannel", "OneDnnRequantizationRangePerChannelOp");
  r.TypeConstraint("T", TF_QINT32);
  for (const char* h : {"input_min", "input_max", "output_min", "output_max"}) r.HostMemory(h);
  r.Register<RequantizationRangePerChannelOp>();
}

}  // namespace itex_amd
