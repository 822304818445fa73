// Dequantize / _ITEXDequantize op kernel (itex/core/kernels/common/dequantize_op.h:43-186).
#include <mutex>
#include <string>
#include <vector>

#include "device_vector_cache.h"
#include "itexhip.h"
#include "op_kernel.h"
#include "qparams.h"

namespace itex_amd {
namespace {

using qparams::Mode;

class DequantizeOp : public OpKernel {
 public:
  DequantizeOp(OpKernelConstruction* ctx, TF_DataType T) : T_(T) {
    std::string mode_string;
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("mode", &mode_string));
    ITEX_REQUIRES(ctx, (mode_string == "MIN_COMBINED" || mode_string == "MIN_FIRST" || mode_string == "SCALED"),
                  TF_INVALID_ARGUMENT,
                  "Mode string must be 'MIN_COMBINED', 'MIN_FIRST', or 'SCALED', is '" + mode_string + "'");
    // The reference constructor lets MIN_COMBINED through and then computes with a zero scale (its
    // graph pass never sends that mode here, itex/core/graph/utils/layout_utils.cc:315-355); refuse it.
    ITEX_REQUIRES(ctx, mode_string != "MIN_COMBINED", TF_UNIMPLEMENTED,
                  "Dequantize on this device supports SCALED and MIN_FIRST mode only");
    mode_ = mode_string == "MIN_FIRST" ? Mode::MIN_FIRST : Mode::SCALED;
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("narrow_range", &narrow_range_));
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("axis", &axis_));
    if (ctx->HasAttr("dtype")) {
      TF_DataType dtype = TF_FLOAT;
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("dtype", &dtype));
      ITEX_REQUIRES(ctx, dtype == TF_FLOAT || dtype == TF_BFLOAT16 || dtype == TF_HALF, TF_INVALID_ARGUMENT,
                    "Dequantize produces float, bfloat16 or half");
      dst_type_ = dtype;
    }
  }

  void Compute(OpKernelContext* ctx) override {
    // one Compute at a time per node: the cached device vectors below are reassigned in place, and TensorFlow may run
    // one node from several threads (the reference serialises its kernels the same way, conv_ops.h:786,
    // quantized_matmul_common.h:62)
    std::lock_guard<std::mutex> lock(mu_);
    Tensor src = ctx->input(0);
    Tensor in_min = ctx->input(1);
    Tensor in_max = ctx->input(2);
    if (!ctx->ok()) return;
    const int64_t num_slices = (axis_ > -1) ? in_min.NumElements() : 1;
    ITEX_REQUIRES(ctx, in_min.NumElements() >= 1 && in_max.NumElements() >= num_slices, TF_INVALID_ARGUMENT,
                  "min_range and max_range must hold one value per slice");
    std::vector<float> scale(num_slices);
    std::vector<int32_t> zp(num_slices);
    for (int64_t i = 0; i < num_slices; ++i) {
      float mn = in_min.flat<float>()[i], mx = in_max.flat<float>()[i];  // no range adjustment here
      qparams::ScaleZeroPoint(T_, mode_, /*dequantize=*/true, &mn, &mx, &scale[i], &zp[i]);
      if (mode_ != Mode::MIN_FIRST) zp[i] = 0;
    }
    const std::vector<int64_t> shape = src.shape();
    Tensor dst = ctx->allocate_output(0, dst_type_, shape);
    if (!ctx->ok()) return;
    int st;
    if (num_slices == 1) {
      st = dst_type_ == TF_FLOAT
               ? itexhip_dequantize(src.data(), dst.flat<float>(), src.NumElements(), T_, scale[0], zp[0], ctx->stream())
               : itexhip_dequantize16(src.data(), dst.data(), src.NumElements(), T_, dst_type_, scale[0], zp[0], ctx->stream());
    } else {
      ITEX_REQUIRES(ctx, axis_ < static_cast<int>(shape.size()) && shape[axis_] == num_slices, TF_INVALID_ARGUMENT,
                    "min_range has " + std::to_string(num_slices) + " entries but dimension " + std::to_string(axis_) +
                        " of the input does not");
      int64_t outer = 1, inner = 1;
      for (int d = 0; d < axis_; ++d) outer *= shape[d];
      for (size_t d = axis_ + 1; d < shape.size(); ++d) inner *= shape[d];
      float* sc_dev = scales_.Get(ctx, scale.data(), scale.size(), TF_FLOAT);
      int32_t* zp_dev = zps_.Get(ctx, zp.data(), zp.size(), TF_INT32);
      if (sc_dev == nullptr || zp_dev == nullptr) return;
      st = dst_type_ == TF_FLOAT
               ? itexhip_dequantize_axis(src.data(), dst.flat<float>(), outer, num_slices, inner, T_, sc_dev, zp_dev,
                                         ctx->stream())
               : itexhip_dequantize_axis16(src.data(), dst.data(), outer, num_slices, inner, T_, dst_type_, sc_dev, zp_dev,
                                           ctx->stream());
    }
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                  std::string("Operation received an exception: ") + itexhip_last_error());
  }

 private:
  TF_DataType T_;
  TF_DataType dst_type_ = TF_FLOAT;
  Mode mode_ = Mode::SCALED;
  bool narrow_range_ = false;
  int32_t axis_ = -1;
  std::mutex mu_;
  DeviceVectorCache<float> scales_;
  DeviceVectorCache<int32_t> zps_;
};

struct DequantizeQint8 : DequantizeOp { explicit DequantizeQint8(OpKernelConstruction* c) : DequantizeOp(c, TF_QINT8) {} };
struct DequantizeQuint8 : DequantizeOp { explicit DequantizeQuint8(OpKernelConstruction* c) : DequantizeOp(c, TF_QUINT8) {} };

}  // namespace

// itex/core/kernels/gpu/dequantize_op.cc:24-48 (device: "Dequantize"); the _ITEX name is what the CPU
// graph pass renames to (itex/core/kernels/cpu/dequantize_op.cc:22-40) and is registered too so that
// such graphs stay placeable.
void AddDequantizeKernels() {
  for (const char* op : {"Dequantize", "_ITEXDequantize"}) {
    for (TF_DataType dtype : {TF_FLOAT, TF_BFLOAT16, TF_HALF}) {
      KernelDefBuilder s(op, "DequantizeOp");
      s.TypeConstraint("T", TF_QINT8).TypeConstraint("dtype", dtype).HostMemory("min_range").HostMemory("max_range");
      s.Register<DequantizeQint8>();
      KernelDefBuilder u(op, "DequantizeOp");
      u.TypeConstraint("T", TF_QUINT8).TypeConstraint("dtype", dtype).HostMemory("min_range").HostMemory("max_range");
      u.Register<DequantizeQuint8>();
    }
  }
}

}  // namespace itex_amd
