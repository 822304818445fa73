// QuantizeV2 / _ITEXQuantizeV2 op kernel: attribute parsing, host-side range math and output range
// conventions as in the reference (itex/core/kernels/common/quantize_op.h:68-430), the quantization
// itself on the GPU through itexhip_quantize / itexhip_quantize_axis.
#include <mutex>
#include <cmath>
#include <string>
#include <vector>

#include "device_vector_cache.h"
#include "itexhip.h"
#include "op_kernel.h"
#include "qparams.h"

namespace itex_amd {
namespace {

using qparams::Mode;

class QuantizeV2Op : public OpKernel {
 public:
  // dynamic: the op has no min_range / max_range inputs and takes the range of its input tensor, computed on the device
  // (what the graph pass makes of Reshape -> Min / Max -> QuantizeV2; no counterpart in the reference, whose QuantizeV2
  // always receives the range from other ops)
  QuantizeV2Op(OpKernelConstruction* ctx, TF_DataType T, bool dynamic = false) : T_(T), dynamic_(dynamic) {
    std::string mode_string;
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("mode", &mode_string));
    if (ctx->HasAttr("classic_asymmetric_algorithm")) {
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("classic_asymmetric_algorithm", &classic_));
    }
    ITEX_REQUIRES(ctx, (mode_string == "MIN_COMBINED" || mode_string == "MIN_FIRST" || mode_string == "SCALED"),
                  TF_INVALID_ARGUMENT,
                  "Mode string must be 'MIN_COMBINED', 'MIN_FIRST', or 'SCALED', is '" + mode_string + "'");
    mode_ = mode_string == "MIN_COMBINED" ? Mode::MIN_COMBINED : mode_string == "MIN_FIRST" ? Mode::MIN_FIRST : Mode::SCALED;
    ITEX_REQUIRES(ctx, (mode_string == "SCALED" || mode_string == "MIN_FIRST"), TF_INVALID_ARGUMENT,
                  "_ITEXQuantizeV2 only supports SCALED and MIN_FIRST MODE");
    std::string round_mode_string;
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("round_mode", &round_mode_string));
    ITEX_REQUIRES(ctx, (round_mode_string == "HALF_AWAY_FROM_ZERO" || round_mode_string == "HALF_TO_EVEN"),
                  TF_INVALID_ARGUMENT,
                  "Round mode string must be 'HALF_AWAY_FROM_ZERO' or 'HALF_TO_EVEN', is '" + round_mode_string + "'");
    if (round_mode_string == "HALF_TO_EVEN") {
      ITEX_REQUIRES(ctx, mode_string == "SCALED", TF_INVALID_ARGUMENT,
                    "Round mode 'HALF_TO_EVEN' only supported for mode 'SCALED', but mode is '" + mode_string + "'.");
    }
    // narrow_range is read and, as in the reference, has no effect; rounding is to nearest even in
    // every mode
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("narrow_range", &narrow_range_));
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("axis", &axis_));
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("ensure_minimum_range", &ensure_minimum_range_));
    if (ctx->HasAttr("dtype")) {
      TF_DataType dtype = TF_FLOAT;
      ITEX_REQUIRES_OK(ctx, ctx->GetAttr("dtype", &dtype));
      ITEX_REQUIRES(ctx, dtype == TF_FLOAT || dtype == TF_BFLOAT16, TF_UNIMPLEMENTED,
                    "_ITEXQuantizeV2 on this device takes float or bfloat16 input");
      src_type_ = dtype;
    }
  }

  void Compute(OpKernelContext* ctx) override {
    // one Compute at a time per node: the cached device vectors below are reassigned in place, and TensorFlow may run
    // one node from several threads (the reference serialises its kernels the same way, conv_ops.h:786,
    // quantized_matmul_common.h:62)
    std::lock_guard<std::mutex> lock(mu_);
    Tensor src = ctx->input(0);
    if (!ctx->ok()) return;
    ITEX_REQUIRES(ctx, src.dtype() == src_type_, TF_INVALID_ARGUMENT, "QuantizeV2 input type does not match the kernel");
    Tensor in_min, in_max;
    if (dynamic_) {
      ITEX_REQUIRES(ctx, axis_ == -1 && src_type_ == TF_FLOAT, TF_INVALID_ARGUMENT,
                    "the dynamic-range QuantizeV2 quantizes a float tensor per tensor");
      // reduction, parameter math and quantization are enqueued back to back (itexhip_quantize_dynamic) and the host
      // only waits once, at the end, for the two floats of the output range.  (The legacy MIN_FIRST algorithm to
      // qint8 takes the path below: range to the host, then QuantizeV2 as usual.)
      const bool device_params = src.NumElements() > 0 &&
                                 (mode_ == Mode::SCALED || (mode_ == Mode::MIN_FIRST && (classic_ || T_ == TF_QUINT8)));
      if (device_params) {
        Tensor dst = ctx->allocate_output(0, T_, src.shape());
        Tensor out_min = ctx->allocate_output(1, TF_FLOAT, {});
        Tensor out_max = ctx->allocate_output(2, TF_FLOAT, {});
        Tensor state = ctx->allocate_temp(TF_FLOAT, {ITEXHIP_DYNAMIC_STATE_FLOATS});
        if (!ctx->ok()) return;
        float range[2] = {0.0f, 0.0f};
        int st = itexhip_quantize_dynamic(src.flat<float>(), dst.data(), src.NumElements(), T_,
                                          mode_ == Mode::SCALED ? ITEXHIP_SCALED : classic_ ? ITEXHIP_MIN_FIRST_CLASSIC : ITEXHIP_MIN_FIRST,
                                          ensure_minimum_range_,
                                          state.flat<float>(), ctx->stream());
        if (st == ITEXHIP_OK) st = itexhip_memcpy_d2h(range, state.flat<float>() + 2, sizeof(range), ctx->stream());
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
        out_min.flat<float>()[0] = range[0];
        out_max.flat<float>()[0] = range[1];
        return;
      }
      in_min = ctx->allocate_temp(TF_FLOAT, {}, /*on_host=*/true);
      in_max = ctx->allocate_temp(TF_FLOAT, {}, /*on_host=*/true);
      Tensor range = ctx->allocate_temp(TF_FLOAT, {2});
      if (!ctx->ok()) return;
      float host_range[2] = {0.0f, 0.0f};  // the range of an empty tensor, as Min / Max give no usable value there
      if (src.NumElements() > 0) {
        int st = itexhip_minmax_f32(src.flat<float>(), src.NumElements(), range.flat<float>(), ctx->stream());
        if (st == ITEXHIP_OK) st = itexhip_memcpy_d2h(host_range, range.data(), sizeof(host_range), ctx->stream());
        ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
      }
      in_min.flat<float>()[0] = host_range[0];
      in_max.flat<float>()[0] = host_range[1];
    } else {
      in_min = ctx->input(1);
      in_max = ctx->input(2);
      if (!ctx->ok()) return;
    }

    const int64_t num_slices = (axis_ > -1) ? in_min.NumElements() : 1;
    ITEX_REQUIRES(ctx, in_min.NumElements() >= 1 && in_max.NumElements() >= num_slices, TF_INVALID_ARGUMENT,
                  "min_range and max_range must hold one value per slice");
    std::vector<float> mn(num_slices), mx(num_slices), scale(num_slices), addend(num_slices, 0.0f);
    for (int64_t i = 0; i < num_slices; ++i) {
      ITEX_REQUIRES(ctx, qparams::AdjustRange(in_min.flat<float>()[i], in_max.flat<float>()[i], ensure_minimum_range_,
                                              &mn[i], &mx[i]),
                    TF_INVALID_ARGUMENT, "input_max_range must be larger than input_min_range.");
    }
    const bool legacy = mode_ == Mode::MIN_FIRST && !classic_;
    for (int64_t i = 0; i < num_slices; ++i) {
      if (!legacy) {
        int32_t zp = 0;
        qparams::ScaleZeroPoint(T_, mode_, /*dequantize=*/false, &mn[i], &mx[i], &scale[i], &zp);
        addend[i] = (mode_ == Mode::MIN_FIRST) ? static_cast<float>(zp) : 0.0f;  // destination zero point
      } else {
        scale[i] = qparams::LegacyMinFirstScale(T_, mn[i], mx[i]);
        const float shift = -mn[i];
        addend[i] = shift * scale[i];  // second source of the scaled binary add
      }
    }

    const std::vector<int64_t> shape = src.shape();
    int64_t outer = 1, slices = 1, inner = 1;
    if (num_slices > 1) {
      ITEX_REQUIRES(ctx, axis_ < static_cast<int>(shape.size()) && shape[axis_] == num_slices, TF_INVALID_ARGUMENT,
                    "min_range has " + std::to_string(num_slices) + " entries but dimension " + std::to_string(axis_) +
                        " of the input does not");
      for (int d = 0; d < axis_; ++d) outer *= shape[d];
      slices = shape[axis_];
      for (size_t d = axis_ + 1; d < shape.size(); ++d) inner *= shape[d];
    }

    Tensor dst = ctx->allocate_output(0, T_, shape);
    const std::vector<int64_t> mm_shape = (num_slices == 1) ? std::vector<int64_t>{} : in_min.shape();
    Tensor out_min = dynamic_ ? ctx->allocate_output(1, TF_FLOAT, mm_shape) : ctx->forward_input_or_allocate_output(1, 1, mm_shape, TF_FLOAT);
    Tensor out_max = dynamic_ ? ctx->allocate_output(2, TF_FLOAT, mm_shape) : ctx->forward_input_or_allocate_output(2, 2, mm_shape, TF_FLOAT);
    if (!ctx->ok()) return;

    int st;
    if (num_slices == 1) {
      st = src_type_ == TF_BFLOAT16
               ? itexhip_quantize_bf16(src.data(), dst.data(), src.NumElements(), T_, scale[0], addend[0], ctx->stream())
               : itexhip_quantize(src.flat<float>(), dst.data(), src.NumElements(), T_, scale[0], addend[0], ctx->stream());
    } else {
      std::vector<float> both(scale);
      both.insert(both.end(), addend.begin(), addend.end());
      float* dev = params_.Get(ctx, both.data(), both.size(), TF_FLOAT);
      if (dev == nullptr) return;
      st = src_type_ == TF_BFLOAT16
               ? itexhip_quantize_axis_bf16(src.data(), dst.data(), outer, slices, inner, T_, dev, dev + num_slices,
                                            ctx->stream())
               : itexhip_quantize_axis(src.flat<float>(), dst.data(), outer, slices, inner, T_, dev, dev + num_slices,
                                       ctx->stream());
    }
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                  std::string("Operation received an exception: ") + itexhip_last_error());

    // output ranges; the outputs may alias the inputs, which were consumed above
    for (int64_t i = 0; i < num_slices; ++i) {
      if (T_ == TF_QUINT8 && mode_ == Mode::SCALED) {
        out_min.flat<float>()[i] = 0.0f;
        out_max.flat<float>()[i] = mx[i];
      } else {
        out_min.flat<float>()[i] = mn[i];
        out_max.flat<float>()[i] = mx[i];
      }
    }
  }

 private:
  TF_DataType T_;
  bool dynamic_ = false;
  TF_DataType src_type_ = TF_FLOAT;
  Mode mode_ = Mode::SCALED;
  bool classic_ = false;
  bool narrow_range_ = false;
  int32_t axis_ = -1;
  float ensure_minimum_range_ = 0.01f;
  std::mutex mu_;
  DeviceVectorCache<float> params_;
};

struct QuantizeQint8 : QuantizeV2Op { explicit QuantizeQint8(OpKernelConstruction* c) : QuantizeV2Op(c, TF_QINT8) {} };
struct QuantizeQuint8 : QuantizeV2Op { explicit QuantizeQuint8(OpKernelConstruction* c) : QuantizeV2Op(c, TF_QUINT8) {} };
struct DynQuantizeQint8 : QuantizeV2Op { explicit DynQuantizeQint8(OpKernelConstruction* c) : QuantizeV2Op(c, TF_QINT8, true) {} };
struct DynQuantizeQuint8 : QuantizeV2Op { explicit DynQuantizeQuint8(OpKernelConstruction* c) : QuantizeV2Op(c, TF_QUINT8, true) {} };

}  // namespace

// names and host-memory arguments as registered by the reference for a device
// (itex/core/kernels/gpu/quantize_op.cc:24-51)
void AddQuantizeKernels() {
  for (const char* op : {"QuantizeV2", "_ITEXQuantizeV2"}) {
    const bool itex = op[0] == '_';
    KernelDefBuilder s8(op, "QuantizeV2Op");
    s8.TypeConstraint("T", TF_QINT8);
    if (itex) s8.TypeConstraint("dtype", TF_FLOAT);
    s8.HostMemory("min_range").HostMemory("max_range").HostMemory("output_min").HostMemory("output_max");
    s8.Register<QuantizeQint8>();
    KernelDefBuilder u8(op, "QuantizeV2Op");
    u8.TypeConstraint("T", TF_QUINT8);
    if (itex) u8.TypeConstraint("dtype", TF_FLOAT);
    u8.HostMemory("min_range").HostMemory("max_range").HostMemory("output_min").HostMemory("output_max");
    u8.Register<QuantizeQuint8>();
  }
  // _ITEXQuantizeV2 from a bfloat16 tensor (:38-51)
  KernelDefBuilder bs8("_ITEXQuantizeV2", "QuantizeV2Op");
  bs8.TypeConstraint("T", TF_QINT8).TypeConstraint("dtype", TF_BFLOAT16);
  bs8.HostMemory("min_range").HostMemory("max_range").HostMemory("output_min").HostMemory("output_max");
  bs8.Register<QuantizeQint8>();
  KernelDefBuilder bu8("_ITEXQuantizeV2", "QuantizeV2Op");
  bu8.TypeConstraint("T", TF_QUINT8).TypeConstraint("dtype", TF_BFLOAT16);
  bu8.HostMemory("min_range").HostMemory("max_range").HostMemory("output_min").HostMemory("output_max");
  bu8.Register<QuantizeQuint8>();
  // the dynamic-range form made by this plugin's graph pass
  KernelDefBuilder ds8("_ITEXQuantizeV2DynamicRange", "QuantizeV2Op");
  ds8.TypeConstraint("T", TF_QINT8).TypeConstraint("dtype", TF_FLOAT).HostMemory("output_min").HostMemory("output_max");
  ds8.Register<DynQuantizeQint8>();
  KernelDefBuilder du8("_ITEXQuantizeV2DynamicRange", "QuantizeV2Op");
  du8.TypeConstraint("T", TF_QUINT8).TypeConstraint("dtype", TF_FLOAT).HostMemory("output_min").HostMemory("output_max");
  du8.Register<DynQuantizeQuint8>();
}

}  // namespace itex_amd
