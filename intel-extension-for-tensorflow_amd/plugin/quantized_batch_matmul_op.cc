// _QuantizedBatchMatMul, _QuantizedBatchMatMulV2AndDequantize and _QuantizedFusedBatchMatMulV2AndDequantize
// op kernels: the host half of itex/core/kernels/common/batch_matmul_op.h (BatchMatMulOp::Init :88-273,
// GetPrimitiveDesc :361-419, QuantizedBatchMatMulV2Op :439-522) - attribute parsing, input indices, shape
// and broadcast resolution, the output scale - with the product itself in one itexhip_qbatch_matmul launch.
#include <algorithm>
#include <cmath>
#include <string>
#include <vector>

#include "itexhip.h"
#include "op_kernel.h"

namespace itex_amd {
namespace {

class QuantizedBatchMatMulOp : public OpKernel {
 public:
  QuantizedBatchMatMulOp(OpKernelConstruction* ctx, TF_DataType t_out, bool is_v2) : t_out_(t_out), is_v2_(is_v2) {
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("adj_x", &adj_x_));
    ITEX_REQUIRES_OK(ctx, ctx->GetAttr("adj_y", &adj_y_));
    std::vector<std::string> fused_ops;
    if (ctx->HasAttr("fused_ops")) ITEX_REQUIRES_OK(ctx, ctx->GetAttr("fused_ops", &fused_ops));
    int32_t num_args = 0;
    if (is_v2) {  // :461-465
      min_x_idx_ = static_cast<int>(fused_ops.size()) + 1;
    } else {      // :466-485
      if (ctx->HasAttr("num_args")) {
        ITEX_REQUIRES_OK(ctx, ctx->GetAttr("num_args", &num_args));
        if (ctx->HasAttr("fused_ops"))
          ITEX_REQUIRES(ctx, num_args == static_cast<int32_t>(fused_ops.size()), TF_INVALID_ARGUMENT,
                        "_QuantizedFusedBatchMatMulV2AndDequantize should have same number of additional inputs as the "
                        "number of fusions");
      }
      min_x_idx_ = num_args + 2;
    }
    std::string joined;
    for (const std::string& f : fused_ops) joined += (joined.empty() ? "" : ",") + f;
    for (const std::string& f : fused_ops) {
      if (f == "Mul") algs_.push_back(ITEXHIP_BIN_MUL);
      else if (f == "Add") algs_.push_back(ITEXHIP_BIN_ADD);
      else if (f == "Dequantize" || f == "Quantized" || f == "Requantize") continue;  // set the output scale only
      else
        ITEX_REQUIRES(ctx, false, TF_UNIMPLEMENTED, "Fusion is not implemented for QuantizedBatchMatMul: [" + joined + "]");
    }
    ITEX_REQUIRES(ctx, algs_.size() <= ITEXHIP_BMM_MAX_BINARY, TF_UNIMPLEMENTED,
                  "The number of Binary op fusion in BatchMatMul is: " + std::to_string(algs_.size()) +
                      ", which is greater than " + std::to_string(ITEXHIP_BMM_MAX_BINARY));
    // the binary operands are read with the output's element type (:393-394); an op whose operand type
    // attribute says otherwise cannot be honoured
    for (const char* attr : {"T", "U"}) {
      if (!algs_.empty() && ctx->HasAttr(attr)) {
        TF_DataType t = t_out;
        ITEX_REQUIRES_OK(ctx, ctx->GetAttr(attr, &t));
        ITEX_REQUIRES(ctx, t == t_out, TF_UNIMPLEMENTED,
                      "the fused Mul / Add operands of the quantized BatchMatMul must have the output's type");
      }
    }
  }

  void Compute(OpKernelContext* ctx) override {
    Tensor x = ctx->input(0);
    Tensor y = ctx->input(1);
    if (!ctx->ok()) return;
    ITEX_REQUIRES(ctx, ctx->num_inputs() >= min_x_idx_ + 4, TF_INVALID_ARGUMENT, "the min / max inputs are missing");
    Tensor min_x = ctx->input(min_x_idx_), max_x = ctx->input(min_x_idx_ + 1);
    Tensor min_y = ctx->input(min_x_idx_ + 2), max_y = ctx->input(min_x_idx_ + 3);
    if (!ctx->ok()) return;
    ITEX_REQUIRES(ctx, x.dtype() == TF_QINT8 && y.dtype() == TF_QINT8, TF_INVALID_ARGUMENT,
                  "the quantized BatchMatMul takes qint8 operands");
    ITEX_REQUIRES(ctx, x.dims() >= 2 && y.dims() >= 2, TF_INVALID_ARGUMENT, "BatchMatMul operands must have rank >= 2");
    const std::vector<int64_t> xs = x.shape(), ys = y.shape();
    int64_t d0 = xs[xs.size() - 2], d1 = xs[xs.size() - 1], d2 = ys[ys.size() - 2], d3 = ys[ys.size() - 1];
    if (adj_x_) std::swap(d0, d1);
    if (adj_y_) std::swap(d2, d3);
    ITEX_REQUIRES(ctx, d1 == d2, TF_INVALID_ARGUMENT,
                  "Input[0] mismatch Input[1] shape :" + std::to_string(d1) + " vs. " + std::to_string(d2));

    itexhip_bmm_params p{};
    p.M = d0; p.K = d1; p.N = d3;
    p.adj_x = adj_x_; p.adj_y = adj_y_;
    p.out_type = t_out_;
    // batch broadcast (MatMulBCast, :105-109)
    const int nbx = static_cast<int>(xs.size()) - 2, nby = static_cast<int>(ys.size()) - 2, nb = std::max(nbx, nby);
    ITEX_REQUIRES(ctx, nb <= ITEXHIP_BMM_MAX_BATCH_DIMS, TF_UNIMPLEMENTED,
                  "quantized BatchMatMul with more than " + std::to_string(ITEXHIP_BMM_MAX_BATCH_DIMS) + " batch dimensions");
    p.n_batch_dims = nb;
    std::vector<int64_t> out_shape(nb + 2);
    {
      int64_t sx = d0 * d1, sy = d2 * d3;
      for (int i = nb - 1; i >= 0; --i) {
        const int ix = i - (nb - nbx), iy = i - (nb - nby);
        const int64_t dx = ix >= 0 ? xs[ix] : 1, dy = iy >= 0 ? ys[iy] : 1;
        ITEX_REQUIRES(ctx, dx == dy || dx == 1 || dy == 1, TF_INVALID_ARGUMENT,
                      "Input tensors must have compatible batch dimensions");
        p.batch_dims[i] = out_shape[i] = dx == 1 ? dy : dx;
        p.x_batch_stride[i] = dx == 1 ? 0 : sx;
        p.y_batch_stride[i] = dy == 1 ? 0 : sy;
        sx *= dx;
        sy *= dy;
      }
    }
    out_shape[nb] = d0;
    out_shape[nb + 1] = d3;

    // output scale (:497-515; mul_value starts at 1)
    const float range_lhs = std::max(std::abs(min_x.flat<float>()[0]), std::abs(max_x.flat<float>()[0]));
    const float range_rhs = std::max(std::abs(min_y.flat<float>()[0]), std::abs(max_y.flat<float>()[0]));
    const float scale_output = range_lhs * range_rhs / (127.0f * 127.0f);
    p.scale = 1.0f * scale_output;

    // fused Mul / Add operands follow y (:377-413)
    std::vector<Tensor> operands;
    p.n_binary = static_cast<int>(algs_.size());
    for (int b = 0; b < p.n_binary; ++b) {
      operands.push_back(ctx->input(2 + b));
      if (!ctx->ok()) return;
      const Tensor& t = operands.back();
      ITEX_REQUIRES(ctx, t.dtype() == t_out_, TF_INVALID_ARGUMENT, "a fused Mul / Add operand must have the output's type");
      const std::vector<int64_t> ts = t.shape();
      itexhip_bmm_binary& bin = p.binary[b];
      bin.alg = algs_[b];
      bin.data = t.data();
      if (t.NumElements() != 1) {
        ITEX_REQUIRES(ctx, ts.size() == out_shape.size(), TF_INVALID_ARGUMENT,
                      "Binary input of FusedBatchMatMul must be scalar or have the rank of the output");
        int64_t st = 1;
        for (int i = nb + 1; i >= 0; --i) {
          ITEX_REQUIRES(ctx, ts[i] == out_shape[i] || ts[i] == 1, TF_INVALID_ARGUMENT,
                        "Binary input of FusedBatchMatMul does not broadcast to the output");
          const int64_t s = ts[i] == 1 ? 0 : st;
          if (i == nb + 1) bin.stride_n = s;
          else if (i == nb) bin.stride_m = s;
          else bin.batch_stride[i] = s;
          st *= ts[i];
        }
      }
    }

    Tensor out = ctx->allocate_output(0, t_out_, out_shape);
    if (!ctx->ok()) return;
    const int st = itexhip_qbatch_matmul(&p, x.flat<int8_t>(), y.flat<int8_t>(), out.data(), ctx->stream());
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                  std::string("Operation received an exception: ") + itexhip_last_error());
  }

 private:
  TF_DataType t_out_;
  bool is_v2_;
  bool adj_x_ = false, adj_y_ = false;
  int min_x_idx_ = 2;
  std::vector<int> algs_;
};

template <int TOUT, bool V2>
struct BmmKernel : QuantizedBatchMatMulOp {
  explicit BmmKernel(OpKernelConstruction* c) : QuantizedBatchMatMulOp(c, static_cast<TF_DataType>(TOUT), V2) {}
};

template <int TOUT, bool V2>
void Reg(const char* op, const char* out_attr, std::initializer_list<const char*> host_args) {
  KernelDefBuilder b(op, "QuantizedBatchMatMulV2Op");
  b.TypeConstraint("T1", TF_QINT8).TypeConstraint("T2", TF_QINT8).TypeConstraint(out_attr, static_cast<TF_DataType>(TOUT));
  for (const char* h : host_args) b.HostMemory(h);
  b.Register<BmmKernel<TOUT, V2>>();
}

template <bool V2>
void RegAllOutputs(const char* op, const char* out_attr, std::initializer_list<const char*> host_args) {
  Reg<TF_FLOAT, V2>(op, out_attr, host_args);
  Reg<TF_BFLOAT16, V2>(op, out_attr, host_args);
  Reg<TF_HALF, V2>(op, out_attr, host_args);
}

}  // namespace

// Names, type constraints and host-memory arguments as registered by the reference for a device
// (itex/core/kernels/gpu/matmul_op.cc:612-655); the _ITEX names are the CPU-side renames
// (itex/core/graph/native_layout/native_layout.cc:177-190), registered as well.
void AddQuantizedBatchMatMulKernels() {
  for (const char* op : {"_QuantizedBatchMatMulV2AndDequantize", "_ITEXQuantizedBatchMatMulV2AndDequantize",
                         "_QuantizedFusedBatchMatMulV2AndDequantize", "_ITEXQuantizedFusedBatchMatMulV2AndDequantize"})
    RegAllOutputs<false>(op, "Toutput", {"min_x", "max_x", "min_y", "max_y"});
  for (const char* op : {"_QuantizedBatchMatMul", "_ITEXQuantizedBatchMatMul"})
    RegAllOutputs<true>(op, "Tout", {"host_inputs", "host_outputs"});
}

}  // namespace itex_amd
