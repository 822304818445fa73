// _QuantizedTranspose and QuantizedReshape: the data-movement ops between the quantized linears and the
// quantized BatchMatMuls of an attention block.  Both pass the tensor's min / max through unchanged
// (itex/core/kernels/common/transpose_op.h:197-236, quantized_reshape_op.h:36-195).
#include <string>
#include <vector>

#include "itexhip.h"
#include "op_kernel.h"

namespace itex_amd {
namespace {

int ElemSize(TF_DataType t) { return t == TF_QINT32 ? 4 : 1; }

bool ScalarLike(const Tensor& t) { return t.dims() == 0 || (t.dims() == 1 && t.dim_size(0) == 1); }

// element i of an int32 / int64 host tensor
int64_t IndexAt(const Tensor& t, int64_t i) {
  return t.dtype() == TF_INT64 ? t.flat<int64_t>()[i] : static_cast<int64_t>(t.flat<int32_t>()[i]);
}

class QuantizedTransposeOp : public OpKernel {
 public:
  explicit QuantizedTransposeOp(OpKernelConstruction*) {}

  void Compute(OpKernelContext* ctx) override {
    Tensor x = ctx->input(0);
    Tensor perm = ctx->input(1);
    Tensor min_x = ctx->input(2);
    Tensor max_x = ctx->input(3);
    if (!ctx->ok()) return;
    const int rank = x.dims();
    ITEX_REQUIRES(ctx, perm.dims() == 1, TF_INVALID_ARGUMENT, "perm must be a vector");
    ITEX_REQUIRES(ctx, perm.dtype() == TF_INT32 || perm.dtype() == TF_INT64, TF_INVALID_ARGUMENT, "perm must be int32 or int64");
    ITEX_REQUIRES(ctx, perm.NumElements() == rank, TF_INVALID_ARGUMENT,
                  "transpose expects a vector of size " + std::to_string(rank) + ". But input(1) is a vector of size " +
                      std::to_string(perm.NumElements()));
    ITEX_REQUIRES(ctx, rank <= 8, TF_UNIMPLEMENTED, "quantized Transpose of more than 8 dimensions");
    const std::vector<int64_t> xs = x.shape();
    std::vector<int32_t> p(rank);
    std::vector<int64_t> ys(rank);
    std::vector<bool> seen(rank, false);
    for (int i = 0; i < rank; ++i) {
      const int64_t d = IndexAt(perm, i);
      ITEX_REQUIRES(ctx, d >= 0 && d < rank, TF_INVALID_ARGUMENT, std::to_string(d) + " is out of range [0 .. " + std::to_string(rank) + ")");
      ITEX_REQUIRES(ctx, !seen[d], TF_INVALID_ARGUMENT, std::to_string(d) + " is missing or repeated in perm");
      seen[d] = true;
      p[i] = static_cast<int32_t>(d);
      ys[i] = xs[d];
    }
    ITEX_REQUIRES(ctx, ScalarLike(min_x), TF_INVALID_ARGUMENT, "min_x must be a scalar or a vector of 1 element");
    ITEX_REQUIRES(ctx, ScalarLike(max_x), TF_INVALID_ARGUMENT, "max_x must be a scalar or a vector of 1 element");
    Tensor y = ctx->allocate_output(0, x.dtype(), ys);
    if (!ctx->ok()) return;
    const int st = itexhip_transpose(x.data(), y.data(), ElemSize(x.dtype()), rank, xs.data(), p.data(), ctx->stream());
    ITEX_REQUIRES(ctx, st == ITEXHIP_OK, st == ITEXHIP_INVALID_ARGUMENT ? TF_INVALID_ARGUMENT : TF_ABORTED,
                  std::string("Operation received an exception: ") + itexhip_last_error());
    // the range tensors pass through with their shape (set_output of the inputs, :232-233)
    Tensor out_min = ctx->allocate_output(1, TF_FLOAT, min_x.shape());
    Tensor out_max = ctx->allocate_output(2, TF_FLOAT, max_x.shape());
    if (!ctx->ok()) return;
    out_min.flat<float>()[0] = min_x.flat<float>()[0];
    out_max.flat<float>()[0] = max_x.flat<float>()[0];
  }
};

class QuantizedReshapeOp : public OpKernel {
 public:
  explicit QuantizedReshapeOp(OpKernelConstruction*) {}

  void Compute(OpKernelContext* ctx) override {
    Tensor input = ctx->input(0);
    Tensor sizes = ctx->input(1);
    Tensor in_min = ctx->input(2);
    Tensor in_max = ctx->input(3);
    if (!ctx->ok()) return;
    ITEX_REQUIRES(ctx, sizes.dims() <= 1, TF_INVALID_ARGUMENT, "sizes input must be 1-D");
    ITEX_REQUIRES(ctx, sizes.dtype() == TF_INT32 || sizes.dtype() == TF_INT64, TF_INVALID_ARGUMENT,
                  "desired shape must be a DT_INT32 or DT_INT64 vector");
    // quantized_reshape_op.h:52-134: one dimension may be -1 and is inferred
    std::vector<int64_t> shape;
    int64_t product = 1;
    int unknown = -1;
    for (int64_t i = 0; i < sizes.NumElements(); ++i) {
      const int64_t s = IndexAt(sizes, i);
      if (s == -1) {
        ITEX_REQUIRES(ctx, unknown == -1, TF_INVALID_ARGUMENT,
                      "Only one input size may be -1, not both " + std::to_string(unknown) + " and " + std::to_string(i));
        unknown = static_cast<int>(i);
        shape.push_back(1);
      } else {
        ITEX_REQUIRES(ctx, s >= 0, TF_INVALID_ARGUMENT, "Size " + std::to_string(i) + " must be non-negative, not " + std::to_string(s));
        shape.push_back(s);
        product *= s;
      }
    }
    const int64_t n_in = input.NumElements();
    if (unknown != -1) {
      ITEX_REQUIRES(ctx, product > 0 && n_in % product == 0, TF_INVALID_ARGUMENT,
                    "Input to reshape is a tensor with " + std::to_string(n_in) +
                        " values, but the requested shape requires a multiple of " + std::to_string(product));
      shape[unknown] = n_in / product;
      product *= shape[unknown];
    }
    ITEX_REQUIRES(ctx, product == n_in, TF_INVALID_ARGUMENT,
                  "Input to reshape is a tensor with " + std::to_string(n_in) + " values, but the requested shape has " +
                      std::to_string(product));
    ITEX_REQUIRES(ctx, ScalarLike(in_min), TF_INVALID_ARGUMENT, "input_min must be a scalar or a vector of 1 element");
    ITEX_REQUIRES(ctx, ScalarLike(in_max), TF_INVALID_ARGUMENT, "input_max must be a scalar or a vector of 1 element");
    // the output shares the input's buffer when TensorFlow lets it; otherwise the bytes are copied
    Tensor out = ctx->forward_input_or_allocate_output(0, 0, shape, input.dtype());
    if (!ctx->ok()) return;
    if (out.data() != input.data() && n_in > 0) {
      const int st = itexhip_memcpy_d2d_async(out.data(), input.data(), static_cast<size_t>(n_in) * ElemSize(input.dtype()), ctx->stream());
      ITEX_REQUIRES(ctx, st == ITEXHIP_OK, TF_ABORTED, std::string("Operation received an exception: ") + itexhip_last_error());
    }
    Tensor out_min = ctx->allocate_output(1, TF_FLOAT, {});
    Tensor out_max = ctx->allocate_output(2, TF_FLOAT, {});
    if (!ctx->ok()) return;
    out_min.flat<float>()[0] = in_min.flat<float>()[0];
    out_max.flat<float>()[0] = in_max.flat<float>()[0];
  }
};

}  // namespace

// itex/core/kernels/gpu/transpose_op.cc:48-55, gpu/quantized_reshape_op.cc:24-37; the _ITEX names are the
// CPU-side renames (kernels/cpu/transpose_op.cc:33, native_layout.cc:171-172, 197-198)
void AddQuantizedShapeKernels() {
  for (TF_DataType t : {TF_QINT8, TF_QUINT8, TF_QINT32}) {
    for (const char* op : {"_QuantizedTranspose", "_ITEXQuantizedTranspose"}) {
      KernelDefBuilder b(op, "QuantizedTransposeOp");
      b.TypeConstraint("T", t);
      for (const char* h : {"perm", "min_x", "max_x", "min_y", "max_y"}) b.HostMemory(h);
      b.Register<QuantizedTransposeOp>();
    }
    for (const char* op : {"QuantizedReshape", "_ITEXQuantizedReshape"}) {
      KernelDefBuilder b(op, "QuantizedReshapeOp");
      b.TypeConstraint("T", t);
      for (const char* h : {"shape", "input_min", "input_max", "output_min", "output_max"}) b.HostMemory(h);
      b.Register<QuantizedReshapeOp>();
    }
  }
}

}  // namespace itex_amd
