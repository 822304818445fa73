// C++ facade over the TensorFlow kernel C API, in the shape of the reference's adapter
// (itex/core/utils/op_kernel.{h,cc}, plugin_tensor.h): OpKernel / OpKernelConstruction /
// OpKernelContext, RAII tensors, a registration table.  Only what the INT8 kernels need.
#ifndef ITEX_AMD_PLUGIN_OP_KERNEL_H_
#define ITEX_AMD_PLUGIN_OP_KERNEL_H_

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

#include "tf_c_api_subset.h"

namespace itex_amd {

// ---- a tensor handle that releases its TF_Tensor reference ------------------------------------
class Tensor {
 public:
  Tensor() = default;
  explicit Tensor(TF_Tensor* t) : t_(t) {}
  Tensor(Tensor&& o) noexcept : t_(o.t_) { o.t_ = nullptr; }
  Tensor& operator=(Tensor&& o) noexcept {
    if (this != &o) { reset(); t_ = o.t_; o.t_ = nullptr; }
    return *this;
  }
  Tensor(const Tensor&) = delete;
  Tensor& operator=(const Tensor&) = delete;
  ~Tensor() { reset(); }
  void reset() { if (t_) TF_DeleteTensor(t_); t_ = nullptr; }
  bool valid() const { return t_ != nullptr; }
  TF_Tensor* get() const { return t_; }
  void* data() const { return TF_TensorData(t_); }
  template <typename T> T* flat() const { return static_cast<T*>(TF_TensorData(t_)); }
  int dims() const { return TF_NumDims(t_); }
  int64_t dim_size(int i) const { return TF_Dim(t_, i); }
  int64_t NumElements() const { return TF_TensorElementCount(t_); }
  TF_DataType dtype() const { return TF_TensorType(t_); }
  std::vector<int64_t> shape() const {
    std::vector<int64_t> s(dims());
    for (int i = 0; i < dims(); ++i) s[i] = dim_size(i);
    return s;
  }

 private:
  TF_Tensor* t_ = nullptr;
};

// ---- construction context ----------------------------------------------------------------------
class OpKernelConstruction {
 public:
  explicit OpKernelConstruction(TF_OpKernelConstruction* ctx) : ctx_(ctx) {}
  bool HasAttr(const char* name) const;
  // each returns false and records the failure on error
  bool GetAttr(const char* name, std::string* v);
  bool GetAttr(const char* name, bool* v);
  bool GetAttr(const char* name, int32_t* v);
  bool GetAttr(const char* name, int64_t* v);
  bool GetAttr(const char* name, float* v);
  bool GetAttr(const char* name, TF_DataType* v);
  bool GetAttr(const char* name, std::vector<std::string>* v);
  bool GetAttr(const char* name, std::vector<int64_t>* v);
  void CtxFailure(TF_Code code, const std::string& msg);
  bool ok() const { return ok_; }
  std::string name() const;

 private:
  bool Check(TF_Status* st);
  TF_OpKernelConstruction* ctx_;
  bool ok_ = true;
};

// ---- compute context ---------------------------------------------------------------------------
class OpKernelContext {
 public:
  explicit OpKernelContext(TF_OpKernelContext* ctx) : ctx_(ctx) {}
  int num_inputs() const { return TF_NumInputs(ctx_); }
  int num_outputs() const { return TF_NumOutputs(ctx_); }
  Tensor input(int i);
  Tensor allocate_output(int index, TF_DataType dtype, const std::vector<int64_t>& dims);
  // the output aliases input `candidate` when the runtime allows it, else it is freshly allocated
  Tensor forward_input_or_allocate_output(int candidate, int out_index, const std::vector<int64_t>& dims,
                                          TF_DataType dtype);
  Tensor allocate_temp(TF_DataType dtype, const std::vector<int64_t>& dims, bool on_host = false);
  TF_DataType expected_output_dtype(int i) const { return TF_ExpectedOutputDataType(ctx_, i); }
  void* stream();  // hipStream_t of this step
  void CtxFailure(TF_Code code, const std::string& msg);
  bool ok() const { return ok_; }

 private:
  TF_OpKernelContext* ctx_;
  bool ok_ = true;
};

class OpKernel {
 public:
  virtual ~OpKernel() = default;
  virtual void Compute(OpKernelContext* ctx) = 0;
};

// OP_REQUIRES of the reference (itex/core/utils/op_requires.h)
#define ITEX_REQUIRES(CTX, COND, CODE, MSG) \
  do {                                      \
    if (!(COND)) {                          \
      (CTX)->CtxFailure((CODE), (MSG));     \
      return;                               \
    }                                       \
  } while (0)
#define ITEX_REQUIRES_OK(CTX, EXPR) \
  do {                              \
    if (!(EXPR)) return;            \
  } while (0)

size_t DataTypeSize(TF_DataType t);

// ---- registration table -------------------------------------------------------------------------
struct KernelRegistration {
  std::string op_name;
  std::string kernel_label;  // class name, as passed to TF_RegisterKernelBuilder
  std::vector<std::pair<std::string, TF_DataType>> type_constraints;
  std::vector<std::string> host_memory_args;
  void* (*create)(TF_OpKernelConstruction*);
  void (*compute)(void*, TF_OpKernelContext*);
  void (*del)(void*);
};

std::vector<KernelRegistration>& KernelRegistry();
void ComputeTrampoline(void* kernel, TF_OpKernelContext* ctx);
void DeleteTrampoline(void* kernel);
template <class K>
void* CreateTrampoline(TF_OpKernelConstruction* c) {
  OpKernelConstruction ctx(c);
  // like the reference (op_kernel.h:952-963) the object is returned even when construction recorded a
  // failure; the runtime sees the failed status and deletes it
  return static_cast<OpKernel*>(new K(&ctx));
}

class KernelDefBuilder {
 public:
  KernelDefBuilder(const char* op, const char* label) { r_.op_name = op; r_.kernel_label = label; }
  KernelDefBuilder& TypeConstraint(const char* attr, TF_DataType t) { r_.type_constraints.emplace_back(attr, t); return *this; }
  KernelDefBuilder& HostMemory(const char* arg) { r_.host_memory_args.emplace_back(arg); return *this; }
  template <class K>
  void Register() {
    r_.create = &CreateTrampoline<K>;
    r_.compute = &ComputeTrampoline;
    r_.del = &DeleteTrampoline;
    KernelRegistry().push_back(r_);
  }

 private:
  KernelRegistration r_;
};

// hands every entry of the table to TensorFlow (TF_NewKernelBuilder ... TF_RegisterKernelBuilder)
void RegisterKernels(const char* device_type);

// the op kernels fill the table
void AddQuantizeKernels();
void AddDequantizeKernels();
void AddQuantizedMatMulKernels();
void AddQuantizedBatchMatMulKernels();
void AddQuantizedShapeKernels();
void AddQuantizedConvKernels();
void AddRequantizeKernels();
// op definitions for the ops stock TensorFlow does not have
void RegisterOps();

}  // namespace itex_amd
#endif  // ITEX_AMD_PLUGIN_OP_KERNEL_H_
