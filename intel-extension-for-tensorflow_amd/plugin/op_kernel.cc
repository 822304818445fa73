// See op_kernel.h.  Follows the call sequences of itex/core/utils/op_kernel.cc (cited per function).
#include "op_kernel.h"

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>

#include "itexhip.h"

namespace itex_amd {
namespace {
struct StatusPtr {
  TF_Status* s = TF_NewStatus();
  ~StatusPtr() { TF_DeleteStatus(s); }
  operator TF_Status*() const { return s; }
};
bool SyncExec() {
  static const bool v = [] { const char* e = std::getenv("ITEX_SYNC_EXEC"); return e && e[0] == '1'; }();
  return v;
}
}  // namespace

size_t DataTypeSize(TF_DataType t) {
  switch (t) {
    case TF_FLOAT: case TF_INT32: case TF_QINT32: return 4;
    case TF_QINT8: case TF_QUINT8: case TF_INT8: case TF_UINT8: case TF_BOOL: return 1;
    case TF_BFLOAT16: case TF_HALF: case TF_INT16: return 2;
    case TF_DOUBLE: case TF_INT64: return 8;
    default: return 0;
  }
}

// ---- construction (op_kernel.cc:539-633, 752, 777) --------------------------------------------
bool OpKernelConstruction::Check(TF_Status* st) {
  if (TF_GetCode(st) == TF_OK) return true;
  ok_ = false;
  TF_OpKernelConstruction_Failure(ctx_, st);
  return false;
}
void OpKernelConstruction::CtxFailure(TF_Code code, const std::string& msg) {
  StatusPtr st;
  TF_SetStatus(st, code, msg.c_str());
  ok_ = false;
  TF_OpKernelConstruction_Failure(ctx_, st);
}
bool OpKernelConstruction::HasAttr(const char* name) const {
  StatusPtr st;
  return TF_OpKernelConstruction_HasAttr(ctx_, name, st) != 0 && TF_GetCode(st) == TF_OK;
}
std::string OpKernelConstruction::name() const {
  TF_StringView v = TF_OpKernelConstruction_GetName(ctx_);
  return std::string(v.data, v.len);
}
bool OpKernelConstruction::GetAttr(const char* name, std::string* v) {
  StatusPtr st;
  int32_t list_size = 0, total_size = 0;
  TF_OpKernelConstruction_GetAttrSize(ctx_, name, &list_size, &total_size, st);
  if (!Check(st)) return false;
  std::vector<char> buf(static_cast<size_t>(total_size) + 1, 0);
  TF_OpKernelConstruction_GetAttrString(ctx_, name, buf.data(), static_cast<size_t>(total_size), st);
  if (!Check(st)) return false;
  v->assign(buf.data(), static_cast<size_t>(total_size));
  return true;
}
bool OpKernelConstruction::GetAttr(const char* name, bool* v) {
  StatusPtr st;
  unsigned char b = 0;
  TF_OpKernelConstruction_GetAttrBool(ctx_, name, &b, st);
  if (!Check(st)) return false;
  *v = b != 0;
  return true;
}
bool OpKernelConstruction::GetAttr(const char* name, int32_t* v) {
  StatusPtr st;
  TF_OpKernelConstruction_GetAttrInt32(ctx_, name, v, st);
  return Check(st);
}
bool OpKernelConstruction::GetAttr(const char* name, int64_t* v) {
  StatusPtr st;
  TF_OpKernelConstruction_GetAttrInt64(ctx_, name, v, st);
  return Check(st);
}
bool OpKernelConstruction::GetAttr(const char* name, float* v) {
  StatusPtr st;
  TF_OpKernelConstruction_GetAttrFloat(ctx_, name, v, st);
  return Check(st);
}
bool OpKernelConstruction::GetAttr(const char* name, TF_DataType* v) {
  StatusPtr st;
  TF_OpKernelConstruction_GetAttrType(ctx_, name, v, st);
  return Check(st);
}
bool OpKernelConstruction::GetAttr(const char* name, std::vector<std::string>* v) {
  StatusPtr st;
  int32_t list_size = 0, total_size = 0;
  TF_OpKernelConstruction_GetAttrSize(ctx_, name, &list_size, &total_size, st);
  if (!Check(st)) return false;
  v->clear();
  if (list_size <= 0) return true;
  std::vector<char*> values(static_cast<size_t>(list_size));
  std::vector<size_t> lengths(static_cast<size_t>(list_size));
  std::vector<char> storage(static_cast<size_t>(total_size) + 1);
  TF_OpKernelConstruction_GetAttrStringList(ctx_, name, values.data(), lengths.data(), list_size, storage.data(),
                                            static_cast<size_t>(total_size), st);
  if (!Check(st)) return false;
  for (int i = 0; i < list_size; ++i) v->emplace_back(values[i], lengths[i]);
  return true;
}

bool OpKernelConstruction::GetAttr(const char* name, std::vector<int64_t>* v) {
  StatusPtr st;
  int32_t list_size = 0, total_size = 0;
  TF_OpKernelConstruction_GetAttrSize(ctx_, name, &list_size, &total_size, st);
  if (!Check(st)) return false;
  v->assign(static_cast<size_t>(list_size > 0 ? list_size : 0), 0);
  if (list_size <= 0) return true;
  TF_OpKernelConstruction_GetAttrInt64List(ctx_, name, v->data(), list_size, st);
  return Check(st);
}

// ---- compute (op_kernel.cc:108-129, 234-238, 333-340, 437-443, 511-518; op_kernel.h:406) -------
void OpKernelContext::CtxFailure(TF_Code code, const std::string& msg) {
  StatusPtr st;
  TF_SetStatus(st, code, msg.c_str());
  ok_ = false;
  TF_OpKernelContext_Failure(ctx_, st);
}
Tensor OpKernelContext::input(int i) {
  StatusPtr st;
  TF_Tensor* t = nullptr;
  TF_GetInput(ctx_, i, &t, st);
  if (TF_GetCode(st) != TF_OK) {
    ok_ = false;
    TF_OpKernelContext_Failure(ctx_, st);
    return Tensor();
  }
  return Tensor(t);
}
Tensor OpKernelContext::allocate_output(int index, TF_DataType dtype, const std::vector<int64_t>& dims) {
  StatusPtr st;
  int64_t n = 1;
  for (int64_t d : dims) n *= d;
  TF_Tensor* t = TF_AllocateOutput(ctx_, index, dtype, dims.data(), static_cast<int>(dims.size()),
                                   static_cast<size_t>(n) * DataTypeSize(dtype), st);
  if (TF_GetCode(st) != TF_OK || t == nullptr) {
    ok_ = false;
    if (TF_GetCode(st) == TF_OK) TF_SetStatus(st, TF_INTERNAL, "TF_AllocateOutput returned no tensor");
    TF_OpKernelContext_Failure(ctx_, st);
    return Tensor();
  }
  return Tensor(t);
}
Tensor OpKernelContext::forward_input_or_allocate_output(int candidate, int out_index,
                                                         const std::vector<int64_t>& dims, TF_DataType) {
  StatusPtr st;
  int forwarded = -1;
  TF_Tensor* t = TF_ForwardInputOrAllocateOutput(ctx_, &candidate, 1, out_index, dims.data(),
                                                 static_cast<int>(dims.size()), &forwarded, st);
  if (TF_GetCode(st) != TF_OK || t == nullptr) {
    ok_ = false;
    if (TF_GetCode(st) == TF_OK) TF_SetStatus(st, TF_INTERNAL, "TF_ForwardInputOrAllocateOutput returned no tensor");
    TF_OpKernelContext_Failure(ctx_, st);
    return Tensor();
  }
  return Tensor(t);
}
Tensor OpKernelContext::allocate_temp(TF_DataType dtype, const std::vector<int64_t>& dims, bool on_host) {
  StatusPtr st;
  TF_AllocatorAttributes attrs;
  attrs.struct_size = TF_ALLOCATOR_ATTRIBUTES_STRUCT_SIZE;
  attrs.on_host = on_host ? 1 : 0;
  TF_Tensor* t = TF_AllocateTemp(ctx_, dtype, dims.data(), static_cast<int>(dims.size()), &attrs, st);
  if (TF_GetCode(st) != TF_OK || t == nullptr) {
    ok_ = false;
    if (TF_GetCode(st) == TF_OK) TF_SetStatus(st, TF_INTERNAL, "TF_AllocateTemp returned no tensor");
    TF_OpKernelContext_Failure(ctx_, st);
    return Tensor();
  }
  return Tensor(t);
}
void* OpKernelContext::stream() {
  StatusPtr st;
  SP_Stream s = TF_GetStream(ctx_, st);
  if (TF_GetCode(st) != TF_OK || s == nullptr) return nullptr;  // default stream
  return s->stream_handle;
}

// ---- registration (op_kernel.cc:874-941) --------------------------------------------------------
std::vector<KernelRegistration>& KernelRegistry() {
  static std::vector<KernelRegistration> table;
  return table;
}
void ComputeTrampoline(void* kernel, TF_OpKernelContext* c) {
  OpKernelContext ctx(c);
  static_cast<OpKernel*>(kernel)->Compute(&ctx);
  // ITEX_SYNC_EXEC=1: wait for the enqueued work before returning (op_kernel.h:869-905)
  if (SyncExec() && ctx.ok()) itexhip_stream_synchronize(ctx.stream());
}
void DeleteTrampoline(void* kernel) { delete static_cast<OpKernel*>(kernel); }

void RegisterKernels(const char* device_type) {
  for (const KernelRegistration& r : KernelRegistry()) {
    StatusPtr st;
    TF_KernelBuilder* b = TF_NewKernelBuilder(r.op_name.c_str(), device_type, r.create, r.compute, r.del);
    bool good = true;
    for (const auto& tc : r.type_constraints) {
      TF_KernelBuilder_TypeConstraint(b, tc.first.c_str(), tc.second, st);
      if (TF_GetCode(st) != TF_OK) {
        std::fprintf(stderr, "itex_amd: type constraint %s on %s failed: %s\n", tc.first.c_str(), r.op_name.c_str(),
                     TF_Message(st));
        good = false;
      }
    }
    for (const auto& h : r.host_memory_args) TF_KernelBuilder_HostMemory(b, h.c_str());
    if (!good) continue;
    TF_RegisterKernelBuilder(r.kernel_label.c_str(), b, st);  // takes ownership of the builder
    if (TF_GetCode(st) != TF_OK)
      std::fprintf(stderr, "itex_amd: registering %s for %s failed: %s\n", r.kernel_label.c_str(), r.op_name.c_str(),
                   TF_Message(st));
  }
}

}  // namespace itex_amd
