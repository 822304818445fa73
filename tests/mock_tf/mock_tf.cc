// A stand-in for the TensorFlow runtime, for tests: implements the C API subset declared in
// include/tf_c_api_subset.h over plain memory, records kernel and op registrations, and drives
// create / compute / delete of a kernel the way TensorFlow's C kernel wrapper does.  Test
// infrastructure only; it allocates device memory through a callback supplied by the test (PyTorch)
// or from the device plugin's own allocator (mock_device_*), or, without either, from the host heap.
#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

#include "tf_c_api_subset.h"
#include "tf_grappler_subset.h"
#include "tf_stream_executor_subset.h"

// ------------------------------------------------------------------------------------------------
// object definitions
// ------------------------------------------------------------------------------------------------
struct TF_Status {
  TF_Code code = TF_OK;
  std::string msg;
};

namespace {
typedef void* (*AllocFn)(size_t bytes, int on_host);
typedef void (*FreeFn)(void* p, int on_host);
AllocFn g_alloc = nullptr;
FreeFn g_free = nullptr;

struct Buffer {
  void* data = nullptr;
  size_t bytes = 0;
  bool owned = false;
  bool on_host = true;
  int refs = 0;
  ~Buffer() {
    if (owned && data) {
      if (!on_host && g_free) g_free(data, 0);
      else std::free(data);
    }
  }
};
size_t DtypeSize(TF_DataType t) {
  switch (t) {
    case TF_FLOAT: case TF_INT32: case TF_QINT32: return 4;
    case TF_QINT8: case TF_QUINT8: case TF_INT8: case TF_UINT8: case TF_BOOL: return 1;
    case TF_BFLOAT16: case TF_HALF: case TF_INT16: return 2;
    case TF_DOUBLE: case TF_INT64: return 8;
    default: return 1;
  }
}
}  // namespace

struct TF_Tensor {
  TF_DataType dtype;
  std::vector<int64_t> dims;
  std::shared_ptr<Buffer> buf;
};

namespace {
TF_Tensor* NewTensor(TF_DataType dtype, const int64_t* dims, int ndims, bool on_host) {
  auto* t = new TF_Tensor;
  t->dtype = dtype;
  t->dims.assign(dims, dims + ndims);
  int64_t n = 1;
  for (int64_t d : t->dims) n *= d;
  t->buf = std::make_shared<Buffer>();
  t->buf->bytes = static_cast<size_t>(n) * DtypeSize(dtype);
  t->buf->owned = true;
  t->buf->on_host = on_host || g_alloc == nullptr;
  const size_t bytes = t->buf->bytes ? t->buf->bytes : 1;
  t->buf->data = t->buf->on_host ? std::calloc(1, bytes + 64) : g_alloc(bytes, 0);
  return t;
}

struct AttrValue {
  enum Kind { STRING, INT, FLOAT, BOOL, TYPE, STRING_LIST, TYPE_LIST, INT_LIST } kind;
  std::string s;
  int64_t i = 0;
  float f = 0;
  bool b = false;
  TF_DataType t = TF_FLOAT;
  std::vector<std::string> sl;
  std::vector<TF_DataType> tl;
  std::vector<int64_t> il;
};
}  // namespace

struct TF_KernelBuilder {
  std::string op, device, label;
  void* (*create)(TF_OpKernelConstruction*);
  void (*compute)(void*, TF_OpKernelContext*);
  void (*del)(void*);
  std::vector<std::pair<std::string, TF_DataType>> constraints;
  std::vector<std::string> host_memory;
  int priority = 0;
};

struct TF_OpKernelConstruction {
  std::string name;
  std::map<std::string, AttrValue> attrs;
  TF_Status status;
};

struct TF_OpKernelContext {
  struct In { TF_Tensor* t; bool allow_forward; };
  std::vector<In> inputs;
  std::vector<TF_Tensor*> outputs;
  std::vector<int> forwarded_from;
  std::vector<TF_DataType> out_dtypes;
  std::vector<char> out_on_host;
  SP_Stream_st stream{nullptr};
  TF_Status status;
  int temp_allocs = 0;
};

struct TF_OpDefinitionBuilder {
  std::string name;
  std::vector<std::string> inputs, outputs, attrs;
  bool has_shape_fn = false;
};
struct TF_ShapeInferenceContext {
  bool unknown = false;
};

namespace {
std::vector<std::unique_ptr<TF_KernelBuilder>> g_kernels;
std::vector<std::unique_ptr<TF_OpDefinitionBuilder>> g_ops;
std::vector<std::string> g_stock_ops;
std::string g_json;
int g_delete_calls = 0;

struct Node {
  std::string op, device;
  TF_OpKernelConstruction construction;
  TF_OpKernelContext context;
  TF_KernelBuilder* kernel = nullptr;
  void* object = nullptr;
};
}  // namespace

// ------------------------------------------------------------------------------------------------
// the C API
// ------------------------------------------------------------------------------------------------
extern "C" {

TF_Status* TF_NewStatus(void) { return new TF_Status; }
void TF_DeleteStatus(TF_Status* s) { delete s; }
void TF_SetStatus(TF_Status* s, TF_Code code, const char* msg) { s->code = code; s->msg = msg ? msg : ""; }
TF_Code TF_GetCode(const TF_Status* s) { return s->code; }
const char* TF_Message(const TF_Status* s) { return s->msg.c_str(); }

void* TF_TensorData(const TF_Tensor* t) { return t->buf->data; }
int TF_NumDims(const TF_Tensor* t) { return static_cast<int>(t->dims.size()); }
int64_t TF_Dim(const TF_Tensor* t, int i) { return t->dims[i]; }
TF_DataType TF_TensorType(const TF_Tensor* t) { return t->dtype; }
size_t TF_TensorByteSize(const TF_Tensor* t) { return t->buf->bytes; }
int64_t TF_TensorElementCount(const TF_Tensor* t) {
  int64_t n = 1;
  for (int64_t d : t->dims) n *= d;
  return n;
}
void TF_DeleteTensor(TF_Tensor* t) { delete t; }

void TF_DeleteBuffer(TF_Buffer* b) {
  if (b == nullptr) return;
  if (b->data_deallocator) b->data_deallocator(const_cast<void*>(b->data), b->length);
  delete b;
}
static void PutVarint(std::string* s, uint64_t v) {
  while (v >= 0x80) { s->push_back(static_cast<char>(v | 0x80)); v >>= 7; }
  s->push_back(static_cast<char>(v));
}
TF_Buffer* TF_GetAllOpList(void) {
  std::string list;
  auto add = [&](const std::string& name) {
    std::string op;
    op.push_back(0x0a);  // OpDef.name
    PutVarint(&op, name.size());
    op += name;
    op.push_back(0x1a);  // OpDef.output_arg (an unrelated field the reader must skip)
    PutVarint(&op, 2);
    op += "\x0a\x00";
    list.push_back(0x0a);  // OpList.op
    PutVarint(&list, op.size());
    list += op;
  };
  for (const auto& n : g_stock_ops) add(n);
  for (const auto& o : g_ops) add(o->name);
  auto* b = new TF_Buffer;
  char* data = static_cast<char*>(std::malloc(list.size() + 1));
  std::memcpy(data, list.data(), list.size());
  b->data = data;
  b->length = list.size();
  b->data_deallocator = [](void* d, size_t) { std::free(d); };
  return b;
}

TF_KernelBuilder* TF_NewKernelBuilder(const char* op_name, const char* device_name,
                                      void* (*create_func)(TF_OpKernelConstruction*),
                                      void (*compute_func)(void*, TF_OpKernelContext*), void (*delete_func)(void*)) {
  auto* b = new TF_KernelBuilder;
  b->op = op_name;
  b->device = device_name;
  b->create = create_func;
  b->compute = compute_func;
  b->del = delete_func;
  return b;
}
void TF_KernelBuilder_TypeConstraint(TF_KernelBuilder* b, const char* attr_name, const TF_DataType type, TF_Status* status) {
  b->constraints.emplace_back(attr_name, type);
  TF_SetStatus(status, TF_OK, "");
}
void TF_KernelBuilder_HostMemory(TF_KernelBuilder* b, const char* arg_name) { b->host_memory.emplace_back(arg_name); }
void TF_KernelBuilder_Priority(TF_KernelBuilder* b, int32_t p) { b->priority = p; }
void TF_RegisterKernelBuilder(const char* kernel_name, TF_KernelBuilder* builder, TF_Status* status) {
  builder->label = kernel_name;
  // a second registration with the same op, device and constraints is an error in TensorFlow
  for (const auto& k : g_kernels) {
    if (k->op == builder->op && k->device == builder->device && k->constraints == builder->constraints) {
      TF_SetStatus(status, TF_ALREADY_EXISTS, ("duplicate kernel registration for " + builder->op).c_str());
      delete builder;
      return;
    }
  }
  g_kernels.emplace_back(builder);
  TF_SetStatus(status, TF_OK, "");
}

static const AttrValue* FindAttr(TF_OpKernelConstruction* ctx, const char* name, AttrValue::Kind kind, TF_Status* st) {
  auto it = ctx->attrs.find(name);
  if (it == ctx->attrs.end()) {
    TF_SetStatus(st, TF_INVALID_ARGUMENT, (std::string("No attr named '") + name + "' in NodeDef").c_str());
    return nullptr;
  }
  if (it->second.kind != kind) {
    TF_SetStatus(st, TF_INVALID_ARGUMENT, (std::string("Attr '") + name + "' has a different type").c_str());
    return nullptr;
  }
  TF_SetStatus(st, TF_OK, "");
  return &it->second;
}
unsigned char TF_OpKernelConstruction_HasAttr(TF_OpKernelConstruction* ctx, const char* attr_name, TF_Status* status) {
  TF_SetStatus(status, TF_OK, "");
  return ctx->attrs.count(attr_name) ? 1 : 0;
}
void TF_OpKernelConstruction_GetAttrSize(TF_OpKernelConstruction* ctx, const char* attr_name, int32_t* list_size,
                                         int32_t* total_size, TF_Status* status) {
  auto it = ctx->attrs.find(attr_name);
  if (it == ctx->attrs.end()) {
    TF_SetStatus(status, TF_INVALID_ARGUMENT, (std::string("No attr named '") + attr_name + "' in NodeDef").c_str());
    return;
  }
  TF_SetStatus(status, TF_OK, "");
  const AttrValue& a = it->second;
  switch (a.kind) {
    case AttrValue::STRING: *list_size = -1; *total_size = static_cast<int32_t>(a.s.size()); break;
    case AttrValue::STRING_LIST: {
      *list_size = static_cast<int32_t>(a.sl.size());
      int32_t t = 0;
      for (const auto& s : a.sl) t += static_cast<int32_t>(s.size());
      *total_size = t;
      break;
    }
    case AttrValue::TYPE_LIST: *list_size = static_cast<int32_t>(a.tl.size()); *total_size = -1; break;
    case AttrValue::INT_LIST: *list_size = static_cast<int32_t>(a.il.size()); *total_size = -1; break;
    default: *list_size = -1; *total_size = -1; break;
  }
}
void TF_OpKernelConstruction_GetAttrType(TF_OpKernelConstruction* ctx, const char* n, TF_DataType* val, TF_Status* st) {
  if (const AttrValue* a = FindAttr(ctx, n, AttrValue::TYPE, st)) *val = a->t;
}
void TF_OpKernelConstruction_GetAttrInt32(TF_OpKernelConstruction* ctx, const char* n, int32_t* val, TF_Status* st) {
  if (const AttrValue* a = FindAttr(ctx, n, AttrValue::INT, st)) *val = static_cast<int32_t>(a->i);
}
void TF_OpKernelConstruction_GetAttrInt64(TF_OpKernelConstruction* ctx, const char* n, int64_t* val, TF_Status* st) {
  if (const AttrValue* a = FindAttr(ctx, n, AttrValue::INT, st)) *val = a->i;
}
void TF_OpKernelConstruction_GetAttrFloat(TF_OpKernelConstruction* ctx, const char* n, float* val, TF_Status* st) {
  if (const AttrValue* a = FindAttr(ctx, n, AttrValue::FLOAT, st)) *val = a->f;
}
void TF_OpKernelConstruction_GetAttrBool(TF_OpKernelConstruction* ctx, const char* n, unsigned char* val, TF_Status* st) {
  if (const AttrValue* a = FindAttr(ctx, n, AttrValue::BOOL, st)) *val = a->b ? 1 : 0;
}
void TF_OpKernelConstruction_GetAttrString(TF_OpKernelConstruction* ctx, const char* n, char* val, size_t max_length,
                                           TF_Status* st) {
  if (const AttrValue* a = FindAttr(ctx, n, AttrValue::STRING, st)) std::memcpy(val, a->s.data(), std::min(max_length, a->s.size()));
}
void TF_OpKernelConstruction_GetAttrStringList(TF_OpKernelConstruction* ctx, const char* n, char** values, size_t* lengths,
                                               int max_values, void* storage, size_t storage_size, TF_Status* st) {
  const AttrValue* a = FindAttr(ctx, n, AttrValue::STRING_LIST, st);
  if (!a) return;
  char* p = static_cast<char*>(storage);
  size_t used = 0;
  for (int i = 0; i < max_values && i < static_cast<int>(a->sl.size()); ++i) {
    const std::string& s = a->sl[i];
    if (used + s.size() > storage_size) { TF_SetStatus(st, TF_INVALID_ARGUMENT, "storage too small"); return; }
    std::memcpy(p + used, s.data(), s.size());
    values[i] = p + used;
    lengths[i] = s.size();
    used += s.size();
  }
}
void TF_OpKernelConstruction_GetAttrTypeList(TF_OpKernelConstruction* ctx, const char* n, TF_DataType* vals, int max_vals,
                                             TF_Status* st) {
  const AttrValue* a = FindAttr(ctx, n, AttrValue::TYPE_LIST, st);
  if (!a) return;
  for (int i = 0; i < max_vals && i < static_cast<int>(a->tl.size()); ++i) vals[i] = a->tl[i];
}
void TF_OpKernelConstruction_GetAttrInt64List(TF_OpKernelConstruction* ctx, const char* n, int64_t* vals, int max_vals,
                                              TF_Status* st) {
  const AttrValue* a = FindAttr(ctx, n, AttrValue::INT_LIST, st);
  if (!a) return;
  for (int i = 0; i < max_vals && i < static_cast<int>(a->il.size()); ++i) vals[i] = a->il[i];
}
TF_StringView TF_OpKernelConstruction_GetName(TF_OpKernelConstruction* ctx) { return TF_StringView{ctx->name.data(), ctx->name.size()}; }
void TF_OpKernelConstruction_Failure(TF_OpKernelConstruction* ctx, TF_Status* status) {
  if (ctx->status.code == TF_OK) ctx->status = *status;  // the first failure sticks
}

int TF_NumInputs(TF_OpKernelContext* ctx) { return static_cast<int>(ctx->inputs.size()); }
int TF_NumOutputs(TF_OpKernelContext* ctx) { return static_cast<int>(ctx->outputs.size()); }
void TF_GetInput(TF_OpKernelContext* ctx, int i, TF_Tensor** tensor, TF_Status* status) {
  if (i < 0 || i >= static_cast<int>(ctx->inputs.size())) {
    TF_SetStatus(status, TF_OUT_OF_RANGE, "input index out of range");
    *tensor = nullptr;
    return;
  }
  *tensor = new TF_Tensor(*ctx->inputs[i].t);  // a new handle on the same buffer; the caller deletes it
  TF_SetStatus(status, TF_OK, "");
}
void TF_SetOutput(TF_OpKernelContext* ctx, int i, const TF_Tensor* tensor, TF_Status* status) {
  if (i < 0 || i >= static_cast<int>(ctx->outputs.size())) { TF_SetStatus(status, TF_OUT_OF_RANGE, "output index out of range"); return; }
  delete ctx->outputs[i];
  ctx->outputs[i] = new TF_Tensor(*tensor);
  TF_SetStatus(status, TF_OK, "");
}
TF_DataType TF_ExpectedOutputDataType(TF_OpKernelContext* ctx, int i) { return ctx->out_dtypes[i]; }
TF_Tensor* TF_AllocateOutput(TF_OpKernelContext* ctx, int index, TF_DataType dtype, const int64_t* dims, int num_dims,
                             size_t len, TF_Status* status) {
  if (index < 0 || index >= static_cast<int>(ctx->outputs.size())) { TF_SetStatus(status, TF_OUT_OF_RANGE, "output index out of range"); return nullptr; }
  if (dtype != ctx->out_dtypes[index]) { TF_SetStatus(status, TF_INVALID_ARGUMENT, "output dtype does not match the node"); return nullptr; }
  TF_Tensor* t = NewTensor(dtype, dims, num_dims, ctx->out_on_host[index] != 0);
  if (len != t->buf->bytes) { TF_SetStatus(status, TF_INVALID_ARGUMENT, "byte length does not match shape and dtype"); delete t; return nullptr; }
  delete ctx->outputs[index];
  ctx->outputs[index] = new TF_Tensor(*t);
  TF_SetStatus(status, TF_OK, "");
  return t;
}
TF_Tensor* TF_ForwardInputOrAllocateOutput(TF_OpKernelContext* ctx, const int* cand, int ncand, int output_index,
                                           const int64_t* output_dims, int output_num_dims, int* forwarded_input,
                                           TF_Status* status) {
  if (forwarded_input) *forwarded_input = -1;
  for (int c = 0; c < ncand; ++c) {
    const int i = cand[c];
    if (i < 0 || i >= static_cast<int>(ctx->inputs.size()) || !ctx->inputs[i].allow_forward) continue;
    TF_Tensor* in = ctx->inputs[i].t;
    int64_t n_out = 1;
    for (int d = 0; d < output_num_dims; ++d) n_out *= output_dims[d];
    if (TF_TensorElementCount(in) != n_out || in->dtype != ctx->out_dtypes[output_index]) continue;
    auto* t = new TF_Tensor(*in);
    t->dims.assign(output_dims, output_dims + output_num_dims);
    delete ctx->outputs[output_index];
    ctx->outputs[output_index] = new TF_Tensor(*t);
    ctx->forwarded_from[output_index] = i;
    if (forwarded_input) *forwarded_input = i;
    TF_SetStatus(status, TF_OK, "");
    return t;
  }
  int64_t n = 1;
  for (int d = 0; d < output_num_dims; ++d) n *= output_dims[d];
  return TF_AllocateOutput(ctx, output_index, ctx->out_dtypes[output_index], output_dims, output_num_dims,
                           static_cast<size_t>(n) * DtypeSize(ctx->out_dtypes[output_index]), status);
}
TF_Tensor* TF_AllocateTemp(TF_OpKernelContext* ctx, TF_DataType dtype, const int64_t* dims, int num_dims,
                           TF_AllocatorAttributes* attrs, TF_Status* status) {
  ctx->temp_allocs++;
  TF_SetStatus(status, TF_OK, "");
  return NewTensor(dtype, dims, num_dims, attrs && attrs->on_host);
}
void TF_OpKernelContext_Failure(TF_OpKernelContext* ctx, TF_Status* status) {
  if (ctx->status.code == TF_OK) ctx->status = *status;
}
SP_Stream TF_GetStream(TF_OpKernelContext* ctx, TF_Status* status) {
  TF_SetStatus(status, TF_OK, "");
  return &ctx->stream;
}
int64_t TF_StepId(TF_OpKernelContext*) { return 1; }

TF_OpDefinitionBuilder* TF_NewOpDefinitionBuilder(const char* op_name) {
  auto* b = new TF_OpDefinitionBuilder;
  b->name = op_name;
  return b;
}
void TF_OpDefinitionBuilderAddInput(TF_OpDefinitionBuilder* b, const char* s) { b->inputs.emplace_back(s); }
void TF_OpDefinitionBuilderAddOutput(TF_OpDefinitionBuilder* b, const char* s) { b->outputs.emplace_back(s); }
void TF_OpDefinitionBuilderAddAttr(TF_OpDefinitionBuilder* b, const char* s) { b->attrs.emplace_back(s); }
void TF_OpDefinitionBuilderSetShapeInferenceFunction(TF_OpDefinitionBuilder* b,
                                                     void (*fn)(TF_ShapeInferenceContext*, TF_Status*)) {
  b->has_shape_fn = fn != nullptr;
  if (fn) {  // exercise it once
    TF_ShapeInferenceContext c;
    TF_Status st;
    fn(&c, &st);
  }
}
void TF_RegisterOpDefinition(TF_OpDefinitionBuilder* b, TF_Status* status) {
  for (const auto& n : g_stock_ops)
    if (n == b->name) { TF_SetStatus(status, TF_ALREADY_EXISTS, ("Op with name " + b->name).c_str()); delete b; return; }
  for (const auto& o : g_ops)
    if (o->name == b->name) { TF_SetStatus(status, TF_ALREADY_EXISTS, ("Op with name " + b->name).c_str()); delete b; return; }
  g_ops.emplace_back(b);
  TF_SetStatus(status, TF_OK, "");
}
void TF_ShapeInferenceContextSetUnknownShape(TF_ShapeInferenceContext* ctx, TF_Status* status) {
  ctx->unknown = true;
  TF_SetStatus(status, TF_OK, "");
}

// ------------------------------------------------------------------------------------------------
// test driver
// ------------------------------------------------------------------------------------------------
void mock_set_allocator(AllocFn a, FreeFn f) { g_alloc = a; g_free = f; }
void mock_add_stock_op(const char* name) { g_stock_ops.emplace_back(name); }
int mock_delete_calls(void) { return g_delete_calls; }

// ---- the StreamExecutor side: what TensorFlow does with a PluggableDevice plugin after dlopen -----
namespace {
struct DevicePlugin {
  bool loaded = false;
  SE_PlatformRegistrationParams params{};
  SP_Platform platform{};
  SP_PlatformFns fns{};
  SP_Device device{};
  SP_DeviceFns device_fns{};
  SP_StreamExecutor se{};
  SP_TimerFns timer_fns{};
  SP_Stream stream = nullptr;
  std::string last_error;
} g_dev;

void* DeviceAlloc(size_t bytes, int on_host) {
  if (on_host) return g_dev.se.host_memory_allocate(&g_dev.device, bytes);
  SP_DeviceMemoryBase m{};
  g_dev.se.allocate(&g_dev.device, bytes, 0, &m);
  return m.opaque;
}
void DeviceFree(void* p, int on_host) {
  if (on_host) { g_dev.se.host_memory_deallocate(&g_dev.device, p); return; }
  SP_DeviceMemoryBase m{};
  m.struct_size = SP_DEVICE_MEMORY_BASE_STRUCT_SIZE;
  m.opaque = p;
  g_dev.se.deallocate(&g_dev.device, &m);
}
int Check(TF_Status& st, const char* what) {
  if (st.code == TF_OK) return 0;
  g_dev.last_error = std::string(what) + ": " + st.msg;
  return static_cast<int>(st.code);
}
}  // namespace

// dlopen the plugin, call SE_InitPlugin, create device `ordinal`, its stream executor and one stream.
// 0 on success; the struct sizes the plugin reports must be the ones of the API header.
int mock_device_load(const char* path, int ordinal) {
  void* h = dlopen(path, RTLD_NOW | RTLD_GLOBAL);
  if (!h) { g_dev.last_error = std::string("dlopen failed: ") + dlerror(); return 1; }
  auto init = reinterpret_cast<void (*)(SE_PlatformRegistrationParams*, TF_Status*)>(dlsym(h, "SE_InitPlugin"));
  if (!init) { g_dev.last_error = "SE_InitPlugin not exported"; return 2; }
  g_dev.params = SE_PlatformRegistrationParams{};
  g_dev.params.struct_size = SE_PLATFORM_REGISTRATION_PARAMS_STRUCT_SIZE;
  g_dev.platform.struct_size = SP_PLATFORM_STRUCT_SIZE;
  g_dev.fns.struct_size = SP_PLATFORM_FNS_STRUCT_SIZE;
  g_dev.params.platform = &g_dev.platform;
  g_dev.params.platform_fns = &g_dev.fns;
  TF_Status st;
  init(&g_dev.params, &st);
  if (int rc = Check(st, "SE_InitPlugin")) return rc;
  if (g_dev.platform.struct_size != SP_PLATFORM_STRUCT_SIZE || g_dev.fns.struct_size != SP_PLATFORM_FNS_STRUCT_SIZE ||
      !g_dev.platform.name || !g_dev.platform.type || !g_dev.fns.create_device || !g_dev.fns.create_stream_executor) {
    g_dev.last_error = "SE_InitPlugin left the platform tables incomplete";
    return 3;
  }
  int count = 0;
  g_dev.fns.get_device_count(&g_dev.platform, &count, &st);
  if (int rc = Check(st, "get_device_count")) return rc;
  if (ordinal >= count) { g_dev.last_error = "no such device"; return 4; }
  SE_CreateDeviceParams dp{};
  dp.struct_size = SE_CREATE_DEVICE_PARAMS_STRUCT_SIZE;
  dp.ordinal = ordinal;
  dp.device = &g_dev.device;
  g_dev.device.struct_size = SP_DEVICE_STRUCT_SIZE;
  g_dev.fns.create_device(&g_dev.platform, &dp, &st);
  if (int rc = Check(st, "create_device")) return rc;
  SE_CreateDeviceFnsParams fp{};
  fp.struct_size = SE_CREATE_DEVICE_FNS_PARAMS_STRUCT_SIZE;
  fp.device_fns = &g_dev.device_fns;
  g_dev.fns.create_device_fns(&g_dev.platform, &fp, &st);
  if (int rc = Check(st, "create_device_fns")) return rc;
  SE_CreateStreamExecutorParams sp{};
  sp.struct_size = SE_CREATE_STREAM_EXECUTOR_PARAMS_STRUCT_SIZE;
  sp.stream_executor = &g_dev.se;
  g_dev.fns.create_stream_executor(&g_dev.platform, &sp, &st);
  if (int rc = Check(st, "create_stream_executor")) return rc;
  if (g_dev.se.struct_size != SP_STREAMEXECUTOR_STRUCT_SIZE) { g_dev.last_error = "stream executor struct size"; return 5; }
  g_dev.fns.create_timer_fns(&g_dev.platform, &g_dev.timer_fns, &st);
  if (int rc = Check(st, "create_timer_fns")) return rc;
  g_dev.se.create_stream(&g_dev.device, &g_dev.stream, &st);
  if (int rc = Check(st, "create_stream")) return rc;
  g_dev.loaded = true;
  return 0;
}
const char* mock_device_error(void) { return g_dev.last_error.c_str(); }
const char* mock_device_describe(void) {
  static std::string s;
  std::ostringstream os;
  os << "{\"platform_name\":\"" << g_dev.platform.name << "\",\"platform_type\":\"" << g_dev.platform.type
     << "\",\"use_bfc_allocator\":" << int(g_dev.platform.use_bfc_allocator) << ",\"ordinal\":" << g_dev.device.ordinal
     << ",\"hardware_name\":\"" << (g_dev.device.hardware_name ? g_dev.device.hardware_name : "") << "\",\"vendor\":\""
     << (g_dev.device.device_vendor ? g_dev.device.device_vendor : "") << "\",\"pci_bus_id\":\""
     << (g_dev.device.pci_bus_id ? g_dev.device.pci_bus_id : "") << "\",\"memory_bandwidth\":"
     << (g_dev.device_fns.get_memory_bandwidth ? g_dev.device_fns.get_memory_bandwidth(&g_dev.device) : -1) << "}";
  s = os.str();
  return s.c_str();
}
// from now on the mock's device and host-pinned tensors come from the plugin's allocators and kernels
// get the plugin's stream
void mock_device_use_allocator(void) { g_alloc = DeviceAlloc; g_free = DeviceFree; }
void* mock_device_stream(void) { return g_dev.stream ? g_dev.stream->stream_handle : nullptr; }
void* mock_device_alloc(uint64_t bytes) { return DeviceAlloc(bytes, 0); }
void mock_device_free(void* p) { DeviceFree(p, 0); }
void* mock_device_host_alloc(uint64_t bytes) { return DeviceAlloc(bytes, 1); }
void mock_device_host_free(void* p) { DeviceFree(p, 1); }
static SP_DeviceMemoryBase Mem(void* p, uint64_t n) {
  SP_DeviceMemoryBase m{};
  m.struct_size = SP_DEVICE_MEMORY_BASE_STRUCT_SIZE;
  m.opaque = p;
  m.size = n;
  return m;
}
int mock_device_h2d(void* dst, const void* src, uint64_t n, int sync) {
  TF_Status st;
  SP_DeviceMemoryBase m = Mem(dst, n);
  if (sync) g_dev.se.sync_memcpy_htod(&g_dev.device, &m, src, n, &st);
  else g_dev.se.memcpy_htod(&g_dev.device, g_dev.stream, &m, src, n, &st);
  return Check(st, "memcpy_htod");
}
int mock_device_d2h(void* dst, const void* src, uint64_t n, int sync) {
  TF_Status st;
  SP_DeviceMemoryBase m = Mem(const_cast<void*>(src), n);
  if (sync) g_dev.se.sync_memcpy_dtoh(&g_dev.device, dst, &m, n, &st);
  else g_dev.se.memcpy_dtoh(&g_dev.device, g_dev.stream, dst, &m, n, &st);
  return Check(st, "memcpy_dtoh");
}
int mock_device_d2d(void* dst, const void* src, uint64_t n, int sync) {
  TF_Status st;
  SP_DeviceMemoryBase d = Mem(dst, n), s = Mem(const_cast<void*>(src), n);
  if (sync) g_dev.se.sync_memcpy_dtod(&g_dev.device, &d, &s, n, &st);
  else g_dev.se.memcpy_dtod(&g_dev.device, g_dev.stream, &d, &s, n, &st);
  return Check(st, "memcpy_dtod");
}
int mock_device_memset(void* dst, int kind, uint32_t pattern, uint64_t n) {  // kind 0: zero, 8: byte, 32: word
  TF_Status st;
  SP_DeviceMemoryBase m = Mem(dst, n);
  if (kind == 0) g_dev.se.mem_zero(&g_dev.device, g_dev.stream, &m, n, &st);
  else if (kind == 8) g_dev.se.memset(&g_dev.device, g_dev.stream, &m, static_cast<uint8_t>(pattern), n, &st);
  else g_dev.se.memset32(&g_dev.device, g_dev.stream, &m, pattern, n, &st);
  return Check(st, "memset");
}
int mock_device_sync(int all) {
  TF_Status st;
  if (all) g_dev.se.synchronize_all_activity(&g_dev.device, &st);
  else g_dev.se.block_host_until_done(&g_dev.device, g_dev.stream, &st);
  return Check(st, "synchronize");
}
int mock_device_stats(int64_t* out /* 8 values */) {
  SP_AllocatorStats s{};
  if (!g_dev.se.get_allocator_stats(&g_dev.device, &s)) return 1;
  out[0] = s.num_allocs; out[1] = s.bytes_in_use; out[2] = s.peak_bytes_in_use; out[3] = s.largest_alloc_size;
  out[4] = s.bytes_reserved; out[5] = s.largest_free_block_bytes;
  int64_t f = 0, t = 0;
  if (!g_dev.se.device_memory_usage(&g_dev.device, &f, &t)) return 2;
  out[6] = f; out[7] = t;
  return 0;
}
// A second stream that must wait for the first (create_stream_dependency), an event recorded behind the
// work, a host callback behind the event: returns 0 when the callback ran after the event completed and
// the data written on the first stream was visible to the copy on the second.
namespace { volatile int g_callback_ran = 0; void Callback(void* arg, TF_Status* st) { g_callback_ran = *static_cast<int*>(arg); TF_SetStatus(st, TF_OK, ""); } }
int mock_device_stream_event_test(void* dev_buf, void* dev_buf2, uint64_t n, void* host_out) {
  TF_Status st;
  SP_Stream second = nullptr;
  g_dev.se.create_stream(&g_dev.device, &second, &st);
  if (int rc = Check(st, "create_stream")) return rc;
  SP_Event ev = nullptr;
  g_dev.se.create_event(&g_dev.device, &ev, &st);
  if (int rc = Check(st, "create_event")) return rc;
  SP_DeviceMemoryBase a = Mem(dev_buf, n), b = Mem(dev_buf2, n);
  g_dev.se.memset(&g_dev.device, g_dev.stream, &a, 0x5a, n, &st);                  // stream 1: fill a
  g_dev.se.create_stream_dependency(&g_dev.device, second, g_dev.stream, &st);     // stream 2 waits for stream 1
  if (int rc = Check(st, "create_stream_dependency")) return rc;
  g_dev.se.memcpy_dtod(&g_dev.device, second, &b, &a, n, &st);                     // stream 2: b = a
  g_dev.se.record_event(&g_dev.device, second, ev, &st);
  if (int rc = Check(st, "record_event")) return rc;
  g_dev.se.wait_for_event(&g_dev.device, g_dev.stream, ev, &st);                   // stream 1 waits for the copy
  if (int rc = Check(st, "wait_for_event")) return rc;
  g_dev.se.memcpy_dtoh(&g_dev.device, g_dev.stream, host_out, &b, n, &st);         // stream 1: read b back
  static int token = 7;
  g_callback_ran = 0;
  if (!g_dev.se.host_callback(&g_dev.device, g_dev.stream, Callback, &token)) return 100;
  g_dev.se.block_host_for_event(&g_dev.device, ev, &st);
  if (int rc = Check(st, "block_host_for_event")) return rc;
  if (g_dev.se.get_event_status(&g_dev.device, ev) != SE_EVENT_COMPLETE) return 101;
  g_dev.se.block_host_until_done(&g_dev.device, g_dev.stream, &st);
  if (int rc = Check(st, "block_host_until_done")) return rc;
  g_dev.se.get_stream_status(&g_dev.device, g_dev.stream, &st);
  if (int rc = Check(st, "get_stream_status")) return rc;
  for (int spin = 0; spin < 2000 && g_callback_ran != 7; ++spin) {  // the callback runs on a runtime thread
    struct timespec ts = {0, 1000000};
    nanosleep(&ts, nullptr);
  }
  SP_Timer timer = nullptr;
  g_dev.se.create_timer(&g_dev.device, &timer, &st);  // documented as unimplemented
  const bool timer_unimplemented = st.code == TF_UNIMPLEMENTED && g_dev.timer_fns.nanoseconds(timer) == 0;
  g_dev.se.destroy_event(&g_dev.device, ev);
  g_dev.se.destroy_stream(&g_dev.device, second);
  if (g_callback_ran != 7) return 102;
  return timer_unimplemented ? 0 : 103;
}

// dlopen the plugin and call its TF_InitKernel, as TensorFlow does
int mock_load_plugin(const char* path) {
  void* h = dlopen(path, RTLD_NOW | RTLD_GLOBAL);
  if (!h) { std::fprintf(stderr, "mock_tf: dlopen failed: %s\n", dlerror()); return 1; }
  auto init = reinterpret_cast<void (*)(void)>(dlsym(h, "TF_InitKernel"));
  if (!init) { std::fprintf(stderr, "mock_tf: TF_InitKernel not exported\n"); return 2; }
  init();
  return 0;
}

// ---- graph optimizer: TF_InitGraph, then create / optimize / destroy as TensorFlow's plugin optimizer wrapper does
static void* g_plugin_handle = nullptr;
static TP_Optimizer g_optimizer;
static TP_OptimizerConfigs g_optimizer_configs;
static std::string g_optimizer_device;
static std::string g_optimized;

// returns 0 and fills the registration state, or a nonzero code
int mock_graph_init(const char* path) {
  g_plugin_handle = dlopen(path, RTLD_NOW | RTLD_GLOBAL);
  if (!g_plugin_handle) return 1;
  auto init = reinterpret_cast<void (*)(TP_OptimizerRegistrationParams*, TF_Status*)>(dlsym(g_plugin_handle, "TF_InitGraph"));
  if (!init) return 2;
  std::memset(&g_optimizer, 0, sizeof(g_optimizer));
  std::memset(&g_optimizer_configs, 0, sizeof(g_optimizer_configs));
  TP_OptimizerRegistrationParams params;
  std::memset(&params, 0, sizeof(params));
  params.struct_size = TP_OPTIMIZER_REGISTRATION_PARAMS_STRUCT_SIZE;
  params.optimizer = &g_optimizer;
  params.optimizer_configs = &g_optimizer_configs;
  TF_Status st;
  init(&params, &st);
  if (st.code != TF_OK) return 3;
  // what TensorFlow validates (c_api_experimental grappler registration): sizes, device type, the three functions
  if (params.struct_size == 0 || g_optimizer.struct_size == 0 || g_optimizer_configs.struct_size == 0) return 4;
  if (!params.device_type || !params.device_type[0]) return 5;
  if (!g_optimizer.optimize_func) return 6;
  if (params.major_version != GO_MAJOR) return 7;
  g_optimizer_device = params.device_type;
  return 0;
}
const char* mock_graph_device_type(void) { return g_optimizer_device.c_str(); }
int mock_graph_config(const char* name) {
  const std::string n = name;
  if (n == "remapping") return g_optimizer_configs.remapping;
  if (n == "layout_optimizer") return g_optimizer_configs.layout_optimizer;
  if (n == "constant_folding") return g_optimizer_configs.constant_folding;
  return -1;
}
// the grappler item of a run: what the session fetches and what it asked to keep
struct TF_GrapplerItem {
  std::vector<std::string> preserve, fetch;
};
static void ListSize(const std::vector<std::string>& v, int* num_values, size_t* storage_size, TF_Status* status) {
  *num_values = static_cast<int>(v.size());
  *storage_size = 0;
  for (const std::string& s : v) *storage_size += s.size();
  status->code = TF_OK;
}
static void ListFill(const std::vector<std::string>& v, char** values, size_t* lengths, int num_values, void* storage,
                     size_t storage_size, TF_Status* status) {
  char* p = static_cast<char*>(storage);
  size_t used = 0;
  for (int i = 0; i < num_values && i < static_cast<int>(v.size()); ++i) {
    if (used + v[i].size() > storage_size) { status->code = TF_INVALID_ARGUMENT; return; }
    std::memcpy(p + used, v[i].data(), v[i].size());
    values[i] = p + used;
    lengths[i] = v[i].size();
    used += v[i].size();
  }
  status->code = TF_OK;
}
void TF_GetNodesToPreserveListSize(const TF_GrapplerItem* item, int* n, size_t* bytes, TF_Status* st) { ListSize(item->preserve, n, bytes, st); }
void TF_GetNodesToPreserveList(const TF_GrapplerItem* item, char** values, size_t* lengths, int n, void* storage, size_t bytes,
                               TF_Status* st) { ListFill(item->preserve, values, lengths, n, storage, bytes, st); }
void TF_GetFetchNodesListSize(const TF_GrapplerItem* item, int* n, size_t* bytes, TF_Status* st) { ListSize(item->fetch, n, bytes, st); }
void TF_GetFetchNodesList(const TF_GrapplerItem* item, char** values, size_t* lengths, int n, void* storage, size_t bytes,
                          TF_Status* st) { ListFill(item->fetch, values, lengths, n, storage, bytes, st); }

static std::vector<std::string> SplitCsv(const char* csv) {
  std::vector<std::string> out;
  if (!csv) return out;
  std::string cur;
  for (const char* c = csv; ; ++c) {
    if (*c == ',' || *c == 0) { if (!cur.empty()) out.push_back(cur); cur.clear(); if (*c == 0) break; }
    else cur.push_back(*c);
  }
  return out;
}

// runs the optimizer on a serialized GraphDef; the result is read with mock_graph_result / _size.  `preserve` / `fetch`:
// comma-separated node names of the grappler item (null: the optimizer gets no item at all)
int mock_graph_optimize_item(const void* graph, size_t len, const char* preserve, const char* fetch) {
  void* opt = g_optimizer.create_func ? g_optimizer.create_func() : nullptr;
  TF_Buffer in{graph, len, nullptr};
  TF_Buffer out{nullptr, 0, nullptr};
  TF_Status st;
  TF_GrapplerItem item{SplitCsv(preserve), SplitCsv(fetch)};
  g_optimizer.optimize_func(opt, &in, (preserve || fetch) ? &item : nullptr, &out, &st);
  if (g_optimizer.destroy_func) g_optimizer.destroy_func(opt);
  g_optimized.assign(static_cast<const char*>(out.data), out.length);
  if (out.data_deallocator) out.data_deallocator(const_cast<void*>(out.data), out.length);
  return st.code;
}
int mock_graph_optimize(const void* graph, size_t len) { return mock_graph_optimize_item(graph, len, nullptr, nullptr); }
const void* mock_graph_result(void) { return g_optimized.data(); }
size_t mock_graph_result_size(void) { return g_optimized.size(); }

static std::string Quote(const std::string& s) {
  std::string o = "\"";
  for (char c : s) { if (c == '"' || c == '\\') o.push_back('\\'); o.push_back(c); }
  return o + "\"";
}
const char* mock_dump_registry(void) {
  std::ostringstream os;
  os << "{\"kernels\":[";
  for (size_t i = 0; i < g_kernels.size(); ++i) {
    const auto& k = g_kernels[i];
    os << (i ? "," : "") << "{\"op\":" << Quote(k->op) << ",\"device\":" << Quote(k->device) << ",\"label\":" << Quote(k->label)
       << ",\"constraints\":{";
    for (size_t c = 0; c < k->constraints.size(); ++c)
      os << (c ? "," : "") << Quote(k->constraints[c].first) << ":" << static_cast<int>(k->constraints[c].second);
    os << "},\"host_memory\":[";
    for (size_t h = 0; h < k->host_memory.size(); ++h) os << (h ? "," : "") << Quote(k->host_memory[h]);
    os << "]}";
  }
  os << "],\"ops\":[";
  for (size_t i = 0; i < g_ops.size(); ++i) {
    const auto& o = g_ops[i];
    auto list = [&](const std::vector<std::string>& v) {
      os << "[";
      for (size_t j = 0; j < v.size(); ++j) os << (j ? "," : "") << Quote(v[j]);
      os << "]";
    };
    os << (i ? "," : "") << "{\"name\":" << Quote(o->name) << ",\"inputs\":";
    list(o->inputs);
    os << ",\"outputs\":";
    list(o->outputs);
    os << ",\"attrs\":";
    list(o->attrs);
    os << ",\"shape_fn\":" << (o->has_shape_fn ? "true" : "false") << "}";
  }
  os << "]}";
  g_json = os.str();
  return g_json.c_str();
}

void* mock_node_new(const char* op, const char* device) {
  auto* n = new Node;
  n->op = op;
  n->device = device;
  n->construction.name = std::string("test/") + op;
  return n;
}
static AttrValue& Attr(void* h, const char* name, AttrValue::Kind k) {
  AttrValue& a = static_cast<Node*>(h)->construction.attrs[name];
  a.kind = k;
  return a;
}
void mock_node_attr_string(void* h, const char* name, const char* v) { Attr(h, name, AttrValue::STRING).s = v; }
void mock_node_attr_int(void* h, const char* name, int64_t v) { Attr(h, name, AttrValue::INT).i = v; }
void mock_node_attr_float(void* h, const char* name, float v) { Attr(h, name, AttrValue::FLOAT).f = v; }
void mock_node_attr_bool(void* h, const char* name, int v) { Attr(h, name, AttrValue::BOOL).b = v != 0; }
void mock_node_attr_type(void* h, const char* name, int v) { Attr(h, name, AttrValue::TYPE).t = static_cast<TF_DataType>(v); }
void mock_node_attr_string_list(void* h, const char* name, const char** v, int n) {
  AttrValue& a = Attr(h, name, AttrValue::STRING_LIST);
  a.sl.assign(v, v + n);
}
void mock_node_attr_int_list(void* h, const char* name, const int64_t* v, int n) {
  AttrValue& a = Attr(h, name, AttrValue::INT_LIST);
  a.il.assign(v, v + n);
}
void mock_node_attr_type_list(void* h, const char* name, const int* v, int n) {
  AttrValue& a = Attr(h, name, AttrValue::TYPE_LIST);
  a.tl.clear();
  for (int i = 0; i < n; ++i) a.tl.push_back(static_cast<TF_DataType>(v[i]));
}

// kernel lookup by op, device and type constraints, then create().  Returns the TF_Code of construction
// (TF_NOT_FOUND when no kernel matches).
int mock_node_instantiate(void* h) {
  Node* n = static_cast<Node*>(h);
  n->kernel = nullptr;
  for (const auto& k : g_kernels) {
    if (k->op != n->op || k->device != n->device) continue;
    bool match = true;
    for (const auto& c : k->constraints) {
      auto it = n->construction.attrs.find(c.first);
      if (it == n->construction.attrs.end() || it->second.kind != AttrValue::TYPE || it->second.t != c.second) { match = false; break; }
    }
    if (match) { n->kernel = k.get(); break; }
  }
  if (!n->kernel) {
    n->construction.status.code = TF_NOT_FOUND;
    n->construction.status.msg = "No registered kernel for " + n->op + " on " + n->device;
    return TF_NOT_FOUND;
  }
  n->construction.status = TF_Status();
  n->object = n->kernel->create(&n->construction);
  if (n->construction.status.code != TF_OK && n->object) {  // TensorFlow deletes a kernel whose construction failed
    n->kernel->del(n->object);
    ++g_delete_calls;
    n->object = nullptr;
  }
  return n->construction.status.code;
}
const char* mock_node_construction_message(void* h) { return static_cast<Node*>(h)->construction.status.msg.c_str(); }

void mock_node_clear_io(void* h) {
  Node* n = static_cast<Node*>(h);
  for (auto& in : n->context.inputs) delete in.t;
  for (auto* o : n->context.outputs) delete o;
  n->context.inputs.clear();
  n->context.outputs.clear();
  n->context.forwarded_from.clear();
  n->context.out_dtypes.clear();
  n->context.out_on_host.clear();
  n->context.status = TF_Status();
}
// the tensor wraps caller-owned memory
void mock_node_add_input(void* h, int dtype, const int64_t* dims, int ndims, void* data, int on_host, int allow_forward) {
  Node* n = static_cast<Node*>(h);
  auto* t = new TF_Tensor;
  t->dtype = static_cast<TF_DataType>(dtype);
  t->dims.assign(dims, dims + ndims);
  t->buf = std::make_shared<Buffer>();
  int64_t cnt = 1;
  for (int64_t d : t->dims) cnt *= d;
  t->buf->bytes = static_cast<size_t>(cnt) * DtypeSize(t->dtype);
  t->buf->data = data;
  t->buf->owned = false;
  t->buf->on_host = on_host != 0;
  n->context.inputs.push_back({t, allow_forward != 0});
}
void mock_node_add_output(void* h, int dtype, int on_host) {
  Node* n = static_cast<Node*>(h);
  n->context.outputs.push_back(nullptr);
  n->context.forwarded_from.push_back(-1);
  n->context.out_dtypes.push_back(static_cast<TF_DataType>(dtype));
  n->context.out_on_host.push_back(static_cast<char>(on_host));
}
void mock_node_set_stream(void* h, void* stream) { static_cast<Node*>(h)->context.stream.stream_handle = stream; }
int mock_node_compute(void* h) {
  Node* n = static_cast<Node*>(h);
  if (!n->object) return TF_FAILED_PRECONDITION;
  n->context.status = TF_Status();
  n->kernel->compute(n->object, &n->context);
  return n->context.status.code;
}
const char* mock_node_compute_message(void* h) { return static_cast<Node*>(h)->context.status.msg.c_str(); }
int mock_node_temp_allocs(void* h) { return static_cast<Node*>(h)->context.temp_allocs; }
// returns 0 if the output was produced
int mock_node_output(void* h, int i, int* dtype, int64_t* dims, int* ndims, void** data, int* forwarded_from) {
  Node* n = static_cast<Node*>(h);
  if (i < 0 || i >= static_cast<int>(n->context.outputs.size()) || !n->context.outputs[i]) return 1;
  TF_Tensor* t = n->context.outputs[i];
  *dtype = t->dtype;
  *ndims = static_cast<int>(t->dims.size());
  for (int d = 0; d < *ndims && d < 8; ++d) dims[d] = t->dims[d];
  *data = t->buf->data;
  *forwarded_from = n->context.forwarded_from[i];
  return 0;
}
void mock_node_delete(void* h) {
  Node* n = static_cast<Node*>(h);
  mock_node_clear_io(h);
  if (n->object) { n->kernel->del(n->object); ++g_delete_calls; }
  delete n;
}

}  // extern "C"
