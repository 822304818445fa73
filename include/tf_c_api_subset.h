/*
 * tf_c_api_subset.h - the part of TensorFlow 2.15's public C API that the kernel plugin calls.
 *
 * TensorFlow's headers are not available to this build, so the opaque types and prototypes are
 * declared here with the signatures of tensorflow/c/{kernels.h, kernels_experimental.h, ops.h,
 * tf_tensor.h, tf_status.h, tf_datatype.h, tf_buffer.h} and
 * tensorflow/c/experimental/stream_executor/stream_executor.h.  Each group names the reference call
 * site that uses it (paths relative to the reference tree), which fixes the argument order.
 * The plugin library leaves these symbols undefined; the TensorFlow runtime that dlopen()s the
 * plugin (or the mock host used by the tests) provides them.
 */
#ifndef ITEX_AMD_TF_C_API_SUBSET_H_
#define ITEX_AMD_TF_C_API_SUBSET_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- tf_datatype.h ---------------------------------------------------------------------- */
typedef enum TF_DataType {
  TF_FLOAT = 1,
  TF_DOUBLE = 2,
  TF_INT32 = 3,
  TF_UINT8 = 4,
  TF_INT16 = 5,
  TF_INT8 = 6,
  TF_STRING = 7,
  TF_INT64 = 9,
  TF_BOOL = 10,
  TF_QINT8 = 11,
  TF_QUINT8 = 12,
  TF_QINT32 = 13,
  TF_BFLOAT16 = 14,
  TF_HALF = 19
} TF_DataType;

/* ---- tf_status.h (itex/core/utils/op_kernel.cc:883,900; op_kernel.h:843-851) -------------- */
typedef enum TF_Code {
  TF_OK = 0,
  TF_CANCELLED = 1,
  TF_UNKNOWN = 2,
  TF_INVALID_ARGUMENT = 3,
  TF_NOT_FOUND = 5,
  TF_ALREADY_EXISTS = 6,
  TF_FAILED_PRECONDITION = 9,
  TF_ABORTED = 10,
  TF_OUT_OF_RANGE = 11,
  TF_UNIMPLEMENTED = 12,
  TF_INTERNAL = 13
} TF_Code;
typedef struct TF_Status TF_Status;
TF_Status* TF_NewStatus(void);
void TF_DeleteStatus(TF_Status*);
void TF_SetStatus(TF_Status* s, TF_Code code, const char* msg);
TF_Code TF_GetCode(const TF_Status* s);
const char* TF_Message(const TF_Status* s);

/* ---- tf_tensor.h (op_kernel.cc:118-125; plugin_tensor.h:179-182,527) ----------------------- */
typedef struct TF_Tensor TF_Tensor;
void* TF_TensorData(const TF_Tensor*);
int TF_NumDims(const TF_Tensor*);
int64_t TF_Dim(const TF_Tensor* tensor, int dim_index);
TF_DataType TF_TensorType(const TF_Tensor*);
size_t TF_TensorByteSize(const TF_Tensor*);
int64_t TF_TensorElementCount(const TF_Tensor*);
void TF_DeleteTensor(TF_Tensor*);

/* ---- tf_buffer.h / c_api.h ----------------------------------------------------------------- */
typedef struct TF_Buffer {
  const void* data;
  size_t length;
  void (*data_deallocator)(void* data, size_t length);
} TF_Buffer;
void TF_DeleteBuffer(TF_Buffer*);
/* serialized OpList of every registered op (itex/core/ops/op_init.cc:31-59) */
TF_Buffer* TF_GetAllOpList(void);

typedef struct TF_StringView {
  const char* data;
  size_t len;
} TF_StringView;

/* ---- stream_executor.h: the stream struct body belongs to the plugin
 *      (itex/core/devices/gpu/gpu_device_plugin.h:23-26; op_kernel.h:406) ---------------------- */
typedef struct SP_Stream_st* SP_Stream;
struct SP_Stream_st {
  void* stream_handle; /* hipStream_t */
};

/* ---- kernels.h: registration (op_kernel.cc:883-929) ---------------------------------------- */
typedef struct TF_KernelBuilder TF_KernelBuilder;
typedef struct TF_OpKernelConstruction TF_OpKernelConstruction;
typedef struct TF_OpKernelContext TF_OpKernelContext;
TF_KernelBuilder* TF_NewKernelBuilder(const char* op_name, const char* device_name,
                                      void* (*create_func)(TF_OpKernelConstruction*),
                                      void (*compute_func)(void*, TF_OpKernelContext*),
                                      void (*delete_func)(void*));
void TF_KernelBuilder_TypeConstraint(TF_KernelBuilder* kernel_builder, const char* attr_name,
                                     const TF_DataType type, TF_Status* status);
void TF_KernelBuilder_HostMemory(TF_KernelBuilder* kernel_builder, const char* arg_name);
void TF_KernelBuilder_Priority(TF_KernelBuilder* kernel_builder, int32_t priority_number);
void TF_RegisterKernelBuilder(const char* kernel_name, TF_KernelBuilder* builder, TF_Status* status);

/* ---- kernels.h: construction (op_kernel.cc:539-633, 752, 777) ------------------------------ */
unsigned char TF_OpKernelConstruction_HasAttr(TF_OpKernelConstruction* ctx, const char* attr_name,
                                              TF_Status* status);
void TF_OpKernelConstruction_GetAttrSize(TF_OpKernelConstruction* ctx, const char* attr_name,
                                         int32_t* list_size, int32_t* total_size, TF_Status* status);
void TF_OpKernelConstruction_GetAttrType(TF_OpKernelConstruction* ctx, const char* attr_name,
                                         TF_DataType* val, TF_Status* status);
void TF_OpKernelConstruction_GetAttrInt32(TF_OpKernelConstruction* ctx, const char* attr_name,
                                          int32_t* val, TF_Status* status);
void TF_OpKernelConstruction_GetAttrInt64(TF_OpKernelConstruction* ctx, const char* attr_name,
                                          int64_t* val, TF_Status* status);
void TF_OpKernelConstruction_GetAttrFloat(TF_OpKernelConstruction* ctx, const char* attr_name,
                                          float* val, TF_Status* status);
void TF_OpKernelConstruction_GetAttrBool(TF_OpKernelConstruction* ctx, const char* attr_name,
                                         unsigned char* val, TF_Status* status);
void TF_OpKernelConstruction_GetAttrString(TF_OpKernelConstruction* ctx, const char* attr_name,
                                           char* val, size_t max_length, TF_Status* status);
void TF_OpKernelConstruction_GetAttrStringList(TF_OpKernelConstruction* ctx, const char* attr_name,
                                               char** values, size_t* lengths, int max_values,
                                               void* storage, size_t storage_size, TF_Status* status);
void TF_OpKernelConstruction_GetAttrTypeList(TF_OpKernelConstruction* ctx, const char* attr_name,
                                             TF_DataType* vals, int max_vals, TF_Status* status);
void TF_OpKernelConstruction_GetAttrInt64List(TF_OpKernelConstruction* ctx, const char* attr_name, int64_t* vals,
                                              int max_vals, TF_Status* status);
TF_StringView TF_OpKernelConstruction_GetName(TF_OpKernelConstruction* ctx);
void TF_OpKernelConstruction_Failure(TF_OpKernelConstruction* ctx, TF_Status* status);

/* ---- kernels.h: compute (op_kernel.cc:78-129, 234-238, 333-340, 437-443, 501, 511-518) ------ */
int TF_NumInputs(TF_OpKernelContext* ctx);
int TF_NumOutputs(TF_OpKernelContext* ctx);
/* the caller owns *tensor and releases it with TF_DeleteTensor */
void TF_GetInput(TF_OpKernelContext* ctx, int i, TF_Tensor** tensor, TF_Status* status);
void TF_SetOutput(TF_OpKernelContext* ctx, int i, const TF_Tensor* tensor, TF_Status* status);
TF_DataType TF_ExpectedOutputDataType(TF_OpKernelContext* ctx, int i);
TF_Tensor* TF_AllocateOutput(TF_OpKernelContext* context, int index, TF_DataType dtype,
                             const int64_t* dims, int num_dims, size_t len, TF_Status* status);
TF_Tensor* TF_ForwardInputOrAllocateOutput(TF_OpKernelContext* context, const int* candidate_input_indices,
                                           int num_candidate_input_indices, int output_index,
                                           const int64_t* output_dims, int output_num_dims,
                                           int* forwarded_input, TF_Status* status);
typedef struct TF_AllocatorAttributes {
  size_t struct_size;
  unsigned char on_host; /* 1: allocate in host memory */
} TF_AllocatorAttributes;
#define TF_ALLOCATOR_ATTRIBUTES_STRUCT_SIZE (offsetof(TF_AllocatorAttributes, on_host) + sizeof(unsigned char))
TF_Tensor* TF_AllocateTemp(TF_OpKernelContext* context, TF_DataType dtype, const int64_t* dims,
                           int num_dims, TF_AllocatorAttributes* alloc_attrs, TF_Status* status);
void TF_OpKernelContext_Failure(TF_OpKernelContext* ctx, TF_Status* status);
SP_Stream TF_GetStream(TF_OpKernelContext* ctx, TF_Status* status);
int64_t TF_StepId(TF_OpKernelContext* ctx);

/* ---- ops.h: op definitions for ops stock TensorFlow lacks (itex/core/ops/nn_ops.cc:379-416) -- */
typedef struct TF_OpDefinitionBuilder TF_OpDefinitionBuilder;
typedef struct TF_ShapeInferenceContext TF_ShapeInferenceContext;
TF_OpDefinitionBuilder* TF_NewOpDefinitionBuilder(const char* op_name);
void TF_OpDefinitionBuilderAddInput(TF_OpDefinitionBuilder* builder, const char* input_spec);
void TF_OpDefinitionBuilderAddOutput(TF_OpDefinitionBuilder* builder, const char* output_spec);
void TF_OpDefinitionBuilderAddAttr(TF_OpDefinitionBuilder* builder, const char* attr_spec);
void TF_OpDefinitionBuilderSetShapeInferenceFunction(
    TF_OpDefinitionBuilder* builder, void (*shape_inference_func)(TF_ShapeInferenceContext* ctx, TF_Status* status));
void TF_RegisterOpDefinition(TF_OpDefinitionBuilder* builder, TF_Status* status);
void TF_ShapeInferenceContextSetUnknownShape(TF_ShapeInferenceContext* ctx, TF_Status* status);

/* ---- the plugin's own entry point, looked up by TensorFlow after dlopen
 *      (itex/core/wrapper/itex_cpu_wrapper.cc:99-112 -> itex/core/kernels/xpu_kernel.cc:39) ----- */
void TF_InitKernel(void);

#ifdef __cplusplus
}
#endif
#endif /* ITEX_AMD_TF_C_API_SUBSET_H_ */
