/* The part of TensorFlow's graph-optimizer plugin C API that TF_InitGraph needs
 * (tensorflow/c/experimental/grappler/grappler.h of TF 2.15).  TensorFlow headers are not available to
 * this build, so the declarations are restated here; the struct layouts were written from the public
 * header and could not be compiled against a real TensorFlow.  TF_Buffer and TF_Status come from
 * tf_c_api_subset.h. */
#ifndef ITEX_AMD_TF_GRAPPLER_SUBSET_H_
#define ITEX_AMD_TF_GRAPPLER_SUBSET_H_

#include <stddef.h>
#include <stdint.h>

#include "tf_c_api_subset.h"

#ifdef __cplusplus
extern "C" {
#endif

#define GO_MAJOR 0
#define GO_MINOR 0
#define GO_PATCH 1

typedef enum TF_TriState { TF_TriState_Default = 0, TF_TriState_Off, TF_TriState_On } TF_TriState;

typedef struct TF_GrapplerItem TF_GrapplerItem;

/* switches for TensorFlow's own optimizers while this plugin's optimizer is registered */
typedef struct TP_OptimizerConfigs {
  size_t struct_size;
  void* ext;
  TF_TriState disable_model_pruning;
  TF_TriState implementation_selector;
  TF_TriState function_optimization;
  TF_TriState common_subgraph_elimination;
  TF_TriState arithmetic_optimization;
  TF_TriState debug_stripper;
  TF_TriState constant_folding;
  TF_TriState shape_optimization;
  TF_TriState auto_mixed_precision;
  TF_TriState auto_mixed_precision_onednn_bfloat16;
  TF_TriState auto_mixed_precision_mkl;
  TF_TriState pin_to_host_optimization;
  TF_TriState layout_optimizer;
  TF_TriState remapping;
  TF_TriState loop_optimization;
  TF_TriState dependency_optimization;
  TF_TriState auto_parallel;
  TF_TriState memory_optimization;
  TF_TriState scoped_allocator_optimization;
} TP_OptimizerConfigs;
#define TP_OPTIMIZER_CONFIGS_STRUCT_SIZE (offsetof(TP_OptimizerConfigs, scoped_allocator_optimization) + sizeof(TF_TriState))

typedef struct TP_Optimizer {
  size_t struct_size;
  void* ext;
  void* (*create_func)(void);
  /* graph_buf / optimized_graph_buf hold serialized GraphDef protos; the callee allocates the output's data
   * and sets its data_deallocator */
  void (*optimize_func)(void* optimizer, const TF_Buffer* graph_buf, const TF_GrapplerItem* item,
                        TF_Buffer* optimized_graph_buf, TF_Status* status);
  void (*destroy_func)(void* optimizer);
} TP_Optimizer;
#define TP_OPTIMIZER_STRUCT_SIZE (offsetof(TP_Optimizer, destroy_func) + sizeof(void (*)(void*)))

typedef struct TP_OptimizerRegistrationParams {
  size_t struct_size;
  void* ext;
  int32_t major_version;
  int32_t minor_version;
  int32_t patch_version;
  const char* device_type;
  TP_OptimizerConfigs* optimizer_configs;
  TP_Optimizer* optimizer;
} TP_OptimizerRegistrationParams;
#define TP_OPTIMIZER_REGISTRATION_PARAMS_STRUCT_SIZE (offsetof(TP_OptimizerRegistrationParams, optimizer) + sizeof(TP_Optimizer*))

/* Provided by TensorFlow: the names a rewrite must keep (the item's fetch nodes and its nodes to preserve).  Called as
 * the reference does (itex/core/graph/utils/grappler_item.cc:23-68): size query first, then the list into caller-owned
 * storage; values[i] / lengths[i] are not NUL-terminated. */
void TF_GetNodesToPreserveListSize(const TF_GrapplerItem* item, int* num_values, size_t* storage_size, TF_Status* status);
void TF_GetNodesToPreserveList(const TF_GrapplerItem* item, char** values, size_t* lengths, int num_values, void* storage,
                               size_t storage_size, TF_Status* status);
void TF_GetFetchNodesListSize(const TF_GrapplerItem* item, int* num_values, size_t* storage_size, TF_Status* status);
void TF_GetFetchNodesList(const TF_GrapplerItem* item, char** values, size_t* lengths, int num_values, void* storage,
                          size_t storage_size, TF_Status* status);

/* looked up by TensorFlow after dlopen of the plugin */
void TF_InitGraph(TP_OptimizerRegistrationParams* params, TF_Status* status);

#ifdef __cplusplus
}
#endif
#endif /* ITEX_AMD_TF_GRAPPLER_SUBSET_H_ */
