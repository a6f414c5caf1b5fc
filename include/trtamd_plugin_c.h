/*
 * Flat C view of the IPluginV3 objects in libtrtamd_bert_plugins.so, for hosts that cannot call
 * C++ virtual functions (ctypes, cgo, JNI ...).  Each function forwards to exactly one interface
 * method of include/NvInferRuntime.h / include/NvInferRuntimePlugin.h; the TensorRT Python
 * bindings expose the same operations (python/src/infer/pyPlugin.cpp: IPluginRegistry.get_creator,
 * IPluginCreatorV3One.create_plugin, IPluginV3OneBuild.get_output_shapes / configure_plugin /
 * supports_format_combination / get_workspace_size, IPluginV3OneRuntime.on_shape_change / enqueue /
 * get_fields_to_serialize).
 *
 * A C++ host does not need this file: it includes trtamd_nvinfer_api.h (or the real NvInfer
 * headers) and talks to getPluginRegistry() directly.
 */
#ifndef TRTAMD_PLUGIN_C_H
#define TRTAMD_PLUGIN_C_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TRTAMD_PLUGIN_API __attribute__((visibility("default")))
#define TRTAMD_MAX_DIMS 8

/* nvinfer1::PluginField, same memory layout (include/NvInferRuntimePlugin.h:703-741). */
typedef struct trtamd_plugin_field
{
    char const* name;
    void const* data;
    int32_t type;   /* nvinfer1::PluginFieldType */
    int32_t length;
} trtamd_plugin_field;

/* nvinfer1::DynamicPluginTensorDesc flattened; for the runtime calls only dims/type/format/scale
 * are read. */
typedef struct trtamd_tensor_desc
{
    int32_t nb_dims;
    int64_t dims[TRTAMD_MAX_DIMS];
    int64_t min[TRTAMD_MAX_DIMS];
    int64_t max[TRTAMD_MAX_DIMS];
    int64_t opt[TRTAMD_MAX_DIMS];
    int32_t type;   /* nvinfer1::DataType */
    int32_t format; /* nvinfer1::TensorFormat */
    float scale;
} trtamd_tensor_desc;

typedef void* trtamd_creator_t; /* nvinfer1::IPluginCreatorV3One* */
typedef void* trtamd_plugin_t;  /* nvinfer1::IPluginV3* */

/* getPluginRegistry()->getCreator(name, version, ns); NULL when nothing is registered. */
TRTAMD_PLUGIN_API trtamd_creator_t trtamd_plugin_get_creator(char const* name, char const* version, char const* ns);
/* getPluginRegistry()->getAllCreators(): number of creators; names/versions of creator i. */
TRTAMD_PLUGIN_API int32_t trtamd_plugin_num_creators(void);
TRTAMD_PLUGIN_API char const* trtamd_plugin_creator_name(int32_t index);
TRTAMD_PLUGIN_API char const* trtamd_plugin_creator_version(int32_t index);
/* IPluginCreatorV3One::getFieldNames(): returns nbFields, *fields points at creator-owned storage. */
TRTAMD_PLUGIN_API int32_t trtamd_plugin_creator_field_names(trtamd_creator_t creator, trtamd_plugin_field const** fields);
/* IPluginCreatorV3One::createPlugin(name, fc, phase); phase 0 = kBUILD, 1 = kRUNTIME.  NULL on failure. */
TRTAMD_PLUGIN_API trtamd_plugin_t trtamd_plugin_create(trtamd_creator_t creator, char const* layer_name,
    trtamd_plugin_field const* fields, int32_t nb_fields, int32_t phase);
/* delete plugin */
TRTAMD_PLUGIN_API void trtamd_plugin_destroy(trtamd_plugin_t plugin);
/* IPluginV3::clone() */
TRTAMD_PLUGIN_API trtamd_plugin_t trtamd_plugin_clone(trtamd_plugin_t plugin);
/* IPluginV3OneCore */
TRTAMD_PLUGIN_API char const* trtamd_plugin_name(trtamd_plugin_t plugin);
TRTAMD_PLUGIN_API char const* trtamd_plugin_version(trtamd_plugin_t plugin);
TRTAMD_PLUGIN_API char const* trtamd_plugin_namespace(trtamd_plugin_t plugin);
/* IPluginV3OneBuild */
TRTAMD_PLUGIN_API int32_t trtamd_plugin_nb_outputs(trtamd_plugin_t plugin);
TRTAMD_PLUGIN_API int32_t trtamd_plugin_output_types(
    trtamd_plugin_t plugin, int32_t* out_types, int32_t nb_outputs, int32_t const* in_types, int32_t nb_inputs);
/* getOutputShapes with every input extent a constant: in[i].dims are the extents, out[i].nb_dims
 * and out[i].dims receive the evaluated expressions. */
TRTAMD_PLUGIN_API int32_t trtamd_plugin_output_shapes(trtamd_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc* out, int32_t nb_outputs);
/* in_out holds nb_inputs input descriptors followed by nb_outputs output descriptors. */
TRTAMD_PLUGIN_API int32_t trtamd_plugin_supports_format(
    trtamd_plugin_t plugin, int32_t pos, trtamd_tensor_desc const* in_out, int32_t nb_inputs, int32_t nb_outputs);
TRTAMD_PLUGIN_API int32_t trtamd_plugin_configure(trtamd_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc const* out, int32_t nb_outputs);
TRTAMD_PLUGIN_API size_t trtamd_plugin_workspace_size(trtamd_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc const* out, int32_t nb_outputs);
/* IPluginV3OneRuntime */
TRTAMD_PLUGIN_API int32_t trtamd_plugin_on_shape_change(trtamd_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc const* out, int32_t nb_outputs);
TRTAMD_PLUGIN_API int32_t trtamd_plugin_enqueue(trtamd_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc const* out, int32_t nb_outputs, void const* const* inputs,
    void* const* outputs, void* workspace, void* stream);
/* getFieldsToSerialize(): returns nbFields (-1 on failure); storage is owned by the plugin and
 * valid until its next getFieldsToSerialize call or destruction. */
TRTAMD_PLUGIN_API int32_t trtamd_plugin_fields_to_serialize(trtamd_plugin_t plugin, trtamd_plugin_field const** fields);

/* ---- the deprecated IPluginV2DynamicExt / IPluginCreator versions ("Legacy" plugins of the reference:
 *      emb 1-3, skip 1-4, qkv 1-3; plugin/bertQKVToContextPlugin/qkvToContextPluginLegacy.cpp:46-48 and
 *      siblings).  One function per interface method, as above. ------------------------------------- */
typedef void* trtamd_legacy_creator_t; /* nvinfer1::IPluginCreator* */
typedef void* trtamd_legacy_plugin_t;  /* nvinfer1::IPluginV2DynamicExt* */

/* registry lookup restricted to IPluginCreator ("PLUGIN CREATOR_V1") creators */
TRTAMD_PLUGIN_API trtamd_legacy_creator_t trtamd_legacy_get_creator(char const* name, char const* version, char const* ns);
TRTAMD_PLUGIN_API int32_t trtamd_legacy_creator_field_names(trtamd_legacy_creator_t creator,
    trtamd_plugin_field const** fields);
/* IPluginCreator::createPlugin(name, fc) / deserializePlugin(name, data, length); NULL on failure */
TRTAMD_PLUGIN_API trtamd_legacy_plugin_t trtamd_legacy_create(trtamd_legacy_creator_t creator, char const* layer_name,
    trtamd_plugin_field const* fields, int32_t nb_fields);
TRTAMD_PLUGIN_API trtamd_legacy_plugin_t trtamd_legacy_deserialize(trtamd_legacy_creator_t creator,
    char const* layer_name, void const* data, size_t length);
/* IPluginV2::destroy(), clone(), getPluginType(), getPluginVersion(), getNbOutputs(), getTensorRTVersion() */
TRTAMD_PLUGIN_API void trtamd_legacy_destroy(trtamd_legacy_plugin_t plugin);
TRTAMD_PLUGIN_API trtamd_legacy_plugin_t trtamd_legacy_clone(trtamd_legacy_plugin_t plugin);
TRTAMD_PLUGIN_API char const* trtamd_legacy_type(trtamd_legacy_plugin_t plugin);
TRTAMD_PLUGIN_API char const* trtamd_legacy_version(trtamd_legacy_plugin_t plugin);
TRTAMD_PLUGIN_API int32_t trtamd_legacy_nb_outputs(trtamd_legacy_plugin_t plugin);
TRTAMD_PLUGIN_API int32_t trtamd_legacy_tensorrt_version(trtamd_legacy_plugin_t plugin);
/* initialize() / terminate() */
TRTAMD_PLUGIN_API int32_t trtamd_legacy_initialize(trtamd_legacy_plugin_t plugin);
TRTAMD_PLUGIN_API void trtamd_legacy_terminate(trtamd_legacy_plugin_t plugin);
/* getSerializationSize() / serialize(buffer) */
TRTAMD_PLUGIN_API size_t trtamd_legacy_serialization_size(trtamd_legacy_plugin_t plugin);
TRTAMD_PLUGIN_API void trtamd_legacy_serialize(trtamd_legacy_plugin_t plugin, void* buffer);
/* getOutputDataType(index, inputTypes, nbInputs) */
TRTAMD_PLUGIN_API int32_t trtamd_legacy_output_type(
    trtamd_legacy_plugin_t plugin, int32_t index, int32_t const* in_types, int32_t nb_inputs);
/* getOutputDimensions(index, inputs, nbInputs, exprBuilder) with constant extents; returns 0 on success */
TRTAMD_PLUGIN_API int32_t trtamd_legacy_output_dims(trtamd_legacy_plugin_t plugin, int32_t index,
    trtamd_tensor_desc const* in, int32_t nb_inputs, trtamd_tensor_desc* out);
TRTAMD_PLUGIN_API int32_t trtamd_legacy_supports_format(trtamd_legacy_plugin_t plugin, int32_t pos,
    trtamd_tensor_desc const* in_out, int32_t nb_inputs, int32_t nb_outputs);
TRTAMD_PLUGIN_API void trtamd_legacy_configure(trtamd_legacy_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc const* out, int32_t nb_outputs);
TRTAMD_PLUGIN_API size_t trtamd_legacy_workspace_size(trtamd_legacy_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc const* out, int32_t nb_outputs);
TRTAMD_PLUGIN_API int32_t trtamd_legacy_enqueue(trtamd_legacy_plugin_t plugin, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc const* out, int32_t nb_outputs, void const* const* inputs,
    void* const* outputs, void* workspace, void* stream);

/* Log capture: when enabled, an ILogger that remembers the last message of severity kERROR or
 * worse is installed (through initLibNvInferPlugins); trtamd_plugin_last_log returns that
 * message ("" if none) and clears it. */
TRTAMD_PLUGIN_API void trtamd_plugin_capture_log(int32_t enable);
TRTAMD_PLUGIN_API char const* trtamd_plugin_last_log(void);

#ifdef __cplusplus
}
#endif

#endif /* TRTAMD_PLUGIN_C_H */
