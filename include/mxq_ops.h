/*
 * mxq_ops.h - C entry points of libmxq_ops.so, the C++ operator host library.
 *
 * libmxq_ops.so holds the NNVM-style registry with the INT8 operators registered
 * under the reference's names and the FCompute<gpu> / FStatefulCompute<gpu> host
 * functions, which call libmxq_hip.so (mxq.h).  The functions below are the small
 * imperative front door a test harness or a language binding uses to drive one
 * operator: they play the role of MXImperativeInvoke
 * (src/c_api/c_api_ndarray.cc:146 in the reference: parse attributes, infer shape
 * and type, hand TBlobs + OpContext to the registered compute function) without
 * the engine, NDArray and storage layers around it.  The caller owns all memory.
 * Return 0 on success, -1 on failure with the text in mxq_ops_last_error().
 */
#ifndef MXQ_OPS_H_
#define MXQ_OPS_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MXQ_MAX_NDIM 8

/* One tensor argument: device pointer, shape, mshadow type flag (mxq.h codes). */
typedef struct {
  void* data;
  int ndim;
  int64_t shape[MXQ_MAX_NDIM];
  int dtype;
} mxq_blob;

const char* mxq_ops_last_error(void);

/* registry introspection */
int mxq_op_count(void);
const char* mxq_op_name(int index);
/* 1 if `op` (name or alias) has the attribute key, e.g. "FCompute<gpu>". */
int mxq_op_has_attr(const char* op, const char* key);

/* A node = operator + parsed attribute dict (nnvm::NodeAttrs). */
int mxq_node_create(const char* op, const char* node_name, int num_attrs, const char** keys,
                    const char** values, void** out_node);
int mxq_node_free(void* node);
int mxq_node_num_inputs(void* node, int* out);
int mxq_node_num_outputs(void* node, int* out);
/* comma-separated names; the string lives as long as the node */
int mxq_node_input_names(void* node, const char** out);
int mxq_node_output_names(void* node, const char** out);
/* FGradient: "operator:node name" of the gradient node made for every input, comma-separated
 * ("" for an operator registered without one); the string lives as long as the node */
int mxq_node_gradient_names(void* node, const char** out);

/* FInferShape / FInferType: unknown shapes have ndim -1, unknown types are -1;
 * both arrays are updated in place. */
int mxq_node_infer_shape(void* node, int num_in, int* in_ndim, int64_t* in_shape, int num_out,
                         int* out_ndim, int64_t* out_shape);
int mxq_node_infer_type(void* node, int num_in, int* in_type, int num_out, int* out_type);
/* bytes of ResourceRequest::kTempSpace the node will ask for (0 if none) */
int mxq_node_temp_bytes(void* node, int num_in, const mxq_blob* in, int num_out,
                        const mxq_blob* out, size_t* bytes);
/* runs FCompute<gpu> or FCreateOpState + FStatefulCompute<gpu> on `stream` */
int mxq_node_forward(void* node, void* stream, int dev_id, int num_in, const mxq_blob* in,
                     int num_out, const mxq_blob* out, void* temp_space, size_t temp_bytes);

/* ---- graph passes over symbol JSON ------------------------------------------------
 * Counterparts of MXQuantizeSymbol and MXSetCalibTableToQuantizedSymbol
 * (src/c_api/c_api_symbolic.cc:916-972, 1031-1050) with the symbol passed as the text
 * of its `-symbol.json`.  dev_type is Context::DeviceType (1 cpu, 2 gpu): a float
 * operator is replaced only if its quantized counterpart has a compute function for
 * that device.  Returned strings belong to the calling thread and stay valid until its
 * next call into this library. */
int mxq_quantize_symbol(const char* symbol_json, int dev_type, int num_excluded_nodes,
                        const char** excluded_nodes, int num_excluded_ops,
                        const char** excluded_ops, int num_offline, const char** offline_params,
                        const char* quantized_dtype, const char* quantize_mode,
                        const char* quantize_granularity, const char** out_symbol_json,
                        int* out_num_calib_names, const char*** out_calib_names);
int mxq_set_calib_table(const char* qsymbol_json, int num_layers, const char** layer_names,
                        const float* min_ranges, const float* max_ranges,
                        const char** out_symbol_json);
/* Loads and re-saves a symbol: nodes reachable from the heads, renumbered in
 * depth-first post-order, as the reference writes them. */
int mxq_symbol_normalize(const char* symbol_json, const char** out_symbol_json);

/* _contrib_calibrate_entropy (src/operator/quantization/calibrate.cc:89-186); host
 * arrays: hist[num_bins] (num_bins odd), hist_edges[num_bins + 1]. */
int mxq_calibrate_entropy(const float* hist, const float* hist_edges, size_t num_bins,
                          int num_quantized_bins, float* out_threshold, float* out_divergence);

/* ---- NDArray list files (`.params`, mx.nd.save / mx.nd.load) ------------------------
 * src/ndarray/ndarray.cc:1856-2146: dense arrays of the V2 / V3 record layouts plus the
 * two legacy layouts on load; V2 (np_shape = 0) or V3 records on save.  Arrays live in
 * host memory (mxq_blob.data is a host pointer here); what mxq_ndlist_get returns stays
 * valid until mxq_ndlist_free. */
int mxq_ndlist_load(const char* path, void** out_handle, int* out_count, int* out_has_names);
int mxq_ndlist_get(void* handle, int index, const char** out_name, int* out_is_none,
                   int* out_dtype, int* out_ndim, const int64_t** out_shape,
                   const void** out_data, size_t* out_bytes);
int mxq_ndlist_free(void* handle);
int mxq_ndlist_save(const char* path, int count, const char** names, const mxq_blob* arrays,
                    int np_shape);

#ifdef __cplusplus
}
#endif
#endif /* MXQ_OPS_H_ */
