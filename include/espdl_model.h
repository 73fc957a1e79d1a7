/*
 * espdl_model.h — C handle API over the C++ host layer (dl::Model, fbs::FbsModel) of
 * libespdl_dl.so, for callers that cannot include C++ headers (Python ctypes, C, other FFIs).
 *
 * The reference exposes this level only as C++ classes; each function names the member it wraps:
 *   graph construction      -> the content an fbs::FbsModel holds (esp-dl/fbs_loader/espdl.fbs:80-145;
 *                              accessor side esp-dl/fbs_loader/include/fbs_model.hpp:23-424)
 *   espdl_model_create      -> dl::Model::Model(fbs::FbsModel*) + load + build
 *                              (esp-dl/dl/model/include/dl_model_base.hpp:150-165, 189-264)
 *   espdl_model_run*        -> dl::Model::run (dl_model_base.hpp:274-310)
 *   espdl_model_test        -> dl::Model::test (dl_model_base.hpp:324)
 *   espdl_model_profile     -> dl::Model::profile / get_module_info (dl_model_base.hpp:331-368)
 *   espdl_model_get_tensor* -> dl::Model::get_input / get_output / get_intermediate (:375-421)
 * All functions return 0 on success and a negative value on failure unless stated otherwise.
 * Host pointers are plain C buffers; nothing here takes or returns a C++ or torch type.
 */
#ifndef ESPDL_MODEL_H
#define ESPDL_MODEL_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct espdl_graph espdl_graph;
typedef struct espdl_model espdl_model;

/* dtype codes = TensorDataType of the .espdl schema (espdl.fbs:24-39): 3 int8, 5 int16, 6 int32, 7 int64 */
#define ESPDL_DTYPE_INT8 3
#define ESPDL_DTYPE_INT16 5
#define ESPDL_DTYPE_INT32 6
#define ESPDL_DTYPE_INT64 7

espdl_graph *espdl_graph_create(const char *name);
void espdl_graph_destroy(espdl_graph *g);
/* A graph read from an `.espdl` container (what fbs::FbsLoader::load does,
 * esp-dl/fbs_loader/src/fbs_loader.cpp:276-360): EDL1 / EDL2 files and PDL1 / PDL2 packages (model_index
 * selects the model, 0 for single-model files), plain payloads only.  Filters stored in the blocked
 * ESP32-S3 / ESP32-P4 order are rewritten to the N-major order the kernels read.  Embedded test vectors
 * become the graph's test inputs / outputs.  NULL on failure, reason in espdl_graph_load_error(). */
espdl_graph *espdl_graph_load_file(const char *path, int32_t model_index);
espdl_graph *espdl_graph_load_memory(const void *data, int64_t size, int32_t model_index);
const char *espdl_graph_load_error(void);
int32_t espdl_graph_input_count(espdl_graph *g);
int32_t espdl_graph_output_count(espdl_graph *g);
/* Copies the bytes of a constant tensor (after any re-layout) into dst when capacity allows; returns
 * its size in bytes, -1 when there is no such initializer. */
int64_t espdl_graph_initializer_bytes(espdl_graph *g, const char *name, void *dst, int64_t capacity);
/* Nodes in execution order, and whether an operator type has a module in this build
 * (ModuleCreator::register_module adds more, esp-dl/dl/module/include/dl_module_creator.hpp:107). */
int32_t espdl_graph_node_count(espdl_graph *g);
const char *espdl_graph_node_op_type(espdl_graph *g, int32_t index);
int32_t espdl_module_is_registered(const char *op_type);
/* Valid until the next call on this thread. */
const char *espdl_graph_input_name(espdl_graph *g, int32_t index);
const char *espdl_graph_output_name(espdl_graph *g, int32_t index);
/* A constant tensor (filter, bias, LUT, PReLU slope, Clip bound); `data` is a host buffer that is copied. */
int espdl_graph_add_initializer(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                                const void *data, const int32_t *exponents, int32_t n_exponents);
/* Shape (per image, leading 1), dtype and exponent of an activation. */
int espdl_graph_add_value_info(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                               int32_t exponent);
int espdl_graph_add_input(espdl_graph *g, const char *name);
int espdl_graph_add_output(espdl_graph *g, const char *name);
int espdl_graph_add_node(espdl_graph *g, const char *name, const char *op_type, const char *const *inputs,
                         int32_t n_inputs, const char *const *outputs, int32_t n_outputs);
int espdl_graph_node_set_int(espdl_graph *g, const char *node, const char *key, int64_t value);
int espdl_graph_node_set_float(espdl_graph *g, const char *node, const char *key, float value);
int espdl_graph_node_set_ints(espdl_graph *g, const char *node, const char *key, const int64_t *values, int32_t n);
int espdl_graph_node_set_string(espdl_graph *g, const char *node, const char *key, const char *value);
/* Known-answer vectors checked by espdl_model_test (whole-batch tensors). */
int espdl_graph_add_test_input(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                               const void *data, int32_t exponent);
int espdl_graph_add_test_output(espdl_graph *g, const char *name, const int32_t *dims, int32_t n_dims, int32_t dtype,
                                const void *data, int32_t exponent);

/* round_mode: 0 half-up (portable C path), 1 half-even.  stream: hipStream_t or NULL (own stream).
 * fuse: bit mask of graph fusions, all exact: 1 folds Conv -> LUT pairs into the conv epilogue, 2 runs
 * depthwise Conv -> 1x1 Conv [-> Add] chains as one kernel, 4 folds the Add behind a dense Conv into the
 * conv epilogue, 8 runs a 1x1 Conv and the GlobalAveragePool behind it as one kernel, 16 keeps the outputs of a
 * Split along the last axis inside its input and lets dense 8-bit Convs write straight into the output of a
 * Concat along the last axis, so that neither copies (31 = all).  The graph must outlive the model. */
espdl_model *espdl_model_create(espdl_graph *g, int32_t batch, int32_t round_mode, void *stream, int32_t fuse);
void espdl_model_destroy(espdl_model *m);
/* Module::forward returns void, as in the reference, so a module whose launch is rejected (an operand
 * that is not on the device, a shape a kernel refuses) can only log.  The model counts what is logged
 * during a pass: run / run_async / synchronize return -2 when a module of the current pass logged an
 * error or a HIP call failed; the tensors of such a pass are not valid results.  enable_graph refuses to
 * capture a plan with a failing module. */
int espdl_model_run(espdl_model *m);       /* enqueue + wait */
int espdl_model_run_async(espdl_model *m); /* enqueue only   */
int espdl_model_synchronize(espdl_model *m);
int espdl_model_enable_graph(espdl_model *m); /* HIP-graph replay of the plan; 0 on success */
int espdl_model_disable_graph(espdl_model *m);
int espdl_model_test(espdl_model *m);
int espdl_model_module_count(espdl_model *m);
/* Per-module timing: fills up to `capacity` entries, returns the module count.
 * names[i] points into storage owned by the model and valid until the next call. */
int espdl_model_profile(espdl_model *m, int32_t repeats, int32_t capacity, const char **names, const char **types,
                        float *latency_us, int64_t *macs, int64_t *bytes);
void espdl_model_print_profile(espdl_model *m);
/* Tensor access by name (input, output or intermediate): device pointer, byte size, shape, exponent. */
void *espdl_model_tensor_device_ptr(espdl_model *m, const char *name);
int64_t espdl_model_tensor_bytes(espdl_model *m, const char *name);
int espdl_model_tensor_shape(espdl_model *m, const char *name, int32_t *dims, int32_t capacity); /* returns rank */
int espdl_model_tensor_exponent(espdl_model *m, const char *name, int32_t *exponent);
/* Elements from one position of the last axis to the next at the device pointer: the last dim for a dense
 * tensor, more for an activation the model keeps inside a wider one (fuse bit 16); -1 for an unknown name.
 * espdl_model_get_tensor always delivers dense data. */
int espdl_model_tensor_channel_pitch(espdl_model *m, const char *name);
int espdl_model_set_input(espdl_model *m, const char *name, const void *host_data, int64_t bytes);
int espdl_model_get_tensor(espdl_model *m, const char *name, void *host_data, int64_t bytes);
int64_t espdl_model_device_bytes(espdl_model *m);
void *espdl_model_stream(espdl_model *m);

#ifdef __cplusplus
}
#endif
#endif /* ESPDL_MODEL_H */
