/*
 * saga_capi.h - C API over the Saga front end (Graph / Node / Tensor) and the hip engine
 * (Context / Program).  One function per method of the C++ interface in saga.hpp that a
 * harness needs (saga.hpp:149-227 tensors, :328-403 graph, :520-570 program and context);
 * used by the Python tests and bench.py through ctypes.  Handles are opaque; every function
 * that can fail returns non-zero (or NULL) and leaves a message for saga_last_error().
 */
#ifndef SAGA_CAPI_H
#define SAGA_CAPI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *saga_tensor_t;
typedef void *saga_node_t;
typedef void *saga_graph_t;
typedef void *saga_context_t;
typedef void *saga_program_t;

/* symbolic extents (DimParam, saga.hpp:50-54) inside dims / shape arrays */
#define SAGA_DIM_BATCH (-1)
#define SAGA_DIM_UNCHANGED (-2)
#define SAGA_DIM_REDUCE (-3)

enum { SAGA_ATTR_INT = 0, SAGA_ATTR_FLOAT = 1, SAGA_ATTR_BOOL = 2, SAGA_ATTR_INTS = 3, SAGA_ATTR_DIMS = 4 };

typedef struct saga_attr {
    const char *name;
    int kind;
    int64_t i;
    double f;
    const int *ints;
    int n_ints;
} saga_attr_t;

/* ProgramConfig (saga.hpp:495-516) plus initial_loss_scale (0 = sum of batch sizes) */
typedef struct saga_program_config {
    float learning_rate;
    float l2_lambda;
    float bn_expavg;
    int tensor_layout; /* 0 auto, 1 NHWC, 2 NCHW */
    int anomaly_detect;
    int disable_op_fusing;
    float initial_loss_scale;
} saga_program_config_t;

const char *saga_last_error(void);

/* makeCPUTensor (with_storage) / makeTensor; dtype as Tensor::DataType */
saga_tensor_t saga_tensor_create(int dtype, int rank, const int64_t *dims, const char *name, int with_storage);
void saga_tensor_release(saga_tensor_t t);
saga_tensor_t saga_tensor_grad(saga_tensor_t t);
int saga_tensor_rank(saga_tensor_t t);
int saga_tensor_dtype(saga_tensor_t t);
int saga_tensor_dims(saga_tensor_t t, int64_t *out);
/* elements in logical row-major order, in the tensor's data type; works for host and device tensors */
int saga_tensor_write(saga_tensor_t t, const void *data, size_t bytes);
int saga_tensor_read(saga_tensor_t t, void *data, size_t bytes);
int saga_tensor_save(saga_tensor_t t, const char *path);
saga_tensor_t saga_tensor_load(const char *path, const char *name);
/* a file holding one ONNX TensorProto (Tensor::loadProtoBuf, reference src/onnx.cpp:777-790); NULL on failure */
saga_tensor_t saga_tensor_load_protobuf(const char *path);
double saga_tensor_sse(saga_tensor_t a, saga_tensor_t b);

saga_graph_t saga_graph_create(void);
void saga_graph_release(saga_graph_t g);
saga_node_t saga_graph_add_node(saga_graph_t g, const char *type, int n_inputs, const char *const *input_names,
                                const saga_tensor_t *inputs, int n_attrs, const saga_attr_t *attrs, const char *name);
saga_node_t saga_graph_add_resnet_bottleneck(saga_graph_t g, saga_tensor_t input, int squeeze, int output,
                                             int downsample, const char *name);
saga_node_t saga_graph_add_resnet(saga_graph_t g, saga_tensor_t input, int output, int downsample, const char *name);
/* ONNX model file -> graph (Graph::load, reference saga.hpp / src/onnx.cpp:750-775); NULL on failure */
saga_graph_t saga_graph_load(const char *path);
/* graph inputs (outputs != 0: outputs) in name order */
int saga_graph_io_count(saga_graph_t g, int outputs);
saga_tensor_t saga_graph_io(saga_graph_t g, int outputs, int index);
/* one text line per node: "type | slot=name:dtype[dims] ... | attr=value ... | slot=name:dtype[dims]";
   returns the length of the full text, writes at most capacity-1 characters plus a terminator */
int saga_graph_describe(saga_graph_t g, char *buf, size_t capacity);
int saga_graph_node_count(saga_graph_t g);
int saga_graph_save_tensors(saga_graph_t g, const char *path, saga_context_t ctx);
int saga_graph_load_tensors(saga_graph_t g, const char *path);
saga_tensor_t saga_graph_named_tensor(saga_graph_t g, const char *name);

void saga_node_release(saga_node_t n);
saga_tensor_t saga_node_output(saga_node_t n, const char *slot);
saga_tensor_t saga_node_input(saga_node_t n, const char *slot);

saga_context_t saga_context_create(void);
void saga_context_release(saga_context_t c);
int saga_context_reset(saga_context_t c);
saga_tensor_t saga_context_resolve(saga_context_t c, saga_tensor_t t);
/* Storage reuse of the context (the role of the reference's liveness + best-fit layout,
 * src/cuda/cuda_analysis.cpp:194-547): bytes of the shared arena and the sum of the sizes of the
 * storages laid out in it.  Both 0 before a program is finalized or with SAGA_HIP_NO_ARENA set. */
int saga_context_memory(saga_context_t c, size_t *arena_bytes, size_t *planned_bytes);

/* phases: 1 PRE, 2 POST, 3 both */
saga_program_t saga_program_create(saga_context_t c, saga_graph_t g, int batch_size, int training,
                                   const saga_program_config_t *cfg, int n_batched, const saga_tensor_t *batched,
                                   const int *phases);
void saga_program_release(saga_program_t p);
int saga_program_finalize(saga_program_t p);
int saga_program_run(saga_program_t p, long batches);
double saga_program_loss_scale(saga_program_t p);
int saga_program_dump(saga_program_t p, const char *path, int detailed);

/* Optimizer state of a training program: Adam's moments and step counts, the fp32 master weights of
 * mixed precision and the loss scale, keyed by tensor name ("sagaO001" file).  No counterpart in the
 * reference, which saves tensors only (Graph::saveTensors, src/graph.cpp:60-104) and so restarts the
 * optimizer after a reload.  Load into a program built from the same graph after its weights are in
 * place; every trained tensor needs a name. */
int saga_program_save_optimizer(saga_program_t p, const char *path);
int saga_program_load_optimizer(saga_program_t p, const char *path);

/* Per-operation-kind timing (HIP events on the program's stream around every operation) with the
 * algorithmic flops / bytes of the timed launches.  No counterpart in the reference, whose only
 * timing is samples per second (src/cuda/cuda_program.cpp:309-312). */
typedef struct saga_profile_row {
    char kind[48];
    long launches;
    double ms;
    double flops;
    double bytes;
} saga_profile_row_t;
int saga_program_set_profiling(saga_program_t p, int on);
int saga_program_profile(saga_program_t p, saga_profile_row_t *rows, int capacity);

#ifdef __cplusplus
}
#endif
#endif
