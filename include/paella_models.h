/*
 * paella_models.h -- C-ABI of the model zoo and graph executor that stand where the reference has
 * TVM-compiled model libraries.
 *
 * In the reference every model adapter loads "<model>-cuda_llis-pack.so" through the TVM runtime and calls
 * its "run" function, which launches one generated kernel per scheduler stage
 * (reference jobs/tvm_mnist/tvm_mnist.cpp:24-47; model list: jobs/tvm_<model>/, compile lines
 * sosp23_artifact/setup/onnx2tvm_all.sh:15-23).  Here a model is a static graph of the operators in
 * paella_ops.h with seeded fp32 weights; an executor issues it one stage at a time so the scheduler can
 * interleave stages of different requests.
 *
 * Model names: mnist, resnet18, resnet34, resnet50, mobilenetv2, inception_v3, squeezenet1_1, googlenet,
 * densenet121, ultraface320, arcfaceresnet100 -- or "onnx:<path>" for an ONNX file, which is imported on first use
 * (graph and trained weights; batch 1, fp32) where the reference compiles it with TVM
 * (reference sosp23_artifact/setup/onnx2tvm_all.sh:15-23).  Every entry point below takes either kind of name; for an
 * imported model the seed is ignored.  Operators read: Conv, BatchNormalization, Relu, Clip, PRelu, LeakyRelu, Add, Sub,
 * Mul, Div (with constants), MaxPool, AveragePool, GlobalAveragePool, GlobalMaxPool, Gemm, MatMul, Concat, Softmax, LRN,
 * Flatten, Reshape, Squeeze, Unsqueeze, Dropout, Identity, Constant, and Shape/Gather/Cast over static shapes; a file that
 * needs anything else makes the call fail (PAELLA_EINVAL) with the reason on stderr.
 *
 * Seeded weights: tensor number t of a model (creation order, listed by paella_model_describe) is filled
 * with value_i = float(normal_i * std_t), normal_i = sqrt(-2 ln u1) cos(2 pi u2),
 * u = ((splitmix64(seed*0x9E3779B97F4A7C15 + t*0xD1B54A32D192ED03 + 2i [+1]) >> 11) + 0.5) * 2^-53,
 * evaluated in double; "uniform" tensors take lo + (hi-lo)*u1; "constant" tensors a fixed value.
 *
 * Return value: 0 ok, negative PAELLA_E* for bad arguments, positive hipError_t for runtime failures.
 */
#ifndef PAELLA_MODELS_H
#define PAELLA_MODELS_H

#include <stddef.h>
#include <stdint.h>

#include "paella_ops.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct paella_model paella_model;   /* graph + packed weights resident on the device; shared, immutable */
typedef struct paella_exec paella_exec;     /* activations of one in-flight request */

/* ---- no GPU needed */
/* Comma-separated list of model names. */
const char* paella_model_names(void);
/* Bytes of the input / output tensor of a model. */
int paella_model_io_bytes(const char* name, size_t* in_bytes, size_t* out_bytes);
/* JSON description of the graph (buffers, weight tensors with stream/std/shape, nodes in stage order).
 * Writes at most cap bytes including the terminating NUL; *needed gets the full size. */
/* Writes the I/O-shape sidecar of a model: input dims, -1, output dims, one per line (the format of the
 * reference's sosp23_artifact/tvm_models_dim/<model>.dim). */
int paella_model_write_dim(const char* name, const char* path);
int paella_model_describe(const char* name, char* json, size_t cap, size_t* needed);
/* Algorithmic totals of one forward pass. */
int paella_model_totals(const char* name, double* macs, double* params, double* flops, double* bytes, int* stages);
/* The launches a model is executed as (see paella_model_num_stages below), computed on the host without a device:
 * for every launch its number of operators followed by their node indices.  Returns the number of ints the list
 * takes (written up to `capacity`), negative on error. */
int paella_model_launch_plan(const char* name, int* out, size_t capacity);
/* Fills out[i] with element i of weight tensor `tensor` of the model under `seed` (host memory). */
int paella_model_weight_values(const char* name, uint64_t seed, int tensor, float* out, size_t count);

/* ---- device */
/* Returns the process-wide instance for (name, seed), building and uploading it on first use. */
int paella_model_get(const char* name, uint64_t seed, paella_model** out);
/* A stage is one launch: one operator of the graph, up to four convs that do not depend on each other sharing a
 * grid (paella_conv2d_launch_group), or a per-channel scale-shift operator followed by the conv that applies it to
 * its own input (paella_conv2d_launch_transformed; when several convs read the scale-shift result, it is listed with
 * the first of them and the others apply it as well; its own output is never written).  Stages follow the graph's node order except where a conv is moved next to
 * partners, which never reorders two nodes of which one reads or overwrites what the other writes.  With
 * PAELLA_CONV_PAIRS=0 in the environment when the model is built, stage i is node i. */
int paella_model_num_stages(const paella_model* m);
/* Number of operators of stage i; their node indices, in launch order, go to nodes[0 .. min(count, capacity) - 1]. */
int paella_model_stage_nodes(const paella_model* m, int stage, int* nodes, int capacity);
/* Launch shape of stage i in the scheduler's units (vgprs read from the loaded code object). */
int paella_model_stage_dims(const paella_model* m, int stage, paella_launch_dims* dims);
/* Operator name ("conv", "dwconv", "dense", "pool", "gap", "eltwise", "softmax", "lrn") and algorithmic work of stage i
 * (of both convs for a pair). */
int paella_model_stage_work(const paella_model* m, int stage, const char** op, double* flops, double* bytes);

int paella_exec_create(const paella_model* m, paella_exec** out);
int paella_exec_destroy(paella_exec* e);
/* Device pointers of the request's input and output tensors. */
void* paella_exec_input(paella_exec* e);
void* paella_exec_output(paella_exec* e);
/* Makes the stages read the request's input from / write its output to memory of the caller instead of the request's own
 * device buffers -- pinned host memory the device can address, 16-byte aligned, at least the model's input / output
 * size: small tensors then cross PCIe inside the first / last kernel and need no copy stage of their own.  NULL restores
 * the device buffer.  PAELLA_ENOSUP if the graph cannot do without the buffer (a stage reads the output back, or writes
 * into the input buffer).  No counterpart in the reference, whose adapters always copy (jobs/tvm_mnist/tvm_mnist.cpp:38-46). */
int paella_exec_bind_input(paella_exec* e, void* device_visible);
int paella_exec_bind_output(paella_exec* e, void* device_visible);
/* Issues stage i on `stream`; notifier may be NULL. */
int paella_exec_launch_stage(paella_exec* e, int stage, void* stream, uint32_t job_id, void* notifier);
/* All stages back to back on one stream, un-instrumented (plain single-stream serving). */
int paella_exec_forward(paella_exec* e, void* stream);

#ifdef __cplusplus
}
#endif
#endif
