/*
 * mnv_host.h - C entry points of the C++ host layer (libmnv_host.so).
 *
 * The host layer is the C++ mirror of Minerva's operator and device interface
 * (namespace minerva: Scale, DataShard, closures, Context, hip::<Op> functions with
 * the parameter lists of minerva/op/impl/cuda.h:10-48, FnBundle dispatch, HipDevice
 * with a pooled allocator and four streams, and a sequential graph runner).  C++
 * callers include minerva_amd/host/*.h directly.  These few C functions exist so that
 * tests, the benchmark and foreign-language bindings can drive that C++ layer without
 * a C++ compiler: they create a runtime (device + runner), run one operator through
 * the full Task -> HipDevice -> FnBundle -> hip::<Op> -> C ABI path on host tensors,
 * and run the training graphs of the benchmark configurations.
 *
 * Every function returns 0 on success and -1 on failure; mnvh_last_error() then
 * describes the failed check (the reference aborts the process instead).
 */
#ifndef MNV_HOST_H_
#define MNV_HOST_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MNVH_MAX_DIMS 8

/* A host tensor: column-major data, extent dims[0..ndims-1], dimension 0 fastest. */
typedef struct {
  const float* data;
  int ndims;
  int dims[MNVH_MAX_DIMS];
} mnvh_tensor;

const char* mnvh_last_error(void);

/* sync_each_op: 1 = synchronise the stream after every operator, as the reference device
 * does (minerva/device/device.cpp:221); 0 = operators stay in flight on one stream in
 * program order and the caller synchronises with mnvh_runtime_sync; 2 = dataflow: operators
 * stay in flight on the device's four streams (a chain of dependent operators shares a
 * stream, independent chains get different ones), every output carries an event recorded
 * behind its producer and a consumer on another stream waits for it on the GPU -- what the
 * reference's scheduler achieves by waiting on the host after every operator.  Results are
 * bit-identical in all three modes. */
int mnvh_runtime_create(int gpu_id, int sync_each_op, void** runtime);
/* The same with the pooled allocator's threshold (default 200 GiB): when the bytes held
 * exceed it, every cached block is released (minerva/device/pooled_data_store.cpp:27-33);
 * in dataflow mode a stream recycles blocks that other streams still use (and waits for
 * them) once the pool holds half of it, instead of allocating. */
int mnvh_runtime_create_pool(int gpu_id, int sync_each_op, size_t pool_bytes, void** runtime);
int mnvh_runtime_destroy(void* runtime);
int mnvh_runtime_sync(void* runtime);
int mnvh_runtime_ops_issued(void* runtime, unsigned long long* count);
int mnvh_runtime_pool_stats(void* runtime, size_t* total_bytes, size_t* cached_blocks);
/* Dataflow mode, since the runtime was created: how often a consumer's stream was made to
 * wait for a producer on another stream, and how often a stream was made to wait for other
 * streams before it reused a recycled block. */
int mnvh_runtime_dataflow_stats(void* runtime, unsigned long long* producer_waits,
                                unsigned long long* recycle_waits);
/* Switches a live runtime between the one-stream order (enable = 0: mode 0 above) and dataflow
 * placement.  Drains the device first; every tensor stays valid, and tensors created before
 * the switch are tracked from their first use in the new mode. */
int mnvh_runtime_set_dataflow(void* runtime, int enable);
/* Dataflow mode: places the following operators on worker stream `stream` (0..3), -1 returns to
 * automatic placement (an operator follows its newest input that is still in flight).  What
 * owl.set_device is between devices in the reference, between the streams of one device. */
int mnvh_runtime_set_stream(void* runtime, int stream);

/* Per-operator device timing (two events per operator on its own stream).  The read
 * synchronises, writes one "name<TAB>launches<TAB>total_ms" line per operator name and
 * clears the record. */
int mnvh_runtime_profile(void* runtime, int enable);
/* Times only the operators whose name contains name_part (NULL or "": all).  The events
 * cost a few microseconds of idle GPU each; a step timed with all of them runs ~5% slower. */
int mnvh_runtime_profile_filter(void* runtime, const char* name_part);
int mnvh_runtime_profile_read(void* runtime, char* text_out, size_t capacity);

/*
 * Runs one operator on host tensors through the whole host stack.  `op` and
 * `params` (all passed as doubles):
 *   "arithmetic" [type]                 "arithmetic_const" [type, val, side]
 *   "elewise" [type]                    "norm_arithmetic" [type]        (vector = input 1)
 *   "matmult"  "trans"                  "reshape" [d0, d1, ...]
 *   "reduction" [type, dim]             "maxindex" [dim]
 *   "sigmoid_forward" "relu_forward" "tanh_forward"
 *   "sigmoid_backward" "relu_backward" "tanh_backward"      inputs: diff, top, bottom
 *   "activation_forward" [alg]          "activation_backward" [alg]
 *   "softmax_forward" [alg]             "softmax_backward" [alg]        inputs: diff, top
 *   "conv_forward" [ph, pw, sv, sh]             inputs: bottom, filter, bias
 *   "conv_backward_data" [ph, pw, sv, sh]       inputs: diff, bottom, filter
 *   "conv_backward_filter" [ph, pw, sv, sh]     inputs: diff, bottom, filter
 *   "conv_backward_bias"                        inputs: diff
 *   "pooling_forward" [alg, h, w, sv, sh, ph, pw]      inputs: bottom
 *   "pooling_backward" [alg, h, w, sv, sh, ph, pw]     inputs: diff, top, bottom
 *   "fill" [val, d0, d1, ...]
 * and the opt-in fused operators (minerva_amd/host/hip_fused_ops.h):
 *   "conv_forward_relu" [ph, pw, sv, sh]          inputs: bottom, filter, bias
 *   "conv_backward_data_relu" [ph, pw, sv, sh]    inputs: diff, bottom, filter
 *   "pooling_backward_relu" [h, w, sv, sh, ph, pw]      inputs: diff, top, bottom
 *   "matmult_bias" [relu]                         inputs: a, b, bias {m,1}
 *   "matmult_relu_backward"                       inputs: a, b, bottom
 *   "sgd_update" [scale]                          inputs: w, g
 * Enum values follow minerva/op/closure.h:8-24 and narray/convolution_info.h:19-57
 * (arithmetic 0 add 1 sub 2 mult 3 div; elewise 0 exp 1 ln 2 negative; reduction 0 sum
 * 1 max; softmax 0 instance 1 channel; activation 0 sigmoid 1 relu 2 tanh; pooling 0 max
 * 1 average).  The result is written to `out` (capacity out_capacity floats) and its
 * extent to out_ndims / out_dims.
 */
int mnvh_op(void* runtime, const char* op, const mnvh_tensor* inputs, int n_inputs,
            const double* params, int n_params, float* out, size_t out_capacity,
            int* out_ndims, int* out_dims);

/* Device-resident tensors, for graphs of operators that do not go through host memory
 * between operators.  `op` / `params` as for mnvh_op; a tensor is freed (its block goes back
 * to the device's pool) by mnvh_tensor_free even while operators that use it are queued.
 * mnvh_tensor_info reports the extent and the worker stream the producer was placed on. */
int mnvh_tensor_create(void* runtime, const mnvh_tensor* host, void** tensor);
int mnvh_tensor_op(void* runtime, const char* op, void* const* inputs, int n_inputs,
                   const double* params, int n_params, void** out);
int mnvh_tensor_info(void* tensor, int* ndims, int* dims /* MNVH_MAX_DIMS */, int* stream);
int mnvh_tensor_read(void* runtime, void* tensor, float* out, size_t out_capacity);
int mnvh_tensor_free(void* tensor);

/* Restarts the sequence the seeds of the "randn" / "rand_bernoulli" operators are drawn from. */
int mnvh_set_random_seed(unsigned long long seed);

/* Runs `count` independent element-wise additions through the device's thread pool
 * (four workers, four streams) and returns the results; exercises PushTask with
 * non-light tasks and the completion listener. */
int mnvh_concurrent_adds(void* runtime, const float* a, const float* b, size_t n, int count,
                         float* out /* count * n floats */);

/* Training graphs.  kind: "mlp" (784-256-10), "cnn" (MNIST CNN; variant 0 = conv2 pad 0
 * + 2x2/2 pooling, 1 = the reference app's pad 2 + 3x3/3), "alexnet". */
/* "alexnet": variant 0 = no dropout (the benchmark configuration), 1 = the reference
 * application's drop6 / drop7 with rate 0.5, masks from the restartable seed sequence */
int mnvh_net_create(void* runtime, const char* kind, int batch, int variant, void** net);
int mnvh_net_destroy(void* net);
int mnvh_net_num_params(void* net, int* count);
int mnvh_net_param_info(void* net, int index, char* name_out /* >= 16 bytes */, size_t* floats);
int mnvh_net_set_param(void* net, const char* name, const float* host, size_t floats);
/* name: a parameter ("w0"...), "prob", or "g_<param>" (gradient of the last step) */
int mnvh_net_read(void* net, const char* name, float* host_out, size_t floats);
/* Opt-in fast path: the following steps use the fused operators (convolution + ReLU, data /
 * pooling gradient + ReLU gradient, inner product + bias [+ ReLU], inner product + ReLU
 * gradient, one-kernel SGD update) instead of the separate ones.  No counterpart in the
 * reference; parameters, gradients and probabilities keep their bits. */
int mnvh_net_set_fused(void* net, int on);
/* For tests: the following steps of an "alexnet" network also keep their activations, read
 * with mnvh_net_read as "act1" ... "act10" (the outputs of conv1+relu, pool1, conv2+relu,
 * pool2, conv3..5+relu, pool5, fc6, fc7 after ReLU and dropout). */
int mnvh_net_keep_activations(void* net, int on);
/* Uploads one batch; it stays resident in HBM for the following steps. */
int mnvh_net_load_batch(void* net, const float* data, size_t data_floats, const float* label,
                        size_t label_floats);
/* Loads the NEXT batch while the step in flight keeps the GPU busy: the copy runs on a second
 * worker stream through pinned staging memory into a second pair of tensors (what the
 * reference's trainer gets from its data provider thread and the engine's ArrayLoader operator,
 * owl/owl/net/trainer.py:118-145, op/impl/cuda.cpp:592-598).  The next mnvh_net_step trains on
 * it.  Returns when the copy is complete; the caller's buffers may then be reused. */
int mnvh_net_prefetch_batch(void* net, const float* data, size_t data_floats, const float* label,
                            size_t label_floats);
/* One forward + backward + SGD step on the resident batch (on the prefetched one, if one was
 * loaded since the last step). */
int mnvh_net_step(void* net, float lr);
/* Records one step on the resident batch into a HIP graph (nothing of it is applied:
 * parameters are unchanged afterwards), for networks whose step is launch-bound.  The
 * reference has no counterpart: its device launches and synchronises operator by operator.
 * A replay runs the same kernels in the same order on the same buffers as mnvh_net_step
 * with the recorded lr and then copies the new parameters over the old ones, so results
 * are bit-identical to eager steps.  While the recording exists, mnvh_net_load_batch and
 * mnvh_net_set_param overwrite the resident buffers in place, mnvh_net_step is refused,
 * and "prob" / "g_<param>" hold the values of the latest replay.  A network with dropout
 * is refused (its masks come from seeds drawn on the host in every step). */
int mnvh_net_capture_step(void* net, float lr, size_t* num_nodes /* may be NULL */);
/* Replays the recording `steps` times; sync_each_step != 0 waits after every replay,
 * otherwise only after the last. */
int mnvh_net_replay(void* net, int steps, int sync_each_step);
int mnvh_net_release_graph(void* net);

#ifdef __cplusplus
}
#endif
#endif /* MNV_HOST_H_ */
