/*
 * mnv_hip.h - C ABI of the MI355X (gfx950) operator library that replaces the
 * cuBLAS / cuDNN / .cu launchers behind Minerva's GPU operator layer.
 *
 * Every entry point mirrors one launcher of the reference's
 * minerva/op/impl/cuda/cuda_perform.h (cited per function) with the CUDA handle
 * types replaced by an opaque stream pointer.  Conventions:
 *   - all tensors are fp32, column-major, dimension 0 fastest (reference
 *     minerva/common/scale.cpp:182-191): matrices are {rows, cols} with the row
 *     index fastest, image batches are {W,H,C,N} (= NCHW bytes), filters are
 *     {S,R,Cin,Cout} (= KCRS bytes);
 *   - all pointers are device pointers unless the name says host;
 *   - inputs and outputs never alias; the callee never allocates or frees
 *     tensors and keeps no state between calls; launches are asynchronous on
 *     `stream` (a hipStream_t cast to void*, NULL = the default stream) and the
 *     caller synchronises, as the reference device does after every operator
 *     (minerva/device/device.cpp:214-222);
 *   - return value: 0 on success, a hipError_t value (> 0) when the runtime
 *     reports an error, MNV_ERR_INVALID (-1) for arguments the kernels cannot
 *     take (null pointer, non-positive extent, extent beyond 2^31-1 where the
 *     reference's int arguments are mirrored), MNV_ERR_WORKSPACE (-2) when a
 *     caller-provided workspace is too small;
 *   - kernels that need device scratch take it as (workspace, workspace_bytes);
 *     the matching *_workspace_bytes function tells how much.  A NULL workspace
 *     is always accepted and selects a path that needs none.
 */
#ifndef MNV_HIP_H_
#define MNV_HIP_H_

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MNV_OK 0
#define MNV_ERR_INVALID (-1)
#define MNV_ERR_WORKSPACE (-2)
#define MNV_ERR_TOO_LARGE (-3)

typedef void* mnv_stream_t;

/* ---- device, streams, memory: replaces the CUDA runtime calls of
 *      minerva/device/device.cpp:146-222 and system/minerva_system.cpp:21-33 ---- */
int mnv_device_count(int* count);
int mnv_device_set(int device);
/* name_out: at least 256 bytes.  cu_count / clock_khz / hbm_bytes may be NULL. */
int mnv_device_info(int device, char* name_out, int* cu_count, int* clock_khz, size_t* hbm_bytes);
int mnv_stream_create(mnv_stream_t* stream);
int mnv_stream_destroy(mnv_stream_t stream);
int mnv_stream_sync(mnv_stream_t stream);
int mnv_device_sync(void);
int mnv_malloc(void** ptr, size_t bytes);
int mnv_free(void* ptr);
int mnv_host_malloc(void** ptr, size_t bytes); /* pinned host memory */
int mnv_host_free(void* ptr);
int mnv_memcpy_h2d(void* dst, const void* src_host, size_t bytes, mnv_stream_t stream);
int mnv_memcpy_d2h(void* dst_host, const void* src, size_t bytes, mnv_stream_t stream);
int mnv_memcpy_d2d(void* dst, const void* src, size_t bytes, mnv_stream_t stream);
/* Events for timing on the stream the kernels run on. */
int mnv_event_create(void** event);
/* An event that carries no time stamp, for ordering only, and the wait that makes every
 * later call on `stream` start after the work recorded before `event`: what replaces the
 * reference's cudaStreamSynchronize after every operator (minerva/device/device.cpp:221)
 * when operators on different streams depend on each other. */
int mnv_event_create_ordering(void** event);
int mnv_stream_wait_event(mnv_stream_t stream, void* event);
int mnv_event_destroy(void* event);
int mnv_event_record(void* event, mnv_stream_t stream);
int mnv_event_sync(void* event);
int mnv_event_elapsed_ms(void* start, void* stop, float* ms);
/* Stream capture into a HIP graph.  No counterpart in the reference, which launches and
 * synchronises every operator by itself (minerva/device/device.cpp:204-221); for callers
 * whose step is a fixed sequence of short kernels and therefore launch-bound.  Between
 * begin and end every call of this library on `stream` (not NULL) is recorded instead of
 * run; only kernel launches may be recorded, so the sequence must have run once before
 * (one-time set-up), must not allocate, synchronise or copy from host memory
 * (mnv_select, mnv_memcpy_h2d/d2h), and must use the same buffers on every replay.
 * end_capture returns the instantiated graph and optionally its node count;
 * abort_capture ends a capture whose recording failed and discards it. */
int mnv_graph_begin_capture(mnv_stream_t stream);
int mnv_graph_end_capture(mnv_stream_t stream, void** graph_exec, size_t* num_nodes);
int mnv_graph_abort_capture(mnv_stream_t stream);
int mnv_graph_launch(void* graph_exec, mnv_stream_t stream);
int mnv_graph_destroy(void* graph_exec);
const char* mnv_error_string(int status);

/* ---- elementwise binary: c[i] = a[i] (op) b[i]
 * CudaPerformAdd / CudaPerformSub / CudaPerformDotMult / CudaPerformDotDiv
 * (cuda_perform.h:12-16).  One IEEE operation per element. ---- */
int mnv_add(const float* a, const float* b, float* c, size_t n, mnv_stream_t stream);
int mnv_sub(const float* a, const float* b, float* c, size_t n, mnv_stream_t stream);
int mnv_mul(const float* a, const float* b, float* c, size_t n, mnv_stream_t stream);
int mnv_div(const float* a, const float* b, float* c, size_t n, mnv_stream_t stream);

/* ---- scalar arithmetic: CudaPerformConstAdd, CudaPerformLeftConstSub,
 * CudaPerformScale, CudaPerformLeftConstDiv (cuda_perform.h:18,21-23).
 *   const_add y = x + v   const_sub y = x - v   const_rsub y = v - x
 *   const_mul y = x * v   const_div y = x / v (a true division, as the CPU
 *   implementation basic.cpp:99-103 does)   const_rdiv y = v / x ---- */
int mnv_const_add(const float* x, float* y, float v, size_t n, mnv_stream_t stream);
int mnv_const_sub(const float* x, float* y, float v, size_t n, mnv_stream_t stream);
int mnv_const_rsub(const float* x, float* y, float v, size_t n, mnv_stream_t stream);
int mnv_const_mul(const float* x, float* y, float v, size_t n, mnv_stream_t stream);
int mnv_const_div(const float* x, float* y, float v, size_t n, mnv_stream_t stream);
int mnv_const_rdiv(const float* x, float* y, float v, size_t n, mnv_stream_t stream);

/* ---- elementwise unary: CudaPerformElewiseExp / Ln / Negative
 * (cuda_perform.h:43-45) ---- */
int mnv_exp(const float* x, float* y, size_t n, mnv_stream_t stream);
int mnv_ln(const float* x, float* y, size_t n, mnv_stream_t stream);
int mnv_neg(const float* x, float* y, size_t n, mnv_stream_t stream);
/* ThresholdNorm (CPU-only in the reference, basic.cpp:110-123):
 * y = |x| > threshold ? |x| / x * threshold : x, i.e. x clipped to [-threshold, threshold]. */
int mnv_threshold_norm(const float* x, float* y, float threshold, size_t n, mnv_stream_t stream);

/* ---- broadcast arithmetic on an {m,n} matrix: CudaPerformNorm{Add,Sub,Mult,Div}
 * On{Col,Row} (cuda_perform.h:25-33).
 *   *_col: vec has n entries (shape {1,n}); res[r + c*m] = matrix[r + c*m] (op) vec[c]
 *   *_row: vec has m entries (shape {m,1}); res[r + c*m] = matrix[r + c*m] (op) vec[r] ---- */
int mnv_norm_add_col(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);
int mnv_norm_sub_col(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);
int mnv_norm_mul_col(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);
int mnv_norm_div_col(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);
int mnv_norm_add_row(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);
int mnv_norm_sub_row(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);
int mnv_norm_mul_row(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);
int mnv_norm_div_row(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t stream);

/* ---- reductions of an {m,n} matrix: CudaPerformReduction{Sum,Max}On{Col,Row}
 * (cuda_perform.h:35-38).
 *   *_col: reduce dimension 0; out has n entries, out[c] = reduce_r in[r + c*m]
 *   *_row: reduce dimension 1; out has m entries, out[r] = reduce_c in[r + c*m] ---- */
int mnv_reduce_sum_col(const float* in, float* out, int m, int n, mnv_stream_t stream);
int mnv_reduce_max_col(const float* in, float* out, int m, int n, mnv_stream_t stream);
int mnv_reduce_sum_row(const float* in, float* out, int m, int n, mnv_stream_t stream);
int mnv_reduce_max_row(const float* in, float* out, int m, int n, mnv_stream_t stream);

/* ---- arg-max: CudaPerformMaxIndexOn{Col,Row} (cuda_perform.h:40-41).  The index
 * of the first maximum (lowest index wins ties, NaN never replaces the running
 * maximum), stored as float.  *_col: along dimension 0 (out has n entries);
 * *_row: along dimension 1 (out has m entries). ---- */
int mnv_maxindex_col(const float* in, float* out, int m, int n, mnv_stream_t stream);
int mnv_maxindex_row(const float* in, float* out, int m, int n, mnv_stream_t stream);

/* ---- SGEMM: CudaPerformMatMult (cuda_perform.h:17; cublasSgemm N,N, alpha 1,
 * beta 0, cuda_perform.cu:66-70).  C{m,n} = A{m,k} * B{k,n}, all column-major with
 * leading dimensions m, k, m.  The workspace (optional) lets skinny products split
 * the k range over more workgroups.  Each matrix may hold up to 2^31 - 1 elements (the
 * reference's int counts).  One launch reads A and B through 32-bit byte offsets, i.e. up
 * to 2^29 - 1 elements each; beyond that the product runs as several launches over column
 * panels and k ranges (later k ranges accumulate into C): slower, and summed range by
 * range.
 * mnv_sgemm_nn_plan reports how a product of these extents is launched with a workspace of
 * that size (no counterpart in the reference, where the plan is cuBLAS's own): tile_rows is
 * 128 or 64 (square tiles) or 256 (256 x 128), k_ranges the number of partial results reduced by a second
 * kernel (1: none), groups 4 when four wavefront groups of a workgroup share a tile and add
 * their quarters of the k range through LDS.  The plan depends on (m, n, k, workspace_bytes)
 * only, never on the operands. ---- */
size_t mnv_sgemm_nn_workspace_bytes(int m, int n, int k);
int mnv_sgemm_nn_plan(int m, int n, int k, size_t workspace_bytes, int* tile_rows, int* k_ranges,
                      int* groups);
int mnv_sgemm_nn(const float* a, const float* b, float* c, int m, int n, int k,
                 void* workspace, size_t workspace_bytes, mnv_stream_t stream);

/* The same product for callers that cannot allocate device memory or lend a workspace (code
 * under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  No counterpart
 * in the reference, whose launchers allocate at will (cuda_perform.cu:253,674).  The split-k
 * partial sums live in a device array of MNV_SGEMM_STATIC_SCRATCH_BYTES that is part of the
 * library image on every GPU; the call allocates and frees nothing and returns the bits
 * mnv_sgemm_nn returns with a workspace of that size.  Limit: m*n*2 floats must fit the
 * array (m*n <= 4 Mi elements), else MNV_ERR_TOO_LARGE -- larger outputs fill the chip
 * without splitting, call mnv_sgemm_nn with a NULL workspace for them.  All calls on one GPU
 * share the array: calls that overlap on one GPU (different streams or threads) race; calls
 * on one stream do not.  Nothing in the array needs clearing between calls (every partial
 * sum that is read was written by the same call).  The first call on a device looks the
 * array's address up (hipGetSymbolAddress): make it outside a graph capture. ---- */
#define MNV_SGEMM_STATIC_SCRATCH_BYTES (32u << 20)
int mnv_sgemm_nn_static(const float* a, const float* b, float* c, int m, int n, int k,
                        mnv_stream_t stream);

/* ---- transpose: CudaPerformTranspose (cuda_perform.h:19; cublasSgeam T,N).
 * a is {m,n}; c is {n,m}; c[j + i*n] = a[i + j*m]. ---- */
int mnv_transpose(const float* a, float* c, int m, int n, mnv_stream_t stream);

/* ---- copy / fill: CudaPerformReshape (cuda_perform.h:43, n counts floats here),
 * CudaPerformFill (cuda_perform.h:69) ---- */
int mnv_copy(const float* in, float* out, size_t n, mnv_stream_t stream);
int mnv_fill(float* dst, size_t n, float v, mnv_stream_t stream);

/* ---- activations: CudaPerform{Sigmoid,Relu,Tanh}{Forward,Backward}
 * (cuda_perform.h:55-60).  The reference describes the tensor as n*c*h*w
 * elements; the op is elementwise so only the count is passed.
 *   forward : top = f(bottom); relu is x > 0 ? x : 0
 *   backward: sigmoid bd = td*top*(1-top); relu bd = bottom > 0 ? td : 0;
 *             tanh bd = td*(1-top*top) ---- */
int mnv_sigmoid_fwd(const float* bottom, float* top, size_t n, mnv_stream_t stream);
int mnv_relu_fwd(const float* bottom, float* top, size_t n, mnv_stream_t stream);
int mnv_tanh_fwd(const float* bottom, float* top, size_t n, mnv_stream_t stream);
int mnv_sigmoid_bwd(const float* bottom, const float* top, const float* top_diff,
                    float* bottom_diff, size_t n, mnv_stream_t stream);
int mnv_relu_bwd(const float* bottom, const float* top, const float* top_diff,
                 float* bottom_diff, size_t n, mnv_stream_t stream);
int mnv_tanh_bwd(const float* bottom, const float* top, const float* top_diff,
                 float* bottom_diff, size_t n, mnv_stream_t stream);

/* ---- softmax: CudaPerform{Instance,Channel}Softmax{Forward,Backward}
 * (cuda_perform.h:51-54).  Tensor {W,H,C,N}.  instance: over the C*H*W values of
 * each image; channel: over C for each (n,h,w).  backward:
 * bottom_diff_i = top_i * (top_diff_i - sum_j top_diff_j * top_j). ---- */
int mnv_softmax_instance_fwd(const float* bottom, float* top, int num_images, int num_channels,
                             int height, int width, mnv_stream_t stream);
int mnv_softmax_channel_fwd(const float* bottom, float* top, int num_images, int num_channels,
                            int height, int width, mnv_stream_t stream);
int mnv_softmax_instance_bwd(const float* top_diff, const float* top, float* bottom_diff,
                             int num_images, int num_channels, int height, int width,
                             mnv_stream_t stream);
int mnv_softmax_channel_bwd(const float* top_diff, const float* top, float* bottom_diff,
                            int num_images, int num_channels, int height, int width,
                            mnv_stream_t stream);

/* ---- convolution: CudaPerformConv{Forward,BackwardData,BackwardFilter,BackwardBias}
 * (cuda_perform.h:47-50).  True convolution (flipped filter), zero padding:
 *   top[n,k,i,j] = bias[k] + sum_{c,r,s} bottom[n,c,i*sv-ph+r,j*sh-pw+s]
 *                                        * filter[k,c,R-1-r,S-1-s]
 *   top_height = (bottom_height + 2*pad_height - filter_height)/stride_vertical + 1.
 * backward_data takes the bottom extent (not the top extent the reference
 * launcher re-derives it from, cuda_perform.cu:277) so that inexact fits work,
 * and writes every element of bottom_diff.  backward_filter overwrites
 * filter_diff (beta = 0).  The workspace (optional everywhere) holds a re-ordered copy of
 * the filter for forward / backward_data (which then read the reduction dimension as
 * (tap, channel) and spend no address arithmetic per 16-channel slab) and the split
 * partial sums for backward_filter; without it a slower, equally exact path runs.
 * One launch reads bottom, top and filter through 32-bit byte offsets (fewer than 2^29
 * elements each).  A batch whose bottom or top is larger (up to 2^31 - 1 elements) runs as
 * several launches over chunks of images, the filter gradient accumulating chunk by chunk;
 * only a single image or a filter of 2^29 elements and more is refused (MNV_ERR_INVALID).
 * 3 x 3 and 5 x 5 filters at unit stride may run by minimal filtering (Winograd): F(2 x 2, 3 x 3),
 * 16 multiplies per 2 x 2 outputs of a channel pair instead of 36, F(4 x 4, 3 x 3), 36 per 4 x 4
 * outputs, or F(5 x 5, 3 x 3), 49 per 5 x 5 outputs -- whichever needs fewer products for the
 * plane at hand, a smaller tile on a near tie --, F(4 x 4, 5 x 5), 64 per 4 x 4 outputs instead
 * of 400: as 16 / 36 / 49 / 64 matrix products between transforms of 4 x 4 ... 8 x 8 tiles, summed
 * in fp32; backward_filter by F(3 x 3, m x m) / F(5 x 5, 4 x 4) with the sum over the tiles as the
 * products' reduction.  Results differ from the direct sum by a few 1e-6 of the output's
 * largest element (up to about 6e-6 with 6 x 6 tiles, up to about 2.5e-5 with 7 x 7 and 8 x 8
 * tiles; the bound of the convolutions is 1e-4).  forward / backward_data need a bottom / top
 * channel count that is a multiple of 16.  The path wants the workspace the size queries
 * report (16 ... 64 transformed values per tile and channel of both tensors), 16-byte aligned;
 * with less it runs in groups of images, with less than one image needs the direct kernels
 * run. ---- */
/* Selects when the three passes take the minimal-filtering path.  0: never; 1 (initial):
 * where a cost estimate from the extents (multiplies saved against transformed values moved;
 * in practice layers of about 200 channels and more whose direct pass takes over 100 us)
 * puts it at 80% of the direct kernels' time or less; 2: wherever it applies; 3 / 4 / 5: as 2
 * with the tile of 3 x 3 filters pinned to 2 x 2 / 4 x 4 / 5 x 5 outputs (3: 5 x 5 filters stay
 * direct; the most accurate setting that still uses the path).
 * Process-wide; returns the previous mode; any other value only queries.  No reference
 * counterpart: cuDNN picks its algorithm out of sight (CUDNN_CONVOLUTION_FWD_PREFER_FASTEST,
 * cuda_perform.cu:227-264). */
int mnv_conv_winograd_mode(int mode);
/* Measurement aid (no reference counterpart; a benchmark's way to time the MFMA kernel of a
 * minimal-filtering pass apart from the transform kernels around it).  While enabled, every
 * launch of the matrix products of such a pass is bracketed by an event pair on its stream
 * (about 4 us of idle GPU per launch); enabling drops earlier records.  _read waits for the
 * recorded launches of one kind (0: forward / backward_data products, 1: backward_filter
 * products with the reduction of their shares) and reports their number, their summed device
 * milliseconds and the flops of the products (2 x points x channels x channels x tiles).
 * Not for use while a stream is being captured into a graph. */
int mnv_conv_winograd_profile(int enable);
int mnv_conv_winograd_profile_read(int kind, int* launches, double* milliseconds, double* gflop);
size_t mnv_conv_fwd_workspace_bytes(int num_images, int bottom_num_channels,
                                   int top_num_channels, int bottom_height, int bottom_width,
                                   int pad_height, int pad_width, int stride_vertical,
                                   int stride_horizontal, int filter_height, int filter_width);
int mnv_conv_fwd(const float* bottom, const float* filter, const float* bias, float* top,
                 int num_images, int bottom_num_channels, int top_num_channels,
                 int bottom_height, int bottom_width, int pad_height, int pad_width,
                 int stride_vertical, int stride_horizontal, int filter_height,
                 int filter_width, void* workspace, size_t workspace_bytes,
                 mnv_stream_t stream);
size_t mnv_conv_bwd_data_workspace_bytes(int num_images, int bottom_num_channels,
                                        int top_num_channels, int bottom_height,
                                        int bottom_width, int pad_height, int pad_width,
                                        int stride_vertical, int stride_horizontal,
                                        int filter_height, int filter_width);
int mnv_conv_bwd_data(const float* top_diff, const float* filter, float* bottom_diff,
                      int num_images, int bottom_num_channels, int top_num_channels,
                      int bottom_height, int bottom_width, int pad_height, int pad_width,
                      int stride_vertical, int stride_horizontal, int filter_height,
                      int filter_width, void* workspace, size_t workspace_bytes,
                      mnv_stream_t stream);
size_t mnv_conv_bwd_filter_workspace_bytes(int num_images, int bottom_num_channels,
                                           int top_num_channels, int bottom_height,
                                           int bottom_width, int pad_height, int pad_width,
                                           int stride_vertical, int stride_horizontal,
                                           int filter_height, int filter_width);
int mnv_conv_bwd_filter(const float* bottom, const float* top_diff, float* filter_diff,
                        int num_images, int bottom_num_channels, int top_num_channels,
                        int bottom_height, int bottom_width, int pad_height, int pad_width,
                        int stride_vertical, int stride_horizontal, int filter_height,
                        int filter_width, void* workspace, size_t workspace_bytes,
                        mnv_stream_t stream);
/* How mnv_conv_bwd_filter launches a problem with a workspace of `workspace_bytes` on the
 * current device (no reference counterpart: cuDNN chooses its algorithm out of sight,
 * cuda_perform.cu:293-318): rows of the output tile (64 or 128); the k ranges the reduction
 * over images and positions is cut into, each with a partial result in the workspace (1: none);
 * and, when the launch instead has as many workgroups as the chip holds at once, each with the
 * same number of k-slabs ("stream-k": aligned k ranges of every tile, the rest in shares;
 * k_ranges is then 1), the number of workgroups, else 0.  For a batch that runs
 * as several launches, the plan of the first.  Launches nothing. */
int mnv_conv_bwd_filter_plan(int num_images, int bottom_num_channels, int top_num_channels,
                             int bottom_height, int bottom_width, int pad_height, int pad_width,
                             int stride_vertical, int stride_horizontal, int filter_height,
                             int filter_width, size_t workspace_bytes, int* tile_rows,
                             int* k_ranges, int* streamk_workgroups);
/* workspace (optional; 0 bytes = one workgroup per channel) lets each channel's sum be split
 * over image groups whose partial sums are added in a fixed order. */
size_t mnv_conv_bwd_bias_workspace_bytes(int num_images, int top_num_channels);
int mnv_conv_bwd_bias(const float* top_diff, float* bias_diff, int num_images,
                      int top_num_channels, int top_height, int top_width, void* workspace,
                      size_t workspace_bytes, mnv_stream_t stream);

/* ---- pooling: CudaPerform{Max,Average}Pooling{Forward,Backward}
 * (cuda_perform.h:61-64).  pooled = (in + 2*pad - window + stride - 1)/stride + 1,
 * minus one if (pooled-1)*stride >= in + pad (cuda_perform.cu:491-498);
 * mnv_pooled_size computes it.  Window o covers [o*stride - pad, o*stride - pad +
 * window) clipped to the tensor.  max: padding never wins; average: divisor is
 * window_height*window_width (padding counted).  max backward sends each
 * top_diff to the first maximum of its window in (row, column) scan order. ---- */
int mnv_pooled_size(int in, int window, int stride, int pad);
int mnv_maxpool_fwd(const float* bottom, float* top, int num_images, int num_channels,
                    int bottom_height, int bottom_width, int stride_vertical,
                    int stride_horizontal, int window_height, int window_width, int pad_height,
                    int pad_width, mnv_stream_t stream);
int mnv_avgpool_fwd(const float* bottom, float* top, int num_images, int num_channels,
                    int bottom_height, int bottom_width, int stride_vertical,
                    int stride_horizontal, int window_height, int window_width, int pad_height,
                    int pad_width, mnv_stream_t stream);
int mnv_maxpool_bwd(const float* bottom, const float* top, const float* top_diff,
                    float* bottom_diff, int num_images, int num_channels, int bottom_height,
                    int bottom_width, int stride_vertical, int stride_horizontal,
                    int window_height, int window_width, int pad_height, int pad_width,
                    mnv_stream_t stream);
int mnv_avgpool_bwd(const float* bottom, const float* top, const float* top_diff,
                    float* bottom_diff, int num_images, int num_channels, int bottom_height,
                    int bottom_width, int stride_vertical, int stride_horizontal,
                    int window_height, int window_width, int pad_height, int pad_width,
                    mnv_stream_t stream);

/* ---- local response normalisation across channels: CudaPerformLRN{Forward,Backward}
 * (cuda_perform.h:72-76; kernels cuda_kernel.h:223-331).  Tensor {W,H,C,N}.
 *   scale = 1 + alpha/local_size * (sum of bottom^2 over the channel window)
 *   top   = bottom * scale^(-beta)
 * forward writes both `scale` and `top` (the reference passes `scale` as an input
 * tensor and fills it, cuda.cpp:45-59); backward reads them:
 *   bottom_diff = top_diff * scale^(-beta)
 *                 - 2*alpha*beta/local_size * bottom * (sum of top_diff*top/scale over the window)
 * The window of channel c is [c - (local_size-1)/2, c + local_size/2] forward and its
 * mirror image backward, clipped to the channels. ---- */
int mnv_lrn_fwd(const float* bottom, float* scale, float* top, int local_size, float alpha,
                float beta, int num_images, int num_channels, int height, int width,
                mnv_stream_t stream);
int mnv_lrn_bwd(const float* bottom, const float* top, const float* scale, const float* top_diff,
                float* bottom_diff, int local_size, float alpha, float beta, int num_images,
                int num_channels, int height, int width, mnv_stream_t stream);

/* ---- Concat / Slice / Select data movement (reference cuda.cpp:80-155, 644-655).
 * The reference builds Concat and Slice from one CudaPerformCopy (cuda_perform.h:20) per
 * image; here one 2-D copy per input tensor does it: `rows` rows of `row_elems` floats,
 * row r read at src + r*src_pitch and written at dst + r*dst_pitch (pitches in floats,
 * >= row_elems).  Concatenating along dimension d: rows = product of the dimensions above
 * d, row_elems = (extent of this input along d) * (product of the dimensions below d),
 * dst_pitch = the same with the output's extent, dst advanced by the extents of the inputs
 * before it.  mnv_select replaces CudaPerformSelect (cuda_perform.h:76): dst{rows, n} takes
 * columns indices[0..n) of the column-major src{rows, cols}.  The indices are host memory
 * (the closure's vector); they are staged in `workspace` (mnv_select_workspace_bytes,
 * required) instead of the reference's per-call cudaMalloc (cuda_perform.cu:674). ---- */
int mnv_copy_2d(const float* src, float* dst, size_t row_elems, size_t rows, size_t src_pitch,
                size_t dst_pitch, mnv_stream_t stream);
size_t mnv_select_workspace_bytes(int num_indices);
int mnv_select(const float* src, float* dst, const int* indices_host, int num_indices, int rows,
               int cols, void* workspace, size_t workspace_bytes, mnv_stream_t stream);

/* ---- fused epilogues: an opt-in fast path, never taken by the operators above.
 * The reference launches a convolution and then a separate AddTensor for the bias
 * (cuda_perform.cu:227-264), and its applications follow every convolution and inner
 * product with a ReLU, every gradient with the ReLU gradient and finish with
 * w -= lr/batch * g as a scalar multiply and a subtraction
 * (owl/apps/imagenet_alexnet/alexnet.py:73-126, apps/mnist_common.h:185-197).  Each entry
 * point below performs one such pair in the producing kernel's store and returns, bit for
 * bit, what the two separate calls return (same IEEE operations in the same order):
 *   mnv_conv_fwd_relu        = mnv_conv_fwd, then mnv_relu_fwd
 *   mnv_conv_bwd_data_relu   = mnv_conv_bwd_data, then mnv_relu_bwd gated by `bottom`
 *                              (the activations the convolution's input went through ReLU as)
 *   mnv_maxpool_bwd_relu     = mnv_maxpool_bwd, then mnv_relu_bwd gated by `bottom`
 *   mnv_sgemm_nn_bias        = mnv_sgemm_nn, then mnv_norm_add_row with bias{m}, then
 *                              (relu != 0) mnv_relu_fwd
 *   mnv_sgemm_nn_relu_bwd    = mnv_sgemm_nn, then mnv_relu_bwd gated by bottom{m,n}
 *   mnv_sgd_update           = mnv_const_mul(g, scale), then mnv_sub(w, .): w_out = w - scale*g
 *   mnv_sgemm_tn             = mnv_transpose(at{k,m} -> a{m,k}), then mnv_sgemm_nn(a, b); with
 *                              `gate` != NULL followed by mnv_relu_bwd gated by gate{m,n}
 *                              (the inner-product data gradient W^T * sens of
 *                              apps/mnist_common.h:258-262, owl/apps/imagenet_alexnet/alexnet.py:96-99)
 *   mnv_sgemm_nt             = mnv_transpose(bt{n,k} -> b{k,n}), then mnv_sgemm_nn(a, b)
 *                              (the weight gradient sens * act^T of the same lines)
 *   mnv_sgemm_nt_sgd         = mnv_sgemm_nt into a gradient g{m,n}, then mnv_sgd_update(w, g):
 *                              w_out = w - scale * (a * bt^T); the gradient is never stored.
 *                              w_out may be w (each element is read, then written, once)
 *   mnv_conv_bwd_filter_sgd  = mnv_conv_bwd_filter into a gradient, then mnv_sgd_update:
 *                              filter_out = filter - scale * gradient; filter_out may be filter.
 *                              Refused (-1) for problems that mnv_conv_bwd_filter cuts into
 *                              several launches (operands of 2^29 elements and more)
 *                              (gradient and update of apps/mnist_common.h:185-197)
 * Workspaces are those of the unfused entry points (same *_workspace_bytes; for the
 * transposed products mnv_sgemm_nn_workspace_bytes(m, n, k)). ---- */
int mnv_conv_fwd_relu(const float* bottom, const float* filter, const float* bias, float* top,
                      int num_images, int bottom_num_channels, int top_num_channels,
                      int bottom_height, int bottom_width, int pad_height, int pad_width,
                      int stride_vertical, int stride_horizontal, int filter_height,
                      int filter_width, void* workspace, size_t workspace_bytes,
                      mnv_stream_t stream);
int mnv_conv_bwd_data_relu(const float* top_diff, const float* filter, const float* bottom,
                           float* bottom_diff, int num_images, int bottom_num_channels,
                           int top_num_channels, int bottom_height, int bottom_width,
                           int pad_height, int pad_width, int stride_vertical,
                           int stride_horizontal, int filter_height, int filter_width,
                           void* workspace, size_t workspace_bytes, mnv_stream_t stream);
int mnv_maxpool_bwd_relu(const float* bottom, const float* top, const float* top_diff,
                         float* bottom_diff, int num_images, int num_channels, int bottom_height,
                         int bottom_width, int stride_vertical, int stride_horizontal,
                         int window_height, int window_width, int pad_height, int pad_width,
                         mnv_stream_t stream);
int mnv_sgemm_nn_bias(const float* a, const float* b, const float* bias, float* c, int m, int n,
                      int k, int relu, void* workspace, size_t workspace_bytes,
                      mnv_stream_t stream);
int mnv_sgemm_nn_relu_bwd(const float* a, const float* b, const float* bottom, float* c, int m,
                          int n, int k, void* workspace, size_t workspace_bytes,
                          mnv_stream_t stream);
int mnv_sgd_update(const float* w, const float* g, float scale, float* w_out, size_t n,
                   mnv_stream_t stream);
int mnv_sgemm_tn(const float* at, const float* b, const float* gate, float* c, int m, int n, int k,
                 void* workspace, size_t workspace_bytes, mnv_stream_t stream);
int mnv_sgemm_nt(const float* a, const float* bt, float* c, int m, int n, int k, void* workspace,
                 size_t workspace_bytes, mnv_stream_t stream);
int mnv_sgemm_nt_sgd(const float* a, const float* bt, const float* w, float scale, float* w_out,
                     int m, int n, int k, void* workspace, size_t workspace_bytes,
                     mnv_stream_t stream);
int mnv_conv_bwd_filter_sgd(const float* bottom, const float* top_diff, const float* filter,
                            float scale, float* filter_out, int num_images,
                            int bottom_num_channels, int top_num_channels, int bottom_height,
                            int bottom_width, int pad_height, int pad_width, int stride_vertical,
                            int stride_horizontal, int filter_height, int filter_width,
                            void* workspace, size_t workspace_bytes, mnv_stream_t stream);

/* ---- random tensors: CudaPerformRandn / CudaPerformRandBernoulli (cuda_perform.h:66-67).
 * The reference seeds cuRAND from the wall clock per call (cuda.cpp:601,606); here the seed
 * is an argument and the generator is counter based (Philox4x32-10): element block i/4
 * uses counter (lo32, hi32, 0, 0) and key = seed, so equal seeds give equal tensors.
 * mnv_randn: mean + stddev * N(0,1) by Box-Muller (the reference passes its `var` closure
 * field as cuRAND's stddev argument).  mnv_rand_bernoulli: 1.0f with probability p, else 0. ---- */
int mnv_randn(float* dst, size_t n, unsigned long long seed, float mean, float stddev,
              mnv_stream_t stream);
int mnv_rand_bernoulli(float* dst, size_t n, unsigned long long seed, float p,
                       mnv_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* MNV_HIP_H_ */
