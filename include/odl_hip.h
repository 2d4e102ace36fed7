/*
 * odl_hip.h — C ABI of the gfx950 (MI355X) compute backend for OriginDL's hot path.
 *
 * This is the boundary a maintainer of the reference binds to: each entry point below stands where one
 * `origin::cuda::*` free function (include/origin/mat/origin/cuda/cuda_ops.cuh, cuda/factory.cuh) or one
 * device-runtime call of the reference's Storage/Allocator (src/mat/origin/memory) stands today. Plain
 * pointers and sizes only; no C++ types, no torch types.
 *
 * Conventions
 *  - All buffers are DEVICE pointers unless a parameter is named host_*. Tensors are dense, row-major,
 *    float32 unless the name says otherwise; dimensions are int64_t; labels are int32 or int64
 *    (idx_is_i64 selects), max-pool indices are uint64 (the reference's std::vector<size_t>).
 *  - `stream` is a hipStream_t passed as void*; NULL is the null stream, which is what the reference uses
 *    for everything (its host is single-threaded and uses one ordered queue). Launches are asynchronous.
 *  - Every function returns ODL_OK or a negative code and records a message readable through
 *    odl_hip_last_error() (thread-local). ODL_ERR_INVALID_ARG corresponds to the reference's
 *    std::invalid_argument (THROW_INVALID_ARG), ODL_ERR_RUNTIME to std::runtime_error (THROW_RUNTIME_ERROR,
 *    CUDA_CHECK), include/origin/utils/exception.h:37-57.
 *  - Functions that need scratch take (workspace, workspace_bytes); the matching *_workspace_bytes query
 *    says how much. The library never keeps a buffer it hands out or receives.
 *  - There is no CPU fallback: without a visible gfx950 device every compute entry point fails with
 *    ODL_ERR_RUNTIME.
 */
#ifndef ODL_HIP_H
#define ODL_HIP_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ODL_OK 0
#define ODL_ERR_INVALID_ARG (-1)
#define ODL_ERR_RUNTIME (-2)

/* ------------------------------------------------------------------ device runtime ----------------- */
/* include/origin/cuda/cuda.h:25-105 — is_available / device_count / current_device / set_device /
 * device_info / synchronize; src/mat/origin/cuda/cuda_utils.cu:37-91 */
int odl_hip_device_count(int *count);
int odl_hip_set_device(int device);
int odl_hip_get_device(int *device);
int odl_hip_synchronize(void);
/* writes "name | gcnArch | CUs | clock MHz | global MiB" into buf (NUL-terminated, truncated to len) */
int odl_hip_device_info(int device, char *buf, size_t len);
const char *odl_hip_last_error(void);
/* src/mat/origin/memory/allocator.cpp:53-107 (cudaSetDevice + cudaMalloc / cudaFree / cudaMemGetInfo) */
int odl_hip_malloc(void **ptr, size_t bytes);
int odl_hip_free(void *ptr);
int odl_hip_mem_info(size_t *free_bytes, size_t *total_bytes);
/* src/mat/origin/memory/storage.cpp:69-145 — synchronous copies, device-synchronised before D2H.
 * h2d: the reference copies on the null stream, where all its kernels run too, so a copy into recycled memory waits for
 * the kernels that last used it. Created streams here are non-blocking — they and the null stream do not wait for each
 * other — so a caller that launches on a created stream passes that stream: the copy is queued behind everything
 * already on it and the call returns when the data has landed. stream = NULL is the reference's plain blocking copy,
 * ordered only against null-stream work. */
int odl_hip_memcpy_h2d(void *dst, const void *host_src, size_t bytes, void *stream);
int odl_hip_memcpy_d2h(void *host_dst, const void *src, size_t bytes);
int odl_hip_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
int odl_hip_memset(void *dst, int value, size_t bytes, void *stream);

/* Streams and captured graphs. No counterpart in the reference, which launches everything on the null stream
 * (the files under src/mat/origin/cuda create no stream, event or graph): they exist so that a caller can record a step of
 * fixed shapes once and replay it with one submission. A created stream is non-blocking and has the default
 * priority. Between capture_begin and capture_end every launch on that stream is recorded, not run; entry points
 * that synchronise or copy to the host (odl_hip_synchronize, odl_hip_memcpy_d2h, odl_hip_softmax_ce_loss,
 * odl_hip_gather, odl_hip_accuracy) must not be called in between. All entry points clear memory with fill kernels,
 * never with memset nodes. capture_end returns an executable graph; launch replays it on a stream. */
int odl_hip_stream_create(void **stream);
int odl_hip_stream_destroy(void *stream);
int odl_hip_stream_synchronize(void *stream);
int odl_hip_device_synchronize(void); /* every stream of the current device */
/* pinned host memory that kernels can write (hipHostMalloc): for the few words a caller polls after a synchronise */
int odl_hip_host_alloc(void **ptr, size_t bytes);
int odl_hip_host_free(void *ptr);
/* events: a point in a stream's queue the host can wait for without waiting for what was queued after it (the loss of a
 * step is read while the step's backward pass is still running). Created without timing; not to be recorded into a
 * capture. */
int odl_hip_event_create(void **event);
int odl_hip_event_destroy(void *event);
int odl_hip_event_record(void *event, void *stream);
int odl_hip_event_synchronize(void *event);
int odl_hip_graph_capture_begin(void *stream);
int odl_hip_graph_capture_end(void *stream, void **graph_exec);
/* how many nodes (launches) the graph that this thread ended last holds */
int odl_hip_graph_last_node_count(int64_t *nodes);
/* gives up a capture (after an error in the middle of the step being recorded): the stream leaves capture mode,
 * whatever was recorded is discarded, the stream can be used and captured again. A no-op on a stream that is not
 * capturing. */
int odl_hip_graph_capture_abort(void *stream);
int odl_hip_graph_launch(void *graph_exec, void *stream);
int odl_hip_graph_destroy(void *graph_exec);

/* ------------------------------------------------------------------ GEMM ---------------------------- */
/* General row-major SGEMM on FP32 MFMA: C[M,N] = op(A)[M,K] . op(B)[K,N] (+ bias[N] broadcast over rows
 * when bias != NULL). trans_a: A is stored [K,M] (lda >= M) else [M,K] (lda >= K); trans_b: B is stored
 * [N,K] (ldb >= K) else [K,N] (ldb >= N). Replaces origin::cuda::matmul (cuda_ops.cuh matmul;
 * src/mat/origin/cuda/math/mat_mul.cu:1833-1970) and makes the reference's materialised transposes
 * (src/operators/math/mat_mul.cpp:171-174) unnecessary.
 * split_k: 0 = choose automatically, 1 = none, >1 = that many K slices reduced in a fixed order
 * (needs workspace of odl_hip_sgemm_workspace_bytes). */
int odl_hip_sgemm(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const float *A, int64_t lda,
                  const float *B, int64_t ldb, float *C, int64_t ldc, const float *bias, int split_k,
                  void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_sgemm_workspace_bytes(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, int split_k);
/* Linear::forward (src/nn/layers/linear.cpp:80-106) with the activation that follows it applied in the product's epilogue:
 * y[M,N] = act(x[M,K] . w[K,N] + b[N]), activation -1 none, 0 relu, 7 silu (the odl_hip_unary operator numbers).
 * Bit-identical to odl_hip_sgemm with a bias followed by odl_hip_unary; the reference runs Linear and ReLU as separate
 * modules (tests/example/mnist/mlp_mnist.cpp). Workspace: odl_hip_sgemm_workspace_bytes(0, 0, M, N, K, 0). */
int odl_hip_linear_act(const float *x, const float *w, const float *b, int64_t M, int64_t N, int64_t K, int activation,
                       float *y, void *workspace, size_t workspace_bytes, void *stream);

/* Mat::matmul — 2-D x 2-D (batch = 1), 3-D x 2-D (b_is_batched = 0), 3-D x 3-D (b_is_batched = 1);
 * src/mat/origin/cpu/math/matmul.cpp:113-218. The workspace (may be NULL) lets small products be split along K
 * so that they still fill the chip. */
int odl_hip_matmul(const float *a, const float *b, float *c, int64_t batch, int64_t M, int64_t N, int64_t K,
                   int b_is_batched, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_matmul_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int b_is_batched);
/* MatMul::backward (src/operators/math/mat_mul.cpp:123-182): gx[M,K] = gy[M,N] . w[K,N]^T and
 * gw[K,N] = x[M,K]^T . gy[M,N], as NT and TN GEMMs with no transpose copy. Either output may be NULL. */
int odl_hip_matmul_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, int64_t M,
                            int64_t K, int64_t N, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_matmul_backward_workspace_bytes(int64_t M, int64_t K, int64_t N);
/* Backward of Linear::forward's matmul + broadcast_to + add for 2-D inputs (src/nn/layers/linear.cpp:88-104): the two
 * gradients of odl_hip_matmul_backward and gb[N] = gy[M,N] summed over its rows — what Mat::sum_to to the bias's shape
 * gives (src/mat/origin/cpu/math/sum_to.cpp), bit for bit the result of odl_hip_sum_axis(gy, 1, M, N). For a classifier
 * layer (N <= 16, long K) the three are one launch. Any output may be NULL. */
int odl_hip_linear_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, float *gb, int64_t M,
                            int64_t K, int64_t N, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_linear_backward_workspace_bytes(int64_t M, int64_t K, int64_t N);
/* Mat::matmul and MatMul::backward for float64 tensors (the reference's device matmul is a template over the element
 * type and serves double through the kernels it uses for float, src/mat/origin/cuda/math/mat_mul.cu:1911-1954; CPU form
 * src/mat/origin/cpu/math/matmul.cpp:27-41): C[M,N] = op(A)[M,K] . op(B)[K,N] on the FP64 matrix cores, layouts as in
 * odl_hip_sgemm (trans_a: A stored [K,M]; trans_b: B stored [N,K]), `batch` independent products stride_a / stride_b /
 * stride_c doubles apart (stride_b = 0: one B for all, the 3-D x 2-D case). No workspace. */
int odl_hip_dgemm(int trans_a, int trans_b, int64_t M, int64_t N, int64_t K, const double *A, int64_t lda, const double *B,
                  int64_t ldb, double *C, int64_t ldc, int64_t batch, int64_t stride_a, int64_t stride_b, int64_t stride_c,
                  void *stream);
/* Mat::transpose (src/mat/origin/cpu/shape/transpose.cpp:27-77): last two dims of [outer, rows, cols] */
int odl_hip_transpose(const float *src, float *dst, int64_t outer, int64_t rows, int64_t cols, void *stream);

/* ------------------------------------------------------------------ convolution --------------------- */
/* Mat::im2col / Mat::col2im (include/origin/mat/mat.h:462-483; src/mat/origin/cpu/conv/conv2d.cpp:39-377).
 * to_matrix != 0: col is [N*OH*OW, C*KH*KW]; else [N,C,KH,KW,OH,OW]. Zero padding. col2im accumulates each
 * image pixel's taps in ascending (kh, kw) order, as the reference's scatter loop does, so results are
 * bit-identical to it and independent of scheduling (no atomics). */
int odl_hip_im2col(const float *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
                   int PH, int PW, int to_matrix, float *col, void *stream);
int odl_hip_col2im(const float *col, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
                   int PH, int PW, int to_matrix, float *img, void *stream);
/* Mat::conv2d (mat.h:490; conv2d.cpp:404-512): y[N,OC,OH,OW] = NCHW(im2col(x) . W2d^T + b). b may be NULL. */
int odl_hip_conv2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                   int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *y, void *workspace,
                   size_t workspace_bytes, void *stream);
/* The same convolution with an activation applied to each output after the bias, in the kernel's epilogue:
 * activation -1 none, 0 relu, 7 silu (the odl_hip_unary operator numbers). Bit-identical to odl_hip_conv2d followed by
 * odl_hip_unary; the reference has no fused counterpart (its graphs hold nn.Conv2d and nn.SiLU as separate nodes,
 * src/pnnx/operator_mapper.cpp:30-37). Same workspace as odl_hip_conv2d. */
int odl_hip_conv2d_act(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                       int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int activation, float *y,
                       void *workspace, size_t workspace_bytes, void *stream);
/* The same forward for weights that do not change between calls (inference): some shapes read the filter in another
 * order ([OC][tap][C], or blocks of 32 output channels x 8 channels per tap for the small-problem kernel), and
 * odl_hip_conv2d / _act write that copy into the workspace on every call. A caller that keeps its weights can make
 * the copy once — packed_weights_bytes says how large it is for a shape (0: this shape reads the filter as it lies and
 * `packed` is ignored), pack_weights fills it in the order that shape's kernel reads — and pass it to
 * conv2d_act_packed, which then skips the copy. packed = NULL is odl_hip_conv2d_act. No counterpart in the reference (its runner re-uploads the
 * weights on every forward, src/pnnx/pnnx_graph.cpp:341-405). */
size_t odl_hip_conv2d_packed_weights_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                           int SW, int PH, int PW);
int odl_hip_conv2d_pack_weights(const float *w, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                int SW, int PH, int PW, float *packed, void *stream);
int odl_hip_conv2d_act_packed(const float *x, const float *w, const float *packed, const float *b, int64_t N, int64_t C,
                              int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW,
                              int activation, float *y, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_conv2d_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                                      int SH, int SW, int PH, int PW);
/* Mat::conv2d_backward (mat.h:505; conv2d.cpp:514-599) -> gx, gW and (when gb != NULL) gb.
 * Reference-faithful: gy's NCHW buffer is read as a row-major [N*OH*OW, OC] matrix with no permutation
 * (conv2d.cpp:548) for gW and gx; gb is the true per-channel sum of gy (571-578). */
int odl_hip_conv2d_backward(const float *gy, const float *x, const float *w, int64_t N, int64_t C, int64_t H,
                            int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *gx,
                            float *gw, float *gb, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_conv2d_backward_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH,
                                               int KW, int SH, int SW, int PH, int PW);
/* The same five operators on float64 tensors. The reference's device convolution dispatches over the element type
 * (src/mat/origin/cuda/conv/conv2d.cu:412-664: im2col, col2im, conv2d, conv2d_backward) and runs the CPU algorithm
 * (src/mat/origin/cpu/conv/conv2d.cpp:39-599) in that type; here the products run on the FP64 matrix cores
 * (odl_hip_dgemm) with plain gather / scatter kernels around them. Same layouts, same reading of gy as a row-major
 * [N*OH*OW, OC] matrix in the backward pass, same order of the taps in col2im. gx, gw, gb may each be NULL. */
int odl_hip_im2col_f64(const double *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                       int PW, int to_matrix, double *col, void *stream);
int odl_hip_col2im_f64(const double *col, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                       int PW, int to_matrix, double *img, void *stream);
int odl_hip_conv2d_f64(const double *x, const double *w, const double *b, int64_t N, int64_t C, int64_t H, int64_t W,
                       int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, double *y, void *workspace,
                       size_t workspace_bytes, void *stream);
size_t odl_hip_conv2d_f64_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH,
                                          int SW, int PH, int PW);
int odl_hip_conv2d_backward_f64(const double *gy, const double *x, const double *w, int64_t N, int64_t C, int64_t H, int64_t W,
                                int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, double *gx, double *gw, double *gb,
                                void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_conv2d_backward_f64_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW,
                                                   int SH, int SW, int PH, int PW);

/* Kernel selection of the 3x3 / stride 1 / padding 1 convolutions. The kernel that keeps the input patch in LDS is
 * chosen for the forward and the input gradient only when it would launch at least `min_workgroups` workgroups (default:
 * one per compute unit of the device; smaller layers go to the K-sliced implicit kernels, which fill the chip better).
 * This call replaces that threshold for the whole process; a negative value restores the default. It exists so that
 * tests can send small shapes through the LDS-patch kernel. The choice enters the workspace sizes: never change it
 * between a *_workspace_bytes query and the call the query was made for. No counterpart in the reference. */
int odl_hip_set_conv_patch_min_workgroups(int64_t min_workgroups);
/* A convolution node of the reference's graph runner together with the nodes that follow it
 * (src/pnnx/pnnx_graph.cpp:286-528 runs nn.Conv2d, nn.SiLU, pnnx.Expression add and torch.cat one by one;
 * src/mat/origin/cpu/shape/cat.cpp:81-123 then copies every input of the concatenation):
 *   y[n, oc] = residual[n, oc] + act(conv(x)[n, oc] + b[oc])
 * where x, residual and y are NCHW tensors whose images lie x_image_stride / residual_image_stride / y_image_stride
 * floats apart (0: dense), so that each may be a run of channels inside a wider tensor: a convolution writes straight
 * into its part of a concatenation's destination and reads an input that lives in one. residual may be NULL.
 * packed: the filter as odl_hip_conv2d_pack_weights lays it out for this shape (required). Covers small problems only (channels a
 * multiple of 8, square stride and padding, up to about 1.6 GFLOP): odl_hip_conv2d_fused_ok answers 1 for a shape
 * this entry point takes, and a shape it does not take is refused with ODL_ERR_INVALID_ARG — the caller then runs
 * the nodes one by one. The sums are formed in another order than odl_hip_conv2d's large-problem kernels form them
 * (float32 rounding differs in the last bits); odl_hip_conv2d itself sends the shapes covered here through the
 * same kernel. */
int odl_hip_conv2d_fused_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH,
                            int PW);
int odl_hip_conv2d_fused(const float *x, int64_t x_image_stride, const float *packed, const float *b, int64_t N, int64_t C,
                         int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int activation,
                         const float *residual, int64_t residual_image_stride, float *y, int64_t y_image_stride,
                         void *stream);
/* Two convolutions over the same input with the same window, stride, padding and activation (the cv1 / cv2 pair of a
 * detector's C3 block: two nn.Conv2d nodes reading one tensor) run as one: `packed` and b hold the two filters and
 * biases one after the other ([OC, C, KH, KW] packed by odl_hip_conv2d_pack_weights for OC filters, b[OC]); the outputs
 * of filters [0, split) go to y_first [N, split, OH, OW], those of filters [split, OC) to y_second [N, OC - split, OH, OW],
 * each with its own image stride. K is shared between waves as for the member with more filters alone, so two members
 * of equal size (the C3 case) give the floats of two odl_hip_conv2d_fused calls, bit for bit. Covered shapes:
 * odl_hip_conv2d_fused_ok(..., OC, ...). */
int odl_hip_conv2d_fused_pair(const float *x, int64_t x_image_stride, const float *packed, const float *b, int64_t N, int64_t C,
                              int64_t H, int64_t W, int64_t OC, int64_t split, int KH, int KW, int SH, int SW, int PH, int PW,
                              int activation, float *y_first, int64_t y_first_image_stride, float *y_second,
                              int64_t y_second_image_stride, void *stream);
/* One to four convolutions with 1x1 windows (stride 1, no padding, no residual) over the same batch — the stage
 * convolutions of a detect head, nn.Conv2d nodes that do not depend on each other — as one launch. Arrays are host
 * arrays with one entry per member; host_b may be NULL (no member has a bias) or hold NULL entries. Each member gets
 * the floats of its own odl_hip_conv2d_fused call, bit for bit. odl_hip_conv2d_fused_group_ok answers 1 for member shapes
 * this entry point takes. No counterpart in the reference, whose runner executes the nodes one by one
 * (src/pnnx/pnnx_graph.cpp:286-528). */
int odl_hip_conv2d_fused_group_ok(int count, int64_t N, const int64_t *host_C, const int64_t *host_H, const int64_t *host_W,
                                  const int64_t *host_OC);
int odl_hip_conv2d_fused_group(int count, const float *const *host_x, const int64_t *host_x_image_stride, const float *const *host_packed,
                               const float *const *host_b, int64_t N, const int64_t *host_C, const int64_t *host_H,
                               const int64_t *host_W, const int64_t *host_OC, int activation, float *const *host_y,
                               const int64_t *host_y_image_stride, void *stream);
/* Measurement switches, for the whole process (same caveat as above: never between a query and its call):
 * set_conv_direct(0) sends the small problems to the tiled kernels again; set_conv_direct_plan(k_shares, pixel_tiles)
 * fixes how a workgroup of the small-problem kernel is cut (0, 0: its own rule). No counterpart in the reference. */
int odl_hip_set_conv_direct(int enabled);
int odl_hip_set_conv_direct_plan(int k_shares, int pixel_tiles);

/* ------------------------------------------------------------------ reductions / broadcast ---------- */
/* Mat::sum(axis) seen as [outer, axis, inner] -> [outer, inner]
 * (src/mat/origin/cpu/math/sum.cpp:15-90; operation_templates.h:270-333). */
int odl_hip_sum_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst, void *workspace,
                     size_t workspace_bytes, void *stream);
size_t odl_hip_sum_axis_workspace_bytes(int64_t outer, int64_t axis, int64_t inner);
/* odl_hip_sum_axis for callers that cannot allocate device memory and so cannot bring a workspace: code running under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. The
 * partial sums go to an array that is part of the library's device image (8 MiB, held by every GPU the library runs on
 * until the process ends; odl_hip_sum_axis_noalloc_max_bytes returns the size) instead of a workspace; kernels, plan
 * and order of additions are those of odl_hip_sum_axis, so results are bit-identical to it. The call allocates nothing
 * and frees nothing. A reduction whose partial sums (odl_hip_sum_axis_workspace_bytes) do not fit the array is refused
 * with ODL_ERR_INVALID_ARG; the [16384, 4096] -> [4096] bias gradient fits exactly. All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (two streams, two threads) race, so order them. The first call on
 * each device resolves the array's address and must come outside stream capture (ODL_ERR_RUNTIME otherwise). */
int odl_hip_sum_axis_noalloc(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst, void *stream);
size_t odl_hip_sum_axis_noalloc_max_bytes(void);
/* Mat::sum(-1): all elements -> dst[0] (operation_templates.h:342-357) */
int odl_hip_sum_all(const float *src, int64_t n, float *dst, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_sum_all_workspace_bytes(int64_t n);
/* Mat::max(axis) / Mat::max(-1) (src/mat/origin/cpu/math/max.cpp:20-121): NaNs never win (`max_val < v` is false for
 * them), except that the whole-tensor maximum starts from the first element and stays NaN when that is one. A long axis
 * over few columns, and a whole tensor of 65536 elements or more, are scanned by many workgroups whose partial maxima
 * meet through integer atomics: the value is the reference's, but where the maximum is a zero and zeros of both signs
 * occur the result is +0.0f whatever their order (the reference keeps the first one it meets). */
int odl_hip_max_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst, void *stream);
int odl_hip_max_all(const float *src, int64_t n, float *dst, void *stream);
/* Mat::sum_to (mat.h:217; src/mat/origin/cpu/math/sum_to.cpp:11-76): LEFT-aligned shape comparison, one
 * fused pass per contiguous run of reduced dims. Equal shapes copy. A target with more elements ->
 * ODL_ERR_RUNTIME; a reduced shape that cannot be reshaped to the target -> ODL_ERR_INVALID_ARG. */
int odl_hip_sum_to(const float *src, const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                   int dst_ndim, float *dst, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_sum_to_workspace_bytes(const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                                      int dst_ndim);
/* conv bias gradient gy[N,OC,P] -> gb[OC] (conv2d.cpp:566-580) in one pass over gy */
int odl_hip_sum_nchw_channels(const float *gy, int64_t N, int64_t OC, int64_t P, float *gb, void *workspace,
                              size_t workspace_bytes, void *stream);
size_t odl_hip_sum_nchw_channels_workspace_bytes(int64_t N, int64_t OC, int64_t P);
/* Mat::broadcast_to (mat.h:210; operation_templates.h:433-493): RIGHT-aligned, up to 8 dims */
int odl_hip_broadcast_to(const float *src, const int64_t *host_src_shape, int src_ndim,
                         const int64_t *host_dst_shape, int dst_ndim, float *dst, void *stream);

/* ------------------------------------------------------------------ softmax / cross entropy --------- */
/* Softmax::forward over [outer, axis, inner] (src/operators/activation/softmax.cpp:14-76) in one kernel */
int odl_hip_softmax(const float *x, int64_t outer, int64_t axis, int64_t inner, float *y, void *stream);
/* Mat::gather / Mat::one_hot (mat.h:697,705; src/mat/origin/cpu/nn/gather.cpp). gather validates the labels
 * (a device flag read back, one 4-byte D2H, like the reference CUDA backend's label check
 * src/mat/origin/cuda/nn/gather.cu:146-175) and returns ODL_ERR_INVALID_ARG for an out-of-range label;
 * one_hot skips out-of-range labels silently. */
int odl_hip_gather(const float *in, const void *idx, int idx_is_i64, int64_t N, int64_t C, float *out, void *stream);
int odl_hip_one_hot(const void *idx, int idx_is_i64, int64_t N, int64_t C, float *out, void *stream);
/* SoftmaxCrossEntropy::forward (src/operators/loss/softmax_cross_entropy.cpp:17-75), fused:
 * *host_loss = -(1/N) sum_i log(softmax(x)[i, t_i] + 1e-8). Synchronises (the reference's .item<float>()).
 * workspace: N floats + 16 bytes. Out-of-range label -> ODL_ERR_INVALID_ARG. */
int odl_hip_softmax_ce_loss(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, float *host_loss,
                            void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_softmax_ce_loss_workspace_bytes(int64_t N);
/* SoftmaxCrossEntropy::backward (softmax_cross_entropy.cpp:77-111), one pass:
 * gx = (softmax(x) - one_hot(t)) * (gy / N); gy is the host scalar the reference reads with .item<float>() */
int odl_hip_softmax_ce_grad(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, float gy, float *gx,
                            void *stream);
/* The same two without a host round trip, for callers that record the step into a graph: the loss goes to
 * device_loss2[0] (float) and the out-of-range-label flag to device_loss2[1] (int, nonzero = a bad label; the caller
 * decides when to look at it), and the upstream gradient is read from device memory (device_gy[0]). Same kernels,
 * same arithmetic: gy / N is formed in the kernel as the host forms it. host_mirror2 (may be NULL): 8 bytes of pinned
 * host memory from odl_hip_host_alloc that the loss kernel fills with the same two words, so that a caller who has
 * synchronised the stream reads them without queueing a copy. */
int odl_hip_softmax_ce_loss_device(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C,
                                   float *device_loss2, void *host_mirror2, void *workspace, size_t workspace_bytes,
                                   void *stream);
int odl_hip_softmax_ce_grad_device(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C,
                                   const float *device_gy, float *gx, void *stream);
/* odl_hip_softmax_ce_loss_device that also writes unit_gx[N, C], the gradient for an upstream gradient of 1 — the seed
 * Tensor::backward() starts from (src/core/tensor_impl.cpp:94-98) — in the same launch: bit for bit what
 * odl_hip_softmax_ce_grad(x, t, ..., 1.0f) writes (for logits without NaN), so a caller whose upstream gradient is that
 * constant needs no second launch. For the batches odl_hip_softmax_ce_loss_grad_ok names (1 / 0): up to 2048 rows of up to
 * 64 classes. */
int odl_hip_softmax_ce_loss_grad_ok(int64_t N, int64_t C);
int odl_hip_softmax_ce_loss_grad_device(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C,
                                        float *device_loss2, void *host_mirror2, float *unit_gx, void *workspace,
                                        size_t workspace_bytes, void *stream);

/* ------------------------------------------------------------------ pooling ------------------------- */
/* Mat::max_pool2d / max_pool2d_backward (mat.h:560-578; src/mat/origin/cpu/pooling/max_pool2d.cpp:40-224).
 * idx[n,c,oh,ow] = kh*KW+kw of the first maximum (strict >, scan starts at window cell (0,0));
 * padding cells are 0.0, not -inf. idx may be NULL in the forward. */
int odl_hip_max_pool2d(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
                       int PH, int PW, float *y, uint64_t *idx, void *stream);
int odl_hip_max_pool2d_backward(const float *gy, const uint64_t *idx, int64_t N, int64_t C, int64_t H, int64_t W,
                                int KH, int KW, int SH, int SW, int PH, int PW, float *gx, void *stream);
/* max_pool2d_backward followed by the backward of the ReLU whose output x was pooled, in one pass:
 * gx = pool_backward(gy, idx) * (x > 0 ? 1 : 0), the product of src/operators/activation/relu.cpp:23-29 applied to the
 * pooling gradient (MaxPool2d::backward then ReLU::backward, src/operators/pooling/max_pool2d.cpp:60-86), same floats
 * as the two calls in turn. Windows that tile the image exactly (2x2/2, 3x3/3) write each cell once, masked; other
 * windows run the two steps. x has the shape of gx. */
int odl_hip_max_pool2d_backward_relu(const float *gy, const uint64_t *idx, const float *x, int64_t N, int64_t C, int64_t H,
                                     int64_t W, int KH, int KW, int SH, int SW, int PH, int PW, float *gx, void *stream);
/* The same from the pooled tensor y [N, C, OH, OW] instead of the pooling's input x: the cell that receives a window's
 * gradient is its maximum, so (x > 0) there is (y > 0), and every other cell gets the +0 it gets above — same floats.
 * Only for windows that tile the image exactly (2x2/2, 3x3/3, no padding); for the layers whose pooled input was never
 * written (odl_hip_conv2d_relu_max_pool2d). */
int odl_hip_max_pool2d_backward_relu_pooled(const float *gy, const uint64_t *idx, const float *y, int64_t N, int64_t C,
                                            int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH, int PW, float *gx,
                                            void *stream);
/* Conv2d + ReLU + MaxPool2d of a Sequential (src/nn/layers/conv2d.cpp, src/operators/activation/relu.cpp:13-21,
 * src/operators/pooling/max_pool2d.cpp:25-58) in one pass for the layers odl_hip_conv2d_relu_max_pool2d_ok names (1 / 0):
 * a 3x3 / stride 1 / padding 1 convolution with few input channels — a network's first layer — under a 2x2 / stride 2
 * pooling, H and W even. y [N, OC, H/2, W/2] and idx (window-local argmax as in odl_hip_max_pool2d; may be NULL) hold
 * the floats and indices of odl_hip_conv2d_act(relu) followed by odl_hip_max_pool2d; the tensor between them is never
 * written. No workspace. */
int odl_hip_conv2d_relu_max_pool2d_ok(int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC, int KH, int KW, int SH, int SW,
                                      int PH, int PW, int PKH, int PKW, int PSH, int PSW, int PPH, int PPW);
int odl_hip_conv2d_relu_max_pool2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W,
                                   int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int PKH, int PKW, int PSH,
                                   int PSW, int PPH, int PPW, float *y, uint64_t *idx, void *stream);
/* The three calls above with the window-local index in one byte instead of eight (windows of at most 256 cells), for a
 * caller that keeps the indices to itself between a fused layer's forward and backward — the host layer's Conv2d + ReLU +
 * MaxPool2d operator: the same index values, an eighth of their bytes written and read back. odl_hip_max_pool2d_compact
 * takes every window odl_hip_max_pool2d takes as long as the sizes fit 32 bits. */
int odl_hip_max_pool2d_compact(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW,
                               int PH, int PW, float *y, uint8_t *idx8, void *stream);
int odl_hip_max_pool2d_backward_relu_pooled_compact(const float *gy, const uint8_t *idx8, const float *y, int64_t N, int64_t C,
                                                    int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH, int PW,
                                                    float *gx, void *stream);
int odl_hip_conv2d_relu_max_pool2d_compact(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H,
                                           int64_t W, int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, int PKH,
                                           int PKW, int PSH, int PSW, int PPH, int PPW, float *y, uint8_t *idx8, void *stream);

/* ------------------------------------------------------------------ metrics ------------------------- */
/* argmax per row, first maximum (src/utils/metrics.cpp:40-53), and accuracy() (metrics.cpp:11-70) with
 * int32 labels; *host_acc = correct / N. */
int odl_hip_argmax_rows(const float *y, int64_t N, int64_t C, int64_t *out, void *stream);
int odl_hip_accuracy(const float *y, const int32_t *t, int64_t N, int64_t C, float *host_acc, void *workspace,
                     size_t workspace_bytes, void *stream);
size_t odl_hip_accuracy_workspace_bytes(int64_t N);

/* ------------------------------------------------------------------ elementwise --------------------- */
/* origin::cuda::{add,subtract,multiply,divide,gt,eq,ne,lt,le,ge} (cuda_ops.cuh:57-140): op 0 add, 1 sub, 2 mul, 3 div,
 * 4 greater-than, 5 equal, 6 not-equal, 7 less, 8 less-equal, 9 greater-equal (masks of 1.0f / 0.0f);
 * 10 sigmoid_backward(a = gy, b = y) = gy*y*(1-y) (mat.h:399), 11 silu_backward(a = gy, b = x) (mat.h:413),
 * 12 relu_backward(a = gy, b = x) = gy * (x > 0 ? 1 : 0): ReLU::backward's mask and product (relu.cpp:23-52) in one pass.
 * na == nb, or one side has a single element; anything else is the
 * reference's "complex broadcasting" runtime_error. out may alias a or b (add_inplace). */
int odl_hip_binary(int op, const float *a, int64_t na, const float *b, int64_t nb, float *out, void *stream);
/* origin::cuda::{relu,exp,log,negate,square,sqrt,sigmoid,silu}: op 0 relu, 1 exp, 2 log, 3 neg, 4 square, 5 sqrt,
 * 6 sigmoid = 1/(1+exp(-x)) (operation_templates.h:168-175), 7 silu = x*sigmoid(x) (src/mat/origin/cpu/activation/silu.cpp:49-56) */
int odl_hip_unary(int op, const float *a, int64_t n, float *out, void *stream);
/* origin::cuda::pow with a float32 scalar exponent (src/mat/origin/cpu/math/pow.cpp:35-43) */
int odl_hip_pow_scalar(const float *a, int64_t n, float exponent, float *out, void *stream);
/* ------------------------------------------------------------------ element types besides float32 -- */
/* The reference dispatches its elementwise, reduction and conversion operators over six element types
 * (include/origin/mat/origin/device_common/type_dispatcher.h:26-88). Type codes here are its DataType enumerators
 * (include/origin/mat/basic_types.h:19-27): 0 float32, 1 float64, 2 int8, 3 int32, 4 int64, 5 uint8. float32 is what the
 * hot path computes in; with code 0 these entry points forward to the float32 ones above. */
size_t odl_hip_dtype_size(int dtype);
/* origin::cuda::convert_datatype (src/mat/origin/cuda/type_conversion.cu; include/origin/mat/origin/cuda/cuda_kernels.cuh
 * type_conversion_kernel): dst[i] = static_cast<Dst>(src[i]) on the device, any pair of types */
int odl_hip_convert(const void *src, int src_dtype, void *dst, int dst_dtype, int64_t n, void *stream);
/* odl_hip_binary ops 0-9 in any element type; integer arithmetic wraps, an integer division by zero gives 0,
 * comparisons give 0/1 in the operands' type (operation_templates.h:177-240). Same broadcasting rule. */
int odl_hip_binary_dtype(int op, int dtype, const void *a, int64_t na, const void *b, int64_t nb, void *out, void *stream);
/* odl_hip_unary: relu, neg, square in any type; exp, log, sqrt, sigmoid, silu in the floating-point types only
 * (ODL_ERR_INVALID_ARG otherwise — the reference throws for integer inputs, e.g. src/mat/origin/cpu/math/log.cpp) */
int odl_hip_unary_dtype(int op, int dtype, const void *a, int64_t n, void *out, void *stream);
/* pow with a scalar exponent for float32 / float64 (src/mat/origin/cpu/math/pow.cpp:14-44; the operator promotes integer
 * tensors to float32 before it gets here, src/operators/math/pow.cpp) */
int odl_hip_pow_scalar_dtype(int dtype, const void *a, int64_t n, double exponent, void *out, void *stream);
/* origin::cuda::{zeros,ones,full}, from_scalar in any type: host_value points at ONE element of that type on the host */
int odl_hip_fill_dtype(void *dst, int dtype, int64_t n, const void *host_value, void *stream);
/* OriginMat::permute (include/origin/mat/origin/origin_mat.h:75; src/mat/origin/cuda/shape/permute.cu,
 * src/mat/origin/cpu/shape/permute.cpp:22-110): a dense copy whose dimension d is the input's dimension host_perm[d],
 * any element type, up to 8 dimensions. ODL_ERR_INVALID_ARG for an order that is not a permutation. */
int odl_hip_permute(const void *src, int dtype, const int64_t *host_shape, int ndim, const int *host_perm, void *dst,
                    void *stream);
/* Mat::max, Mat::broadcast_to and Mat::sum_to in any element type (src/mat/origin/cuda/math/{max,broadcast_to,sum_to}.cu
 * dispatch over the type; CPU forms src/mat/origin/cpu/math/max.cpp:20-121, operation_templates.h:433-493,
 * src/mat/origin/cpu/math/sum_to.cpp:11-76): the semantics and errors of the float32 entry points above — max starts from
 * the type's lowest value and takes v where `m < v`; the whole-tensor maximum starts from the first element; sum_to
 * compares shapes from the LEFT, integers sum with wrap-around. Type code 0 forwards to the float32 kernels. */
int odl_hip_max_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis, int64_t inner, void *dst, void *stream);
int odl_hip_max_all_dtype(int dtype, const void *src, int64_t n, void *dst, void *stream);
int odl_hip_broadcast_to_dtype(int dtype, const void *src, const int64_t *host_src_shape, int src_ndim,
                               const int64_t *host_dst_shape, int dst_ndim, void *dst, void *stream);
int odl_hip_sum_to_dtype(int dtype, const void *src, const int64_t *host_src_shape, int src_ndim, const int64_t *host_dst_shape,
                         int dst_ndim, void *dst, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_sum_to_dtype_workspace_bytes(int dtype, const int64_t *host_src_shape, int src_ndim,
                                            const int64_t *host_dst_shape, int dst_ndim);
/* Mat::cat and one piece of Mat::split in any element type (src/mat/origin/cuda/shape/{cat,split}.cu dispatch over the
 * type): odl_hip_cat and odl_hip_slice_axis for elements of odl_hip_dtype_size(dtype) bytes. */
int odl_hip_cat_dtype(int dtype, const void *const *host_inputs, const int64_t *host_axis_sizes, int count, int64_t outer,
                      int64_t inner, void *out, void *stream);
int odl_hip_slice_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis_size, int64_t inner, int64_t offset,
                             int64_t length, void *dst, void *stream);
/* Mat::gather, Mat::upsample and Mat::upsample_backward in any element type (src/mat/origin/cuda/nn/gather.cu:189 and
 * upsample.cu:176, 224 dispatch over the type): the semantics of the float32 entry points; gather and the forward are
 * copies, the backward adds in the element type (integers wrap). one_hot gives float32 whatever the labels' type
 * (gather.cu:234). */
int odl_hip_gather_dtype(int dtype, const void *in, const void *idx, int idx_is_i64, int64_t N, int64_t C, void *out,
                         void *stream);
int odl_hip_upsample_nearest_dtype(int dtype, const void *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                                   int scale_h, int scale_w, void *y, void *stream);
int odl_hip_upsample_nearest_backward_dtype(int dtype, const void *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                                            int64_t OW, int scale_h, int scale_w, void *gx, void *stream);
/* Mat::sum over [outer, axis, inner] in any type (operation_templates.h:270-357): integers sum with wrap-around in their
 * own width, float64 in a fixed parallel order. through_float != 0 passes each result through a float on its way back
 * into the element type, which is what the reference's whole-tensor sum does (src/mat/origin/cpu/math/sum.cpp:18-35,83-90). */
int odl_hip_sum_axis_dtype(int dtype, const void *src, int64_t outer, int64_t axis, int64_t inner, int through_float,
                           void *dst, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_sum_axis_dtype_workspace_bytes(int dtype, int64_t outer, int64_t axis, int64_t inner);

/* ------------------------------------------------------------------ detector forward path ------------ */
/* Mat::upsample, mode "nearest" (mat.h:770; src/mat/origin/cpu/nn/upsample.cpp:22-75):
 * y[n,c,oh,ow] = x[n,c,oh/scale_h,ow/scale_w]. Unlike the reference, an output that would index past x is refused. */
int odl_hip_upsample_nearest(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                             int scale_h, int scale_w, float *y, void *stream);
/* Mat::cat (mat.h:797; src/mat/origin/cpu/shape/cat.cpp:20-140): inputs viewed as [outer, axis_size_i, inner] are laid
 * side by side along the axis. host_inputs: `count` device pointers in a host array; host_axis_sizes: their axis extents. */
/* Mat::upsample_backward (mat.h:784; nn/upsample.cpp:80-135): each input pixel sums the scale_h x scale_w block of gy
 * it was copied to, rows then columns ascending (the reference's accumulation order: bit-identical). */
int odl_hip_upsample_nearest_backward(const float *gy, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                                      int scale_h, int scale_w, float *gx, void *stream);
/* Mat::split, one piece (mat.h:805; src/mat/origin/cpu/shape/split.cpp) — the backward of cat: src viewed as
 * [outer, axis_size, inner], dst = src[:, offset:offset+length, :]. */
int odl_hip_slice_axis(const float *src, int64_t outer, int64_t axis_size, int64_t inner, int64_t offset, int64_t length,
                       float *dst, void *stream);
int odl_hip_cat(const float *const *host_inputs, const int64_t *host_axis_sizes, int count, int64_t outer, int64_t inner,
                float *out, void *stream);
/* Mat::yolo_detect_forward (mat.h:719; src/mat/origin/cpu/custom/yolo_detect.cpp:28-166): 1x1 convolution
 * [A*(classes+5), C] (+bias), view [N,A,classes+5,H,W] -> [N, A*H*W, classes+5], sigmoid, xy = (2s+grid)*stride,
 * wh = (2s)^2*anchor. grid / anchor_grid are read with the reference's flat indexing ([A,H,W,2] and
 * [A,anchor_H,anchor_W,2]); entries past grid_elems / anchor_elems count as 0 / 1 as there. */
int odl_hip_yolo_detect_forward(const float *x, const float *conv_w, const float *conv_b, const float *grid,
                                int64_t grid_elems, const float *anchor_grid, int64_t anchor_elems, int64_t anchor_H,
                                int64_t anchor_W, int64_t N, int64_t C, int64_t H, int64_t W, float stride, int num_anchors,
                                int num_classes, float *out, void *workspace, size_t workspace_bytes, void *stream);
size_t odl_hip_yolo_detect_workspace_bytes(int64_t N, int64_t C, int64_t H, int64_t W, int num_anchors, int num_classes);

/* Operators of the detector's graph for tensors that are runs of channels inside a wider NCHW tensor — the inputs of a
 * torch.cat written where the concatenation would copy them (src/mat/origin/cpu/shape/cat.cpp:81-123), and read from
 * there by the nodes that follow. An image stride is the distance in floats from one image of the view to the next
 * (0: dense). Values are those of the dense entry points. No counterpart in the reference, whose runner materialises
 * every node's output (src/pnnx/pnnx_graph.cpp:286-528).
 *  upsample_nearest_view: odl_hip_upsample_nearest; OW and the output stride multiples of 4, y 16-byte aligned.
 *  max_pool2d_chain: `count` K x K / stride 1 / padding K/2 max pools applied one after the other (a detector's SPPF
 *    block); stage j's result goes to channels [(j-1)*C, j*C) of y. One launch, the plane stays in LDS (H*W <= 8192).
 *  copy_images: dst[n][j] = src[n][j] for j < count — one input of a concatenation, or a view made dense.
 *  yolo_decode: the second half of odl_hip_yolo_detect_forward (sigmoid + box decoding of conv[N, A*(classes+5), H, W])
 *    with the stage's rows written out_image_stride floats apart, i.e. straight into the concatenation of the stages.
 *  yolo_decode_stages: yolo_decode for 1 to 4 stages of one head (same N, anchors and classes) in one launch; the
 *    arrays are host arrays with one entry per stage, out[s] the first row of stage s. Same values as one call a stage. */
int odl_hip_upsample_nearest_view(const float *x, int64_t x_image_stride, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH,
                                  int64_t OW, int scale_h, int scale_w, float *y, int64_t y_image_stride, void *stream);
int odl_hip_max_pool2d_chain(const float *x, int64_t x_image_stride, int64_t N, int64_t C, int64_t H, int64_t W, int K,
                             int count, float *y, int64_t y_image_stride, void *stream);
int odl_hip_copy_images(const float *src, int64_t src_image_stride, float *dst, int64_t dst_image_stride, int64_t N,
                        int64_t count, void *stream);
int odl_hip_yolo_decode(const float *conv, const float *grid, int64_t grid_elems, const float *anchor_grid, int64_t anchor_elems,
                        int64_t anchor_H, int64_t anchor_W, int64_t N, int64_t H, int64_t W, float stride, int num_anchors,
                        int num_classes, float *out, int64_t out_image_stride, void *stream);
int odl_hip_yolo_decode_stages(int stages, const float *const *host_conv, const float *const *host_grid, const int64_t *host_grid_elems,
                               const float *const *host_anchor_grid, const int64_t *host_anchor_elems, const int64_t *host_anchor_H,
                               const int64_t *host_anchor_W, int64_t N, const int64_t *host_H, const int64_t *host_W,
                               const float *host_stride, int num_anchors, int num_classes, float *const *host_out,
                               int64_t out_image_stride, void *stream);
/* Mat::yolo_detect_forward (src/mat/origin/cpu/custom/yolo_detect.cpp:28-166) for the 1 to 4 stages of a head in one
 * launch: every stage's 1x1 convolution (x[s] a run with its image stride, packed[s] = odl_hip_conv2d_pack_weights of
 * its filter, host_b NULL or with NULL entries) decoded in the convolution's epilogue and written to out[s], the
 * stage's first row in the tensor that concatenates the stages (out_image_stride floats from image to image). The
 * floats are those of odl_hip_conv2d_fused followed by odl_hip_yolo_decode. ..._ok answers 1 for shapes it takes. */
int odl_hip_yolo_detect_stages_ok(int stages, int64_t N, const int64_t *host_C, const int64_t *host_H, const int64_t *host_W,
                                  int num_anchors, int num_classes);
int odl_hip_yolo_detect_stages_forward(int stages, const float *const *host_x, const int64_t *host_x_image_stride,
                                       const float *const *host_packed, const float *const *host_b, const float *const *host_grid,
                                       const int64_t *host_grid_elems, const float *const *host_anchor_grid,
                                       const int64_t *host_anchor_elems, const int64_t *host_anchor_H, const int64_t *host_anchor_W,
                                       int64_t N, const int64_t *host_C, const int64_t *host_H, const int64_t *host_W,
                                       const float *host_stride, int num_anchors, int num_classes, float *const *host_out,
                                       int64_t out_image_stride, void *stream);

/* Mat::batch_norm_forward / Mat::batch_norm (mat.h:603-631; src/mat/origin/cpu/normalization/batch_norm.cpp:31-258)
 * over x[N, C, P]: P = H*W for num_dims 4, P = 1 for num_dims 2. training != 0: per-channel mean and biased variance
 * of the batch (sum / count, then squared differences from that mean / count), written to mean[C] and var[C];
 * training == 0: mean and var are copies of the running statistics. Then x_norm = (x - mean) / sqrt(var + eps) and
 * y = gamma * x_norm + beta. x_norm may be NULL (the y-only Mat::batch_norm). running_mean / running_var may be NULL
 * in training mode; the workspace is needed in training mode only. */
int odl_hip_batch_norm_forward(const float *x, const float *gamma, const float *beta, const float *running_mean,
                               const float *running_var, int training, float eps, int64_t N, int64_t C, int64_t P,
                               float *y, float *mean, float *var, float *x_norm, void *workspace,
                               size_t workspace_bytes, void *stream);
/* Mat::batch_norm_backward (mat.h:643; batch_norm.cpp:279-418): dbeta = sum gy, dgamma = sum gy * x_norm per channel,
 * gx = (gamma / sqrt(saved_var + eps)) * (gy - dbeta/count - x_norm * dgamma/count). */
int odl_hip_batch_norm_backward(const float *gy, const float *gamma, const float *saved_var, const float *saved_x_norm,
                                float eps, int64_t N, int64_t C, int64_t P, float *gx, float *dgamma, float *dbeta,
                                void *workspace, size_t workspace_bytes, void *stream);
/* The same gradients from x and the saved statistics instead of a saved x_norm: the normalised value is formed again
 * in the kernel, (x - mean) / sqrt(var + eps), the expression — and so the float — of the forward pass. A caller that
 * keeps x anyway (an autograd operator does) need not store x_norm at all and calls the forward with x_norm = NULL. */
int odl_hip_batch_norm_backward_from_x(const float *gy, const float *x, const float *gamma, const float *saved_mean,
                                       const float *saved_var, float eps, int64_t N, int64_t C, int64_t P, float *gx,
                                       float *dgamma, float *dbeta, void *workspace, size_t workspace_bytes,
                                       void *stream);
/* A batch normalisation whose output goes straight into a ReLU, as in the reference's CNN example
 * (tests/example/mnist/conv_mnist.cpp: Conv2d, BatchNorm2d, ReLU, MaxPool2d): y = relu(gamma * x_norm + beta) is
 * written once instead of the normalised tensor and then its ReLU; mean / var as in the plain forward, no x_norm.
 * The backward takes the gradient of the ReLU's OUTPUT: the mask gamma * x_norm + beta > 0 is formed again from x and
 * the saved statistics (the floats of the forward pass), gy is multiplied by 1 or 0 as the separate ReLU backward
 * does (relu.cpp:45-52), and the sums and gx follow from that product. Results equal the two separate steps bit
 * for bit. */
int odl_hip_batch_norm_relu_forward(const float *x, const float *gamma, const float *beta, const float *running_mean,
                                    const float *running_var, int training, float eps, int64_t N, int64_t C, int64_t P,
                                    float *y, float *mean, float *var, void *workspace, size_t workspace_bytes,
                                    void *stream);
int odl_hip_batch_norm_relu_backward_from_x(const float *gy, const float *x, const float *gamma, const float *beta,
                                            const float *saved_mean, const float *saved_var, float eps, int64_t N,
                                            int64_t C, int64_t P, float *gx, float *dgamma, float *dbeta,
                                            void *workspace, size_t workspace_bytes, void *stream);
/* workspace of any of these calls (partial channel sums) */
size_t odl_hip_batch_norm_workspace_bytes(int64_t N, int64_t C, int64_t P);
/* The same on float64 tensors (src/mat/origin/cuda/normalization/batch_norm.cu:497-560 accepts float32 and float64): one
 * workgroup per channel, no workspace. x_norm may be NULL. backward: x_norm_or_x is the saved normalised input
 * (from_x = 0), or x itself with saved_mean (from_x != 0). */
int odl_hip_batch_norm_forward_f64(const double *x, const double *gamma, const double *beta, const double *running_mean,
                                   const double *running_var, int training, double eps, int64_t N, int64_t C, int64_t P,
                                   double *y, double *mean, double *var, double *x_norm, void *stream);
int odl_hip_batch_norm_backward_f64(const double *gy, const double *x_norm_or_x, int from_x, const double *gamma,
                                    const double *saved_mean, const double *saved_var, double eps, int64_t N, int64_t C,
                                    int64_t P, double *gx, double *dgamma, double *dbeta, void *stream);
/* out = a*x + b*y, each product rounded before the sum: the running-statistics update of the BatchNorm layers
 * (src/nn/layers/batch_norm2d.cpp:77-80, batch_norm1d.cpp), which the reference does on the host after four
 * device-to-host copies. out may be x or y. */
int odl_hip_axpby(float a, const float *x, float b, const float *y, int64_t n, float *out, void *stream);

/* Fused optimizer steps. The reference has no Mat virtual for them: Adam::step_one (src/optim/adam.cpp:52-113) and
 * SGD::step_one (src/optim/sgd.cpp:18-75) issue the same arithmetic as ~15 whole-tensor Mat operations per parameter.
 * Each element goes through the identical sequence of separately rounded float operations
 * (m = m*b1 + g*(1-b1); v = v*b2 + (g*g)*(1-b2); p_out = p - ((m*m_hat_scale) / (powf(v*v_hat_scale, 0.5) + eps))*lr),
 * with m_hat_scale = 1/(1-b1^t) and v_hat_scale = 1/(1-b2^t) computed by the caller in float as the reference does.
 * m and v are updated in place; p_out may be p. sgd_step: p_out = p - g*lr (no momentum, no weight decay). */
int odl_hip_adam_step(const float *p, const float *g, float *m, float *v, int64_t n, float beta1, float beta2,
                      float m_hat_scale, float v_hat_scale, float eps, float lr, float *p_out, void *stream);
/* the same step with m_hat_scale and v_hat_scale read from device memory (device_scales[0], [1]): for a step that
 * is recorded into a graph once and replayed, where the step count changes between replays and the caller rewrites
 * the two floats before each one */
int odl_hip_adam_step_device_scales(const float *p, const float *g, float *m, float *v, int64_t n, float beta1,
                                    float beta2, const float *device_scales, float eps, float lr, float *p_out,
                                    void *stream);
int odl_hip_sgd_step(const float *p, const float *g, int64_t n, float lr, float *p_out, void *stream);
/* The same steps over a whole list of parameters in one launch (Optimizer::step, src/optim/optimizer.cpp:19-53, walks
 * the parameters one by one; most of them are biases of a few hundred floats, so the walk is launch-bound). The
 * arguments are host arrays of `count` device pointers and sizes; entry i gets exactly what the one-tensor call
 * gives. adam_step_multi: m_hat_scale[i], v_hat_scale[i] from the host arrays, unless device_scales (an array, or
 * NULL) holds a non-NULL device pointer for entry i (two floats, as in odl_hip_adam_step_device_scales).
 * axpy_multi: y[i] += alpha * x[i], the product rounded before the sum — the WeightDecay hook
 * (include/origin/optim/hooks.h: grad += rate * param) over all parameters. Empty tensors are skipped. */
int odl_hip_adam_step_multi(int count, const float *const *p, const float *const *g, float *const *m, float *const *v,
                            const int64_t *n, float beta1, float beta2, const float *m_hat_scale, const float *v_hat_scale,
                            const float *const *device_scales, float eps, float lr, float *const *p_out, void *stream);
int odl_hip_sgd_step_multi(int count, const float *const *p, const float *const *g, const int64_t *n, float lr,
                           float *const *p_out, void *stream);
int odl_hip_axpy_multi(int count, float alpha, const float *const *x, float *const *y, const int64_t *n, void *stream);
/* The WeightDecay hook and the step it precedes (Optimizer::step runs the hooks, then the steps) in one pass over the
 * parameters: g[i] += weight_decay * p[i] (product rounded, then the sum, as axpy_multi) is written back to g[i] — the
 * caller's gradients hold the decayed values afterwards, as after the hook — and the step uses that g. The floats of
 * axpy_multi followed by adam_step_multi / sgd_step_multi. */
int odl_hip_adam_step_multi_decay(int count, const float *const *p, float *const *g, float *const *m, float *const *v,
                                  const int64_t *n, float weight_decay, float beta1, float beta2, const float *m_hat_scale,
                                  const float *v_hat_scale, const float *const *device_scales, float eps, float lr,
                                  float *const *p_out, void *stream);
int odl_hip_sgd_step_multi_decay(int count, const float *const *p, float *const *g, const int64_t *n, float weight_decay,
                                 float lr, float *const *p_out, void *stream);
/* origin::cuda::{zeros,ones,full} (cuda/factory.cuh:23-50) */
int odl_hip_fill(float *dst, int64_t n, float value, void *stream);

#ifdef __cplusplus
}
#endif
#endif
