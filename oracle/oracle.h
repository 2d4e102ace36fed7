/*
 * CPU oracle for the OriginDL hot path — TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A plain-C, single-threaded restatement of the reference's CPU backend algorithms
 * (src/mat/origin/cpu/** and the operators that compose them), same loop order and the
 * same float rounding points, compiled with -ffp-contract=off so that no FMA is formed
 * (the reference is built -O2 for x86-64, which forms none either).
 *
 * Only the tests, the smoke check and the CPU-baseline leg of the benchmark may load this
 * library; the shipped HIP library never does.
 *
 * Pinning status: every function below is checked against (1) the golden vectors held by the
 * reference's own unit tests, (2) the compiled reference CPU backend (oracle/_ref, built from
 * the reference sources where available) on seeded random inputs, bit for bit, and (3)
 * independent mathematics (numpy closed forms, brute force). No function is "parity unpinned".
 *
 * All matrices are dense row-major float32 unless the name says otherwise. Dimensions are
 * int64_t. Functions that mirror a reference exception return a negative code instead:
 *   ORC_ERR_INVALID_ARG   (-1)  std::invalid_argument in the reference
 *   ORC_ERR_RUNTIME       (-2)  std::runtime_error in the reference
 */
#ifndef ODL_ORACLE_H
#define ODL_ORACLE_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_OK 0
#define ORC_ERR_INVALID_ARG (-1)
#define ORC_ERR_RUNTIME (-2)

/* ---- GEMM ------------------------------------------------------------------------------- */
/* src/mat/origin/cpu/math/matmul.cpp:27-41 (2D), 55-76 (3D x 2D), 91-109 (3D x 3D) */
void orc_matmul(const float *a, const float *b, float *c, int64_t m, int64_t n, int64_t k);
void orc_matmul_batched(const float *a, const float *b, float *c, int64_t batch, int64_t m, int64_t n, int64_t k,
                        int b_is_batched);
/* rows [row0,row1) of C only: rows are independent in the reference loop (used for sampled parity
 * and for the sliced CPU baseline at sizes the full loop cannot finish). */
void orc_matmul_rows(const float *a, const float *b, float *c_rows, int64_t row0, int64_t row1, int64_t n, int64_t k);
/* include/origin/mat/origin/device_common/operation_templates.h:374-390, 401-416 */
void orc_transpose(const float *src, float *dst, int64_t outer, int64_t rows, int64_t cols);
/* src/operators/math/mat_mul.cpp:171-177: gx = gy . transpose(w), gw = transpose(x) . gy,
 * with the transposes materialised and the products run by orc_matmul. */
void orc_matmul_backward(const float *x, const float *w, const float *gy, float *gx, float *gw, int64_t m, int64_t k,
                         int64_t n);

/* ---- convolution ------------------------------------------------------------------------ */
/* include/origin/utils/conv_utils.h: (in + 2p - k) / s + 1 */
int64_t orc_conv_outsize(int64_t in, int64_t k, int64_t s, int64_t p);
/* src/mat/origin/cpu/conv/conv2d.cpp:39-207. to_matrix!=0: col[N*OH*OW, C*KH*KW]; else [N,C,KH,KW,OH,OW] */
int orc_im2col(const float *img, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
               int PW, int to_matrix, float *col);
/* conv2d.cpp:212-377 */
int orc_col2im(const float *col, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
               int PW, int to_matrix, float *img);
/* conv2d.cpp:404-512; b may be NULL */
int orc_conv2d(const float *x, const float *w, const float *b, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OC,
               int KH, int KW, int SH, int SW, int PH, int PW, float *y);
/* conv2d.cpp:514-599 — including the zero-copy reinterpretation of gy[N,OC,OH,OW] as [N*OH*OW, OC]
 * (line 548) and the three-pass bias reduction sum(2).sum(2).sum(0) (571-575). gb may be NULL. */
int orc_conv2d_backward(const float *gy, const float *x, const float *w, int64_t N, int64_t C, int64_t H, int64_t W,
                        int64_t OC, int KH, int KW, int SH, int SW, int PH, int PW, float *gx, float *gw, float *gb);

/* ---- reductions / broadcast -------------------------------------------------------------- */
/* operation_templates.h:270-333 seen as [outer, axis, inner]; sequential over the axis, ascending */
void orc_sum_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst);
/* operation_templates.h:342-357 via src/mat/origin/cpu/math/sum.cpp:82-90 */
float orc_sum_all(const float *src, int64_t n);
/* src/mat/origin/cpu/math/max.cpp:58-117 (axis) and 25-40 (all) */
void orc_max_axis(const float *src, int64_t outer, int64_t axis, int64_t inner, float *dst);
float orc_max_all(const float *src, int64_t n);
/* src/mat/origin/cpu/math/sum_to.cpp:11-76: LEFT-aligned. Returns ORC_ERR_RUNTIME when the target has
 * more elements (line 24-28) and ORC_ERR_INVALID_ARG when the reduced result cannot be reshaped to the
 * target (reshape throws, src/mat/origin/origin_mat.cpp:417-437). dst holds prod(tshape) floats. */
int orc_sum_to(const float *src, const int64_t *sshape, int sn, const int64_t *tshape, int tn, float *dst);
/* operation_templates.h:433-493: RIGHT-aligned */
void orc_broadcast_to(const float *src, const int64_t *sshape, int sn, const int64_t *dshape, int dn, float *dst);

/* ---- softmax / cross entropy ------------------------------------------------------------- */
/* src/operators/activation/softmax.cpp:37-74 on [outer, axis, inner] */
void orc_softmax(const float *x, int64_t outer, int64_t axis, int64_t inner, float *y);
/* src/mat/origin/cpu/nn/gather.cpp:21-88 / 91-158; idx_is_i64 selects the label width */
int orc_gather(const float *in, const void *idx, int idx_is_i64, int64_t N, int64_t C, float *out);
int orc_one_hot(const void *idx, int idx_is_i64, int64_t N, int64_t C, float *out);
/* src/operators/loss/softmax_cross_entropy.cpp:17-75; loss written to *loss */
int orc_softmax_ce_loss(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, float *loss);
/* softmax_cross_entropy.cpp:77-111: gx = (softmax(x) - one_hot(t)) * (gy / N) */
int orc_softmax_ce_grad(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t C, float gy, float *gx);

/* ---- pooling ----------------------------------------------------------------------------- */
/* src/mat/origin/cpu/pooling/max_pool2d.cpp:40-146; idx = kh*KW+kw, first maximum wins, zero padding */
int orc_max_pool2d(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int KH, int KW, int SH, int SW, int PH,
                   int PW, float *y, uint64_t *idx);
/* max_pool2d.cpp:148-224 */
int orc_max_pool2d_backward(const float *gy, const uint64_t *idx, int64_t N, int64_t C, int64_t H, int64_t W, int KH,
                            int KW, int SH, int SW, int PH, int PW, float *gx);

/* ---- metrics ------------------------------------------------------------------------------ */
/* src/utils/metrics.cpp:40-60: host argmax (first maximum, strict >) */
void orc_argmax_rows(const float *y, int64_t N, int64_t C, int64_t *out);
float orc_accuracy(const float *y, const int32_t *t, int64_t N, int64_t C);

/* ---- elementwise (src/mat/origin/cpu/math/{add,subtract,multiply,divide}.cpp, compare.cpp, relu.cpp,
 *      exp.cpp, log.cpp, pow.cpp, negate.cpp, square.cpp) ------------------------------------------ */
/* op: 0 add 1 sub 2 mul 3 div 4 gt-mask(1.0/0.0). na==nb (same shape) or one of them ==1 (single-element
 * broadcast); anything else is the reference's "complex broadcasting" runtime_error. */
int orc_binary(int op, const float *a, int64_t na, const float *b, int64_t nb, float *out);
/* op: 0 relu 1 exp 2 log 3 neg 4 square 5 sqrt */
void orc_unary(int op, const float *a, int64_t n, float *out);
void orc_pow_scalar(const float *a, int64_t n, float e, float *out);

/* detector forward path: nn/upsample.cpp:22-75, shape/cat.cpp:20-140, custom/yolo_detect.cpp:28-166 */
int orc_upsample_nearest(const float *x, int64_t N, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW, int scale_h,
                         int scale_w, float *y);
int orc_cat(const float *const *inputs, const int64_t *axis_sizes, int count, int64_t outer, int64_t inner, float *out);
int orc_yolo_detect_forward(const float *x, const float *conv_w, const float *conv_b, const float *grid, int64_t grid_elems,
                            const float *anchor_grid, int64_t anchor_elems, int64_t anchor_H, int64_t anchor_W, int64_t N,
                            int64_t C, int64_t H, int64_t W, float stride, int num_anchors, int num_classes, float *out);

/* batch normalisation over x[N][C][P] (P = H*W, or 1 for [N][C]): normalization/batch_norm.cpp:31-258, 279-418 */
int orc_batch_norm_forward(const float *x, const float *gamma, const float *beta, const float *running_mean,
                           const float *running_var, int training, float eps, int64_t N, int64_t C, int64_t P, float *y,
                           float *mean, float *var, float *x_norm);
int orc_batch_norm_backward(const float *gy, const float *gamma, const float *saved_var, const float *saved_x_norm,
                            float eps, int64_t N, int64_t C, int64_t P, float *gx, float *dgamma, float *dbeta);

/* ---- whole training steps (compositions restated from the reference's operators/optimizers) --------- */
/* MLP: x[N,D] -> Linear(D,Hd)+ReLU -> Linear(Hd,C) -> softmax CE; backward; WeightDecay hook (grad += wd*p,
 * include/origin/optim/hooks.h:40-65); Adam step t (src/optim/adam.cpp:19-114). Parameters and Adam
 * moments are updated in place; grads (gW1,gb1,gW2,gb2; before weight decay) and the loss are returned. */
int orc_mlp_train_step(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t D, int64_t Hd, int64_t C,
                       float *W1, float *b1, float *W2, float *b2, float *mW1, float *vW1, float *mb1, float *vb1,
                       float *mW2, float *vW2, float *mb2, float *vb2, int step_t, float lr, float beta1, float beta2,
                       float eps, float wd, float *loss, float *gW1, float *gb1, float *gW2, float *gb2,
                       float *logits);

/* CNN (the benchmark's CNN training configuration): x[N,1,S,S] -> conv(1->C1,3x3,p1) ReLU maxpool2 -> conv(C1->C2,3x3,p1) ReLU maxpool2
 * -> flatten -> Linear(F,Hd) ReLU -> Linear(Hd,Cc) -> softmax CE; backward; SGD (src/optim/sgd.cpp:18-75,
 * no momentum, no weight decay). Parameters updated in place. Returns loss, pool indices and all grads. */
int orc_cnn_train_step(const float *x, const void *t, int idx_is_i64, int64_t N, int64_t S, int64_t C1, int64_t C2,
                       int64_t Hd, int64_t Cc, float *Wc1, float *bc1, float *Wc2, float *bc2, float *Wl1, float *bl1,
                       float *Wl2, float *bl2, float lr, float *loss, uint64_t *idx1, uint64_t *idx2, float *gWc1,
                       float *gbc1, float *gWc2, float *gbc2, float *gWl1, float *gbl1, float *gWl2, float *gbl2,
                       float *logits);

#ifdef __cplusplus
}
#endif
#endif
