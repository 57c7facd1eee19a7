/*
 * CPU oracle for Tenmo's fp32 matrix-product path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library restates, in plain C++, the
 * algorithms of the reference's CPU path so that the HIP library can be checked
 * against them and so that a CPU baseline can be timed beside the GPU numbers.
 * Nothing in the product (tenmo_amd/, libtenmo_hip.so) links, loads or calls it.
 *
 * All sizes, offsets and strides are in ELEMENTS.  A view is
 *   element(idx) = data[offset + sum_d idx[d] * strides[d]]
 * exactly as the reference's NDBuffer (tenmo/ndbuffer.mojo, shape/strides/offset).
 */
#ifndef TENMO_ORACLE_CPU_H
#define TENMO_ORACLE_CPU_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORACLE_MAX_RANK 8 /* tenmo/mnemonics.mojo:45 max_rank */

typedef struct {
    const float* data;
    int64_t offset;
    int32_t rank;
    int64_t shape[ORACLE_MAX_RANK];
    int64_t strides[ORACLE_MAX_RANK];
} oracle_view;

/* error handling: every function returns 0 on success, <0 on a condition for
 * which the reference panics; the message is kept per thread. */
const char* oracle_last_error(void);

/* ISA level picked at run time: 16 (AVX-512), 8 (AVX2+FMA) or 1 (portable). */
int oracle_simd_width(void);
void oracle_force_simd_width(int w); /* 0 = auto; tests use it to cover all kernels */
int oracle_num_physical_cores(void);

/* tenmo/strides.mojo:239-266 */
int oracle_is_contiguous(int32_t rank, const int64_t* shape, const int64_t* strides);

/* tenmo/matmul.mojo:258-272 -> 0 dot, 1 vm, 2 mv, 3 mm, -1 invalid */
int oracle_classify_matmul(int32_t rank_a, const int64_t* shape_a, int32_t rank_b, const int64_t* shape_b);

/* tenmo/matmul_cpu.mojo:80-135 (tile table) + :163-547 (three paths).
 * C is dense [m,p]; it is overwritten.  nthreads<=0 -> physical cores.
 * path_out (optional): 0 = 1a, 1 = 1b, 2 = path 2.  tiles_out (optional): TILE_M,N,P. */
int oracle_mm2d_f32(const oracle_view* A, const oracle_view* B, float* C, int nthreads, int* path_out, int* tiles_out);

/* tenmo/matmul_cpu.mojo:568-625 + :628-956.  C dense [batch..., m, p]; out_shape receives the
 * broadcast result shape (rank = max(rankA,rankB)).  row_tile_limit>0 processes only the first
 * row_tile_limit flat work items (used to time a bounded sample of a huge case). */
int oracle_mmnd_f32(const oracle_view* A, const oracle_view* B, float* C, int nthreads,
                    int64_t* out_shape, int32_t* out_rank, int64_t work_item_limit);

/* result shape helper for mm / mv / vm (mode: 3 mm, 2 mv, 1 vm); returns element count or <0 */
int64_t oracle_result_shape(int mode, const oracle_view* A, const oracle_view* B, int64_t* out_shape, int32_t* out_rank);

/* tenmo/matrixvector.mojo:205-286 ; tenmo/vectormatrix.mojo:210-338 ; single thread as the reference */
int oracle_mv_f32(const oracle_view* M, const oracle_view* v, float* out);
int oracle_vm_f32(const oracle_view* v, const oracle_view* M, float* out);
/* backward: grads are dense at the PARENT's shape, zero-filled here then accumulated
 * (tenmo/matrixvector.mojo:19-201, tenmo/vectormatrix.mojo:18-206). dy dense at result shape. */
int oracle_mv_backward_f32(const oracle_view* M, const oracle_view* v, const float* dy, float* dM, float* dv);
int oracle_vm_backward_f32(const oracle_view* v, const oracle_view* M, const float* dy, float* dv, float* dM);
/* tenmo/dotproduct.mojo:56-123 (after the size-1 broadcast) : sum a_i*b_i, fp32, i ascending */
int oracle_dot_f32(const oracle_view* a, const oracle_view* b, float* out);

/* tenmo/sum_mean_reduction.mojo:185-211: reduce dense src[src_shape] to the (right-aligned)
 * target shape by summing leading and size-1-mismatched axes; dst dense at target shape. */
int oracle_sum_over_broadcasted_axes_f32(const float* src, int32_t src_rank, const int64_t* src_shape,
                                         int32_t dst_rank, const int64_t* dst_shape, float* dst);

/* fp64-accumulated references on the same fp32 inputs (the tolerance anchor): */
int oracle_mmnd_f64acc(const oracle_view* A, const oracle_view* B, double* C, int nthreads);
int oracle_mv_f64acc(const oracle_view* M, const oracle_view* v, double* out);
int oracle_vm_f64acc(const oracle_view* v, const oracle_view* M, double* out);

/* ---- MLP-step harness (callers of the path; tenmo/net.mojo:179-216, addition.mojo:73-112,
 * relu.mojo:99-141, crossentropy.mojo:285-432,:775-793, optim.mojo:93-120) ---------------- */
typedef struct oracle_mlp oracle_mlp;
/* dims[0..n_layers] = layer widths (784,128,32,10); weights W_l [in,out] dense, biases [out]; copied in */
oracle_mlp* oracle_mlp_create(int n_layers, const int64_t* dims, const float* const* W, const float* const* b, int64_t max_batch);
void oracle_mlp_destroy(oracle_mlp*);
/* one training step: forward, mean cross-entropy, backward, SGD p -= lr*g.  returns loss */
float oracle_mlp_step(oracle_mlp*, const float* x, const int32_t* y, int64_t batch, float lr, int nthreads);
/* forward only -> logits [batch, dims[n_layers]] */
int oracle_mlp_forward(oracle_mlp*, const float* x, int64_t batch, float* logits, int nthreads);
int oracle_mlp_get_params(oracle_mlp*, int layer, float* W, float* b);
/* last step's parameter gradients */
int oracle_mlp_get_grads(oracle_mlp*, int layer, float* dW, float* db);

/* class-index cross-entropy, tenmo/crossentropy.mojo:285-432 (forward) and :744-770, :451-481
 * (gradient); reduction 0 none, 1 sum, 2 mean */
int oracle_cross_entropy_forward_f32(const float* logits, const int64_t* target, int64_t M, int64_t C, int64_t ignore_index,
                                     float label_smoothing, float* softmax, float* per_sample_loss, float* loss_sum, int32_t* valid_count);
int oracle_cross_entropy_backward_f32(const float* softmax, const int64_t* target, const float* upstream, int64_t M, int64_t C,
                                      int64_t ignore_index, float label_smoothing, int reduction, int32_t valid_count, float* grad);
/* SGD step, tenmo/optim.mojo:93-160 */
int oracle_sgd_step_f32(float* param, const float* grad, float* velocity, int64_t n, float lr, float momentum, float weight_decay);

/* FusedIm2Col.forward on a padded image, tenmo/cnn.mojo:308-507 */
int oracle_conv2d_forward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                              const float* kernel, int64_t c_out, int64_t kh, int64_t kw, const float* bias,
                              int64_t stride, int64_t dilation, float* out);

/* FusedCol2ImBackward: bias, kernel and padded-image gradients, tenmo/cnn.mojo:546-948 */
int oracle_conv2d_backward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                               const float* kernel, int64_t c_out, int64_t kh, int64_t kw, int64_t stride, int64_t dilation,
                               const float* grad_out, float* grad_padded_image, float* grad_kernel, float* grad_bias);

#ifdef __cplusplus
}
#endif
#endif
