/*
 * libtenmo_hip.so — MI355X (gfx950) implementation of Tenmo's fp32 matrix-product path.
 *
 * C ABI only: plain pointers and sizes, no C++ or framework types.  Every pointer named
 * "device" is HIP device memory on the GPU selected by tenmo_hip_init(); every size, offset
 * and stride is in ELEMENTS (fp32), never bytes.  An operand is a view
 *     element(i, j) = base[offset + sum_d batch_coord[d]*batch_stride[d] + i*row_stride + j*col_stride]
 * which is the reference's NDBuffer (shape, strides, offset over shared storage).  Strides may
 * be swapped (transposed view), padded, zero (broadcast) or overlapping; inputs are never written.
 *
 * Calls are enqueued on one library stream and return without waiting unless `sync` is
 * non-zero (the reference enqueues on its DeviceContext and synchronises on demand,
 * tenmo/kernels/matmul_kernel.mojo:259-277).  All functions return 0 on success or a
 * negative tenmo_status; they never abort and never throw.  The message of the last failure on
 * the calling thread is returned by tenmo_hip_last_error() — the text a Mojo caller would put
 * into `raise Error(msg)`.
 *
 * Single caller thread per process is assumed (as in the reference); calls issued from one
 * thread execute in issue order.
 */
#ifndef TENMO_HIP_H
#define TENMO_HIP_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TENMO_MAX_RANK 8 /* tenmo/mnemonics.mojo:45 (max_rank) */

typedef enum {
    TENMO_OK = 0,
    TENMO_ERR_NOT_INITIALIZED = -1,
    TENMO_ERR_INVALID_SHAPE = -2,   /* where the reference panics / raises on shapes */
    TENMO_ERR_INVALID_ARGUMENT = -3,
    TENMO_ERR_HIP = -4,             /* a HIP runtime call failed; message carries hipGetErrorString */
    TENMO_ERR_UNSUPPORTED = -5
} tenmo_status;

/* opcodes of tenmo/mnemonics.mojo:26-30 as returned by tenmo_hip_classify_matmul */
enum { TENMO_OP_DOT = 0, TENMO_OP_VM = 1, TENMO_OP_MV = 2, TENMO_OP_MM = 3, TENMO_OP_INVALID = -1 };

/* NDBuffer as seen by the device code: tenmo/ndbuffer.mojo (shape, strides, offset, storage). */
typedef struct {
    const float* data;  /* device pointer to the first element of the STORAGE */
    int64_t offset;     /* elements */
    int32_t rank;       /* <= TENMO_MAX_RANK */
    int64_t shape[TENMO_MAX_RANK];
    int64_t strides[TENMO_MAX_RANK];
} tenmo_view;

/* ---- lifetime, stream, errors ------------------------------------------------------------ */

/* Selects the GPU, creates the library stream and its scratch.  Idempotent.
 * Replaces: DeviceContext(device_id) in tenmo/device.mojo:87-90. */
int tenmo_hip_init(int device_id);
int tenmo_hip_shutdown(void);
/* == DeviceContext.synchronize(), tenmo/kernels/matmul_kernel.mojo:277 */
int tenmo_hip_sync(void);
const char* tenmo_hip_last_error(void);
/* The hipStream_t all work is enqueued on (as void*), and a way to make the library use the
 * caller's stream instead (NULL restores the library's own). */
void* tenmo_hip_get_stream(void);
int tenmo_hip_set_stream(void* hip_stream);
/* Device facts the caller may want for reporting: number of compute units, name. */
int tenmo_hip_device_info(int* compute_units, char* name, int name_len);
/* Overrides of the automatic kernel selection, for measurement: "gemm_tile" (0: 256x128, 1: 128x128,
 * 2: 64x64, 3: 128x64, 4: 64x128 workgroup tile; -1 automatic), "gemm_splitk" (number of K slices;
 * -1 automatic), "gemm_streamk" (n > 0: persistent stream-K launch with n workgroups per CU, at most two, for the
 * 256x128 / 128x128 tiles, 0: never, -1 automatic), "gemm_smallk" (the persistent short-reduction kernel, K of 17 up to 64 and a plain
 * or accumulating store: 1 wherever it can run, 3 the same and also for K up to 16 — a path the automatic choice does not take —, 0 never,
 * -1 automatic: for results of 2048 and more 64x64 tiles and K a multiple of 16),
 * "gemm_panel" (the persistent K-stream kernel with loading wavefronts of its own, 128x128 tiles, K above 16, plain or
 * accumulating store: 1 wherever it can run, 3 the same with 64x64 tiles and a deeper ring, 0 never, -1 automatic: K of 65 up to 512 and at least
 * three 128x128 tiles per CU), "gemm_resident" (a left operand of a few tile rows, K of 17 up to 256, against a wide right
 * operand with unit stride along N, one matrix, plain store: persistent workgroups that keep their rows of A in LDS and
 * stream B alone; 1 with 128x64 tiles, 2 with 64x64 tiles, 0 never, the default),
 * "fold_reduce" (the gradient of a parent that was broadcast over batch dimensions summed inside the GEMM launch instead
 * of materialised and reduced: 1 wherever it can run, 0 never, -1 automatic), "mlp_fused_tail" (tenmo_hip_mlp_step: the last
 * two layers, the loss, their backward and their update as one launch when they fit one workgroup — batch <= 64, widths
 * <= 128 / 64 / 32: 1 on, 2 the same and the first layer's weight gradient with its update as one launch, 3 the same and the first layer's forward as one launch, 0 off, the default), "cols_wg_per_cu" (workgroups per CU the
 * column-streaming kernel aims for), "cols_join" (vm, mv of a transposed view and skinny products whose reduction is cut
 * into K slices: 1 the slices are added by the last workgroup of the streaming launch — same bits, one launch less —, 0 by a
 * second launch, the default) and "conv_phases" (image gradient of a strided convolution phase by phase:
 * 1 always, 0 never, -1 automatic).  The
 * environment variables TENMO_HIP_GEMM_TILE / TENMO_HIP_GEMM_SPLITK / TENMO_HIP_GEMM_STREAMK / TENMO_HIP_GEMM_SMALLK / TENMO_HIP_GEMM_PANEL set the same at init.
 * No counterpart in the reference, whose tile size is the compile-time TILE_SIZE=32
 * (tenmo/ndbuffer.mojo:63). */
int tenmo_hip_set_tuning(const char* name, int value);
/* Stopwatch on the stream the kernels run on: begin records a HIP event, end records a second
 * one, waits for it and returns the milliseconds between them (the reference times with
 * perf_counter_ns around sync=True calls, profile_gpu.mojo:161-258). */
int tenmo_hip_timer_begin(void);
int tenmo_hip_timer_end(float* elapsed_ms);
/* Shader clock under a full matrix-core load, for reporting beside a throughput figure: every CU runs
 * 4 * rounds fp32 MFMAs per SIMD (64 cycles each) and nothing else, timed with HIP events on the library's stream;
 * effective_mhz = cycles / time.  Synchronises.  No counterpart in the reference. */
int tenmo_hip_clock_probe(int32_t rounds, float* effective_mhz);

/* ---- kernel-level entry points ------------------------------------------------------------ */

/* C[batch..., M, N] (dense, row-major, caller-allocated: the reference allocates the result with
 * enqueue_create_buffer, tenmo/kernels/matmul_kernel.mojo:223) = A[.., M, K] . B[.., K, N].
 * batch_shape is the broadcast result batch shape (rank <= 6); a_/b_batch_strides hold 0 where
 * that operand's dim is 1 or missing (tenmo/kernels/matmul_kernel.mojo:196-214,
 * tenmo/matmul_cpu.mojo:710-724).  Offsets ARE applied (CPU semantics, matmul_cpu.mojo:191,197).
 * accumulate: 0 -> C = A.B (reference semantics); 1 -> C += A.B (fused Gradbox accumulation,
 * tenmo/gradbox.mojo:1358-1364).
 * Replaces: matmul_2d_tiled + MatmulNdGpu.launch, tenmo/kernels/matmul_kernel.mojo:38-120,:128-283. */
int tenmo_hip_gemm_f32(const float* A, int64_t a_off, int64_t a_rs, int64_t a_cs,
                       const float* B, int64_t b_off, int64_t b_rs, int64_t b_cs,
                       float* C, int64_t M, int64_t N, int64_t K,
                       int32_t batch_rank, const int64_t* batch_shape,
                       const int64_t* a_batch_strides, const int64_t* b_batch_strides,
                       int32_t accumulate, int32_t sync);

/* The same product with the element-wise stages that follow it in a Linear layer done in the
 * GEMM store: C = A.B, then + bias[col] (N floats, or NULL), then max(., 0) if relu, then zeroed
 * where mask <= 0 (mask: dense like C, or NULL; with mask = the forward activation of the layer
 * below, dX = dY.W^T comes out already multiplied by the ReLU gradient).
 * Replaces: Matmul.forward followed by Adder.forward in Linear.forward (tenmo/net.mojo:193-201),
 * ReLU.forward and ReLUBackward (tenmo/relu.mojo:99-141, mask = x > 0 at :120-123). */
int tenmo_hip_gemm_epilogue_f32(const float* A, int64_t a_off, int64_t a_rs, int64_t a_cs,
                                const float* B, int64_t b_off, int64_t b_rs, int64_t b_cs,
                                float* C, int64_t M, int64_t N, int64_t K,
                                int32_t batch_rank, const int64_t* batch_shape,
                                const int64_t* a_batch_strides, const int64_t* b_batch_strides,
                                const float* bias, int32_t relu, const float* mask, int32_t sync);

/* out[batch..., m] = Mx[.., m, k] . v[.., k]
 * Replaces: matrix_vector_nd + MatrixVectorNdGpu.launch, tenmo/kernels/matrixvector_kernel.mojo:13-171
 * (which assumes dense inner dims; this entry point honours the strides and offset). */
int tenmo_hip_mv_f32(const float* Mx, int64_t m_off, int64_t m_rs, int64_t m_cs,
                     const float* v, int64_t v_off, int64_t v_s,
                     float* out, int64_t m, int64_t k,
                     int32_t batch_rank, const int64_t* batch_shape,
                     const int64_t* m_batch_strides, const int64_t* v_batch_strides,
                     int32_t accumulate, int32_t sync);

/* out[batch..., n] = v[.., k] . Mx[.., k, n]
 * Replaces: vector_matmul_nd + VectorMatmulNdGpu.launch, tenmo/kernels/vectormatrix_kernel.mojo:13-170. */
int tenmo_hip_vm_f32(const float* v, int64_t v_off, int64_t v_s,
                     const float* Mx, int64_t m_off, int64_t m_rs, int64_t m_cs,
                     float* out, int64_t k, int64_t n,
                     int32_t batch_rank, const int64_t* batch_shape,
                     const int64_t* v_batch_strides, const int64_t* m_batch_strides,
                     int32_t accumulate, int32_t sync);

/* tenmo_hip_vm_f32 for callers that cannot allocate device memory (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments, same kernels and
 * bit-identical results; the only difference is where the partial sums of the K slices live: a static device
 * array of TENMO_VM_NOALLOC_SCRATCH_BYTES that every GPU the library runs on holds until the process ends, instead
 * of the library's grow-only scratch.  The call allocates and frees nothing.  A product whose partial sums
 * (K slices x batches x n floats; the slice count follows the "cols_wg_per_cu" knob) exceed the array is refused with
 * TENMO_ERR_UNSUPPORTED and a message giving both sizes; with the default knob every shape fits.  Every call on a
 * GPU shares that GPU's array: calls that overlap in time on one GPU (two streams, two threads) race. */
#define TENMO_VM_NOALLOC_SCRATCH_BYTES (8u << 20)
int tenmo_hip_vm_f32_noalloc(const float* v, int64_t v_off, int64_t v_s,
                             const float* Mx, int64_t m_off, int64_t m_rs, int64_t m_cs,
                             float* out, int64_t k, int64_t n,
                             int32_t batch_rank, const int64_t* batch_shape,
                             const int64_t* v_batch_strides, const int64_t* m_batch_strides,
                             int32_t accumulate, int32_t sync);

/* out[c] (+)= sum over r < rows of G[g_off + r*g_rs + c], c < cols: the bias gradient of a Linear
 * layer, i.e. the upstream gradient summed over its broadcast (row) axis — what
 * sum_over_broadcasted_axes does for the bias operand of Adder (tenmo/broadcast.mojo:66-88,
 * tenmo/addition.mojo:73-112).  G is streamed once at HBM rate. */
int tenmo_hip_column_sum_f32(const float* G, int64_t g_off, int64_t g_rs, int64_t rows, int64_t cols,
                             float* out, int32_t accumulate, int32_t sync);

/* out[0] = sum_i a[i]*b[i]   (a stride of 0 broadcasts a one-element operand,
 * tenmo/dotproduct.mojo:67-74).  Replaces: DotproductKernel.launch,
 * tenmo/kernels/dotproduct_kernel.mojo:19-110. */
int tenmo_hip_dot_f32(const float* a, int64_t a_off, int64_t a_s,
                      const float* b, int64_t b_off, int64_t b_s,
                      int64_t n, float* out, int32_t sync);

/* ---- view-level entry points: the bodies of the reference's launch functions -------------- */

/* tenmo/matmul.mojo:258-272 */
int tenmo_hip_classify_matmul(int32_t rank_a, const int64_t* shape_a, int32_t rank_b, const int64_t* shape_b);

/* Shape of the result of op (TENMO_OP_MM / _MV / _VM) with the reference's validation
 * (tenmo/kernels/matmul_kernel.mojo:146-177, matrixvector.mojo:213-233, vectormatrix.mojo:218-238);
 * returns the element count (an empty batch product counts as 1 for MM), or a negative status. */
int64_t tenmo_hip_result_shape(int32_t op, const tenmo_view* A, const tenmo_view* B,
                               int64_t* out_shape, int32_t* out_rank);

/* MatmulNdGpu.launch(A, B, sync) — tenmo/kernels/matmul_kernel.mojo:128-283 — with the result
 * buffer supplied by the caller (dense, tenmo_hip_result_shape elements). */
int tenmo_hip_matmul_nd(const tenmo_view* A, const tenmo_view* B, float* C, int32_t sync);
/* Linear.forward on views: out = X.W + bias (bias: W.shape[-1] floats or NULL), then ReLU if
 * relu != 0, in one launch — tenmo/net.mojo:179-216 (+ tenmo/relu.mojo:99-141).  Shapes and
 * broadcasting as tenmo_hip_matmul_nd. */
int tenmo_hip_linear_nd(const tenmo_view* X, const tenmo_view* W, const float* bias, int32_t relu,
                        float* out, int32_t sync);
/* MatrixVectorNdGpu.launch — tenmo/kernels/matrixvector_kernel.mojo:80-171 */
int tenmo_hip_matrix_vector_nd(const tenmo_view* Mx, const tenmo_view* v, float* out, int32_t sync);
/* VectorMatmulNdGpu.launch — tenmo/kernels/vectormatrix_kernel.mojo:80-170 */
int tenmo_hip_vector_matmul_nd(const tenmo_view* v, const tenmo_view* Mx, float* out, int32_t sync);

/* Matmul2dBackward / MatmulNdBackward — tenmo/matmul.mojo:22-54, :99-137.
 * dC is the dense upstream gradient at the result shape.  For each non-NULL grad pointer the
 * gradient  dA = dC . B^T(view)  /  dB = A^T(view) . dC  is reduced over broadcast batch axes to
 * that parent's own shape (sum_over_broadcasted_axes, tenmo/sum_mean_reduction.mojo:185-211) and
 * ADDED into the dense buffer grad_A / grad_B (Ancestor.update_grad(AddTensor),
 * tenmo/ancestry.mojo:72-105).  Pass NULL for a parent that does not require grad (:34, :45). */
int tenmo_hip_matmul_backward(const tenmo_view* A, const tenmo_view* B, const float* dC,
                              float* grad_A, float* grad_B, int32_t sync);
/* Backward of Linear.forward — tenmo/net.mojo:193-201 is Matmul.forward followed by Adder.forward (bias broadcast over
 * the rows), so its backward is Adder's (tenmo/addition.mojo:73-112: the upstream gradient passes through to the product
 * and, summed over the broadcast axes, to the bias — sum_over_broadcasted_axes, tenmo/broadcast.mojo:66-88) followed by
 * tenmo_hip_matmul_backward.  dY: dense upstream gradient at the shape of X.W.  For each non-NULL pointer:
 * grad_X += dY . W^T(view), grad_W += X^T(view) . dY (summed over X's batch axes), grad_bias[c] += sum of dY over every
 * axis but the last.  dY is streamed twice, not three times: the launch that computes grad_W reads dY as its right operand
 * and adds up those fragments on the way (a dense row-major X and dY, one weight matrix; any other form, or grad_W == NULL,
 * takes one extra streaming pass over dY as tenmo_hip_column_sum_f32 does). */
int tenmo_hip_linear_backward(const tenmo_view* X, const tenmo_view* W, const float* dY,
                              float* grad_X, float* grad_W, float* grad_bias, int32_t sync);
/* MatrixVectorMulNdBackward — tenmo/matrixvector.mojo:19-201 (CPU-only in the reference):
 * grad_M += outer(dy, v), grad_v += M^T . dy, both dense at the parents' shapes. */
int tenmo_hip_mv_backward(const tenmo_view* Mx, const tenmo_view* v, const float* dy,
                          float* grad_M, float* grad_v, int32_t sync);
/* VectorMatmulNdBackward — tenmo/vectormatrix.mojo:18-206: grad_v += M . dy, grad_M += outer(v, dy). */
int tenmo_hip_vm_backward(const tenmo_view* v, const tenmo_view* Mx, const float* dy,
                          float* grad_v, float* grad_M, int32_t sync);

/* ---- adjacent operators of the training step ------------------------------------------------ */

/* CrossEntropyFusedKernel.launch — tenmo/kernels/crossentropy_fused_kernel.mojo:285-391 (CPU form:
 * tenmo/crossentropy.mojo:285-432): class-index cross-entropy of logits [M, C] (dense) against
 * target [M] (int64 when target_is_int64, else int32), with ignore_index and label smoothing.
 * Writes softmax_out [M, C] (may be NULL when no gradient is needed), per_sample_loss [M]
 * (0 for ignored rows), loss_sum [1] = their sum and valid_count [1] = rows not ignored — all
 * DEVICE pointers; the mean is loss_sum / valid_count as in crossentropy.mojo:1022-1024.
 * The sum is formed in a fixed order (the reference's kernel uses atomics). */
int tenmo_hip_cross_entropy_forward_f32(const float* logits, const void* target, int32_t target_is_int64,
                                        int64_t M, int64_t C, int64_t ignore_index, float label_smoothing,
                                        float* softmax_out, float* per_sample_loss, float* loss_sum,
                                        int32_t* valid_count, int32_t sync);
/* CrossEntropyFusedKernel.launch_backward — crossentropy_fused_kernel.mojo:192-275, :439-540:
 * grad[m,c] = (softmax[m,c] - (1-ls)*onehot[m,c] - ls/C) * [target[m] != ignore_index] * scale[m];
 * reduction 0 (none): scale = upstream[m]; 1 (sum): upstream[0]; 2 (mean): upstream[0] /
 * max(valid_count, 1).  upstream is a DEVICE pointer.  accumulate != 0 adds into grad_logits (the
 * Gradbox +=) instead of overwriting it. */
int tenmo_hip_cross_entropy_backward_f32(const float* softmax, const void* target, int32_t target_is_int64,
                                         const float* upstream, int64_t M, int64_t C, int64_t ignore_index,
                                         float label_smoothing, int32_t reduction, int32_t valid_count,
                                         float* grad_logits, int32_t accumulate, int32_t sync);
/* FusedIm2Col.forward — tenmo/cnn.mojo:308-507 (what Conv2dFused.invoke, :92-273, calls after it has
 * padded the image): out[n, co, y, x] = bias[co] + sum over (ci, ky, kx) of
 * padded_image[n, ci, y*stride + ky*dilation, x*stride + kx*dilation] * kernel[co, ci, ky, kx], with
 * H_out = (H_pad - (KH + (KH-1)(dilation-1))) / stride + 1 and W_out likewise (:358-365).  All tensors
 * dense: padded_image [N, C_in, H_pad, W_pad], kernel [C_out, C_in, KH, KW], bias [C_out] or NULL (the
 * reference substitutes zeros, :128-131), out [N, C_out, H_out, W_out].  Runs as an implicit GEMM on
 * the matrix-core kernel: the patch matrix is never materialised. */
int tenmo_hip_conv2d_forward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                                 const float* kernel, int64_t c_out, int64_t kh, int64_t kw, const float* bias,
                                 int64_t stride, int64_t dilation, float* out, int32_t sync);
/* FusedCol2ImBackward.backward — tenmo/cnn.mojo:546-948: the three gradients of the fused convolution
 * for the upstream gradient grad_out [N, C_out, H_out, W_out]; each output pointer may be NULL (that
 * parent does not require a gradient):
 *   grad_bias[co]               = sum over (n, y, x) of grad_out                      (:669-713)
 *   grad_kernel[co, ci, ky, kx] = sum over (n, y, x) of grad_out[n, co, y, x] *
 *                                 padded_image[n, ci, y*stride + ky*dilation, x*stride + kx*dilation]   (:716-815)
 *   grad_padded_image[n, ci, y*stride + ky*dilation, x*stride + kx*dilation] += kernel[co, ci, ky, kx] *
 *                                 grad_out[n, co, y, x]   over all (co, ky, kx, y, x)   (:818-948)
 * accumulate != 0 adds into the three outputs (the reference's update_grad(AddTensor), :607-650) instead
 * of overwriting them.  The gradient is with respect to the PADDED image, as in the reference (its Pad
 * operator's backward removes the border).  All three run on the matrix-core GEMM: the kernel gradient
 * with the patches gathered (no patch matrix), the image gradient as a stride-1 convolution of the
 * spread-out upstream gradient with the reversed kernel. */
int tenmo_hip_conv2d_backward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                                  const float* kernel, int64_t c_out, int64_t kh, int64_t kw, int64_t stride, int64_t dilation,
                                  const float* grad_out, float* grad_padded_image, float* grad_kernel, float* grad_bias,
                                  int32_t accumulate, int32_t sync);
/* SGDStep.launch_no_momentum / launch_momentum — tenmo/kernels/sgd_kernel.mojo:56-143 (CPU form:
 * tenmo/optim.mojo:93-160): g += weight_decay * p when weight_decay > 0; with velocity != NULL
 * v = momentum * v + g, p -= lr * v; else p -= lr * g. */
int tenmo_hip_sgd_step_f32(float* param, const float* grad, float* velocity, int64_t n,
                           float lr, float momentum, float weight_decay, int32_t sync);

/* ---- the reference's existing plugin ABI --------------------------------------------------- */

/* Exact CBLAS prototype the reference binds with
 *   get_function[CBLAS_SGEMM_FN]("cblas_sgemm")      tenmo/blashandle.mojo:136-151, :231, :655
 * HOST pointers: operands are staged to the GPU, multiplied there, and C is copied back before
 * the call returns, so `mojo -D BLAS_PATH=/path/libtenmo_hip.so` makes LinearBLAS /
 * SequentialBLAS / BLASMatmul2dBackward run on the GPU unchanged.  Row- and column-major,
 * all four transpose cases, alpha/beta honoured.  Initialises device 0 on first use. */
void cblas_sgemm(int order, int trans_a, int trans_b, int M, int N, int K, float alpha,
                 const float* A, int lda, const float* B, int ldb, float beta, float* C, int ldc);

/* ---- MLP training-step harness (callers of the path) -------------------------------------- */

/* Linear(x.W + b) -> ReLU -> ... -> Linear -> CrossEntropy(mean) -> backward -> SGD(lr), the step
 * of examples/mnist.mojo:150-162 over tenmo/net.mojo:179-216, relu.mojo:99-141,
 * crossentropy.mojo:285-432,:775-793, optim.mojo:93-120.  All GEMMs go through
 * the GEMM kernel with bias, ReLU and the ReLU gradient applied in its store; the remaining
 * element-wise stages are small kernels on the same stream.
 * dims[0..n_layers] are the layer widths; W[l] is [dims[l], dims[l+1]] row-major (the reference
 * stores weights [in, out], net.mojo:91-97), b[l] is [dims[l+1]]; both HOST arrays, copied in. */
typedef struct tenmo_mlp tenmo_mlp;
tenmo_mlp* tenmo_hip_mlp_create(int32_t n_layers, const int64_t* dims,
                                const float* const* W_host, const float* const* b_host, int64_t max_batch);
void tenmo_hip_mlp_destroy(tenmo_mlp*);
/* x: device [batch, dims[0]] dense; y: device int32 [batch].  The mean loss of this step is
 * written to loss_out[0] (device).  No host synchronisation unless sync != 0. */
int tenmo_hip_mlp_step(tenmo_mlp*, const float* x, const int32_t* y, int64_t batch, float lr,
                       float* loss_out, int32_t sync);
/* Same step, replayed from a HIP graph captured on first use (and re-captured when batch, lr or
 * loss_out change): one graph launch instead of ~25 kernel launches.  The reference explains its GPU
 * MNIST time by exactly this launch overhead ("13 kernels per step ... launch latency exceeds
 * compute", docs/from-bytes-to-gradients.md:454).  Inputs are copied into fixed staging buffers
 * first, so x and y may differ from call to call.  Needs the library's own stream. */
int tenmo_hip_mlp_step_graph(tenmo_mlp*, const float* x, const int32_t* y, int64_t batch, float lr,
                             float* loss_out, int32_t sync);
int tenmo_hip_mlp_forward(tenmo_mlp*, const float* x, int64_t batch, float* logits_out, int32_t sync);
/* copy a layer's parameters / last gradients to HOST arrays (synchronises) */
int tenmo_hip_mlp_get_params(tenmo_mlp*, int32_t layer, float* W_host, float* b_host);
int tenmo_hip_mlp_get_grads(tenmo_mlp*, int32_t layer, float* dW_host, float* db_host);

#ifdef __cplusplus
}
#endif
#endif /* TENMO_HIP_H */
