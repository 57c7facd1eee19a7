/* A plain C11 caller of libtenmo_hip.so: what a maintainer of the reference (or of any other host) binds.
 *
 *   gcc -std=c11 -Wall -Wextra -Werror -Iinclude -c tests/c_abi_driver.c          (the header is valid C; every prototype is used)
 *   gcc ... tests/c_abi_driver.c -Ltenmo_amd -ltenmo_hip -L/opt/rocm/lib -lamdhip64 -lm -o driver && ./driver
 *
 * It takes the address of every function include/tenmo_hip.h declares (a symbol that is declared but not exported fails
 * the link), then runs small products with exactly known results through the kernel-level and the view-level entry
 * points, the allocation-free one, the CBLAS prototype on host pointers, and one error path.  Device memory comes from
 * the HIP runtime's three C functions, declared here by hand so that this file needs no HIP header. */
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "tenmo_hip.h"

extern int hipMalloc(void** ptr, size_t bytes);
extern int hipFree(void* ptr);
extern int hipMemcpy(void* dst, const void* src, size_t bytes, int kind); /* 1 = host to device, 2 = device to host */

typedef void (*any_fn)(void);
static const any_fn every_symbol[] = {
    (any_fn)tenmo_hip_init, (any_fn)tenmo_hip_shutdown, (any_fn)tenmo_hip_sync, (any_fn)tenmo_hip_last_error, (any_fn)tenmo_hip_get_stream,
    (any_fn)tenmo_hip_set_stream, (any_fn)tenmo_hip_device_info, (any_fn)tenmo_hip_set_tuning, (any_fn)tenmo_hip_timer_begin,
    (any_fn)tenmo_hip_timer_end, (any_fn)tenmo_hip_clock_probe, (any_fn)tenmo_hip_gemm_f32, (any_fn)tenmo_hip_gemm_epilogue_f32,
    (any_fn)tenmo_hip_mv_f32, (any_fn)tenmo_hip_vm_f32, (any_fn)tenmo_hip_vm_f32_noalloc, (any_fn)tenmo_hip_column_sum_f32, (any_fn)tenmo_hip_dot_f32,
    (any_fn)tenmo_hip_classify_matmul, (any_fn)tenmo_hip_result_shape, (any_fn)tenmo_hip_matmul_nd, (any_fn)tenmo_hip_linear_nd,
    (any_fn)tenmo_hip_matrix_vector_nd, (any_fn)tenmo_hip_vector_matmul_nd, (any_fn)tenmo_hip_matmul_backward, (any_fn)tenmo_hip_linear_backward, (any_fn)tenmo_hip_mv_backward,
    (any_fn)tenmo_hip_vm_backward, (any_fn)tenmo_hip_cross_entropy_forward_f32, (any_fn)tenmo_hip_cross_entropy_backward_f32,
    (any_fn)tenmo_hip_conv2d_forward_f32, (any_fn)tenmo_hip_conv2d_backward_f32, (any_fn)tenmo_hip_sgd_step_f32, (any_fn)cblas_sgemm,
    (any_fn)tenmo_hip_mlp_create, (any_fn)tenmo_hip_mlp_destroy, (any_fn)tenmo_hip_mlp_step, (any_fn)tenmo_hip_mlp_step_graph,
    (any_fn)tenmo_hip_mlp_forward, (any_fn)tenmo_hip_mlp_get_params, (any_fn)tenmo_hip_mlp_get_grads,
};

static int failures = 0;

static void expect(int ok, const char* what) {
    if (!ok) {
        ++failures;
        fprintf(stderr, "FAILED: %s (last error: %s)\n", what, tenmo_hip_last_error());
    }
}

static float* to_device(const float* host, size_t n) {
    void* d = NULL;
    if (hipMalloc(&d, (n ? n : 1) * sizeof(float)) != 0) { fprintf(stderr, "hipMalloc failed\n"); exit(2); }
    if (n && host) hipMemcpy(d, host, n * sizeof(float), 1);
    return (float*)d;
}

static int same(const float* device, const float* want, size_t n, float tol) {
    float* got = (float*)malloc(n * sizeof(float));
    int ok = 1;
    hipMemcpy(got, device, n * sizeof(float), 2);
    for (size_t i = 0; i < n; ++i)
        if (!(fabsf(got[i] - want[i]) <= tol * (1.0f + fabsf(want[i])))) ok = 0;
    free(got);
    return ok;
}

int main(void) {
    enum { M = 5, K = 7, N = 3 };
    float A[M * K], B[K * N], C_want[M * N], Ct_want[M * N], y_want[M], z_want[N], x[K], w[M];
    /* small integers: every product below is exact in fp32 */
    for (int i = 0; i < M * K; ++i) A[i] = (float)((i * 7) % 11 - 5);
    for (int i = 0; i < K * N; ++i) B[i] = (float)((i * 5) % 9 - 4);
    for (int i = 0; i < K; ++i) x[i] = (float)(i % 4 - 1);
    for (int i = 0; i < M; ++i) w[i] = (float)(2 - i);
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            float s = 0.f;
            for (int k = 0; k < K; ++k) s += A[m * K + k] * B[k * N + n];
            C_want[m * N + n] = s;
            Ct_want[m * N + n] = 2.0f * s; /* accumulate onto itself */
        }
    for (int m = 0; m < M; ++m) { y_want[m] = 0.f; for (int k = 0; k < K; ++k) y_want[m] += A[m * K + k] * x[k]; }
    for (int n = 0; n < N; ++n) { z_want[n] = 0.f; for (int k = 0; k < K; ++k) z_want[n] += x[k] * B[k * N + n]; }

    expect(sizeof(every_symbol) / sizeof(every_symbol[0]) == 41, "one table entry per declared function");
    expect(tenmo_hip_sync() == TENMO_ERR_NOT_INITIALIZED, "calls before init are refused");
    if (tenmo_hip_init(0) != TENMO_OK) { fprintf(stderr, "tenmo_hip_init: %s\n", tenmo_hip_last_error()); return 2; }
    int cus = 0;
    char name[128];
    expect(tenmo_hip_device_info(&cus, name, (int)sizeof(name)) == TENMO_OK && cus > 0, "device_info");

    float *dA = to_device(A, M * K), *dB = to_device(B, K * N), *dC = to_device(NULL, M * N), *dx = to_device(x, K), *dw = to_device(w, M);
    float *dy = to_device(NULL, M), *dz = to_device(NULL, N), *dd = to_device(NULL, 1);

    /* C = A.B, then C += A.B */
    expect(tenmo_hip_gemm_f32(dA, 0, K, 1, dB, 0, N, 1, dC, M, N, K, 0, NULL, NULL, NULL, 0, 1) == TENMO_OK, "gemm");
    expect(same(dC, C_want, M * N, 0.f), "gemm result");
    expect(tenmo_hip_gemm_f32(dA, 0, K, 1, dB, 0, N, 1, dC, M, N, K, 0, NULL, NULL, NULL, 1, 1) == TENMO_OK, "gemm accumulate");
    expect(same(dC, Ct_want, M * N, 0.f), "gemm accumulate result");

    /* the same product through views: A as the transposed view of A^T's storage is exercised by the Python tests; here the plain views */
    tenmo_view va, vb;
    memset(&va, 0, sizeof(va));
    memset(&vb, 0, sizeof(vb));
    va.data = dA; va.rank = 2; va.shape[0] = M; va.shape[1] = K; va.strides[0] = K; va.strides[1] = 1;
    vb.data = dB; vb.rank = 2; vb.shape[0] = K; vb.shape[1] = N; vb.strides[0] = N; vb.strides[1] = 1;
    int64_t shape[TENMO_MAX_RANK];
    int32_t rank = 0;
    expect(tenmo_hip_result_shape(TENMO_OP_MM, &va, &vb, shape, &rank) == M * N && rank == 2 && shape[0] == M && shape[1] == N, "result_shape");
    expect(tenmo_hip_matmul_nd(&va, &vb, dC, 1) == TENMO_OK && same(dC, C_want, M * N, 0.f), "matmul_nd");

    /* the backward of y = A.B + bias from the upstream gradient dY = A.B: grad_A = dY.B^T, grad_B = A^T.dY, grad_bias = column sums of dY,
     * each added onto what the gradient buffers hold (zeros here) */
    {
        float gA_want[M * K], gB_want[K * N], gb_want[N], zeros[M * K + K * N + N];
        memset(zeros, 0, sizeof(zeros));
        for (int m = 0; m < M; ++m)
            for (int k = 0; k < K; ++k) { float s = 0.f; for (int n = 0; n < N; ++n) s += C_want[m * N + n] * B[k * N + n]; gA_want[m * K + k] = s; }
        for (int k = 0; k < K; ++k)
            for (int n = 0; n < N; ++n) { float s = 0.f; for (int m = 0; m < M; ++m) s += A[m * K + k] * C_want[m * N + n]; gB_want[k * N + n] = s; }
        for (int n = 0; n < N; ++n) { gb_want[n] = 0.f; for (int m = 0; m < M; ++m) gb_want[n] += C_want[m * N + n]; }
        float *gA = to_device(zeros, M * K), *gB = to_device(zeros, K * N), *gb = to_device(zeros, N), *dY = to_device(C_want, M * N);
        expect(tenmo_hip_linear_backward(&va, &vb, dY, gA, gB, gb, 1) == TENMO_OK, "linear_backward");
        expect(same(gA, gA_want, M * K, 0.f) && same(gB, gB_want, K * N, 0.f) && same(gb, gb_want, N, 0.f), "linear_backward gradients");
        hipFree(gA); hipFree(gB); hipFree(gb); hipFree(dY);
    }

    /* y = A.x, z = x.B (with and without allocation), d = x.x */
    expect(tenmo_hip_mv_f32(dA, 0, K, 1, dx, 0, 1, dy, M, K, 0, NULL, NULL, NULL, 0, 1) == TENMO_OK && same(dy, y_want, M, 0.f), "mv");
    expect(tenmo_hip_vm_f32(dx, 0, 1, dB, 0, N, 1, dz, K, N, 0, NULL, NULL, NULL, 0, 1) == TENMO_OK && same(dz, z_want, N, 0.f), "vm");
    expect(tenmo_hip_vm_f32_noalloc(dx, 0, 1, dB, 0, N, 1, dz, K, N, 0, NULL, NULL, NULL, 0, 1) == TENMO_OK && same(dz, z_want, N, 0.f), "vm without allocation");
    float xx = 0.f;
    for (int i = 0; i < K; ++i) xx += x[i] * x[i];
    expect(tenmo_hip_dot_f32(dx, 0, 1, dx, 0, 1, K, dd, 1) == TENMO_OK && same(dd, &xx, 1, 0.f), "dot");

    /* the reference's plugin prototype, host pointers: C = 1*A.B + 0*C, row-major, no transposes */
    float C_host[M * N];
    memset(C_host, 0, sizeof(C_host));
    cblas_sgemm(101, 111, 111, M, N, K, 1.0f, A, K, B, N, 0.0f, C_host, N);
    expect(memcmp(C_host, C_want, sizeof(C_host)) == 0, "cblas_sgemm");

    /* an error path: inner extents that do not match */
    vb.shape[0] = K + 1;
    expect(tenmo_hip_matmul_nd(&va, &vb, dC, 1) == TENMO_ERR_INVALID_SHAPE && strlen(tenmo_hip_last_error()) > 0, "shape error is reported");

    (void)dw;
    hipFree(dA); hipFree(dB); hipFree(dC); hipFree(dx); hipFree(dw); hipFree(dy); hipFree(dz); hipFree(dd);
    expect(tenmo_hip_shutdown() == TENMO_OK, "shutdown");
    if (failures == 0) printf("c_abi_driver: ok on %s (%d CUs)\n", name, cus);
    return failures != 0;
}
