// Small element-wise / reduction kernels around the matrix products: the reduction of a batched
// gradient to a broadcast parent's shape, outer-product gradients of mv/vm, and the stages of the
// MLP training-step harness (bias add + ReLU, cross-entropy forward/backward, bias gradient, SGD).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "gemm_mfma.hpp"

namespace tenmo {

// ---- shader-clock probe ---------------------------------------------------------------------------
// One wavefront per SIMD on every CU runs `n` rounds of four independent v_mfma_f32_32x32x2_f32 and nothing else.
// An MFMA of this kind occupies the matrix pipe for 16 passes of 4 cycles, so the launch takes 4 * n * 64 shader cycles
// (plus start-up): cycles / measured time is the clock the chip sustains under a full matrix-core load.
__global__ __launch_bounds__(256) void clock_probe_kernel(int n, float seed) {
    f32x16 a0, a1, a2, a3;
#pragma unroll
    for (int e = 0; e < 16; ++e) { a0[e] = 0.f; a1[e] = 0.f; a2[e] = 0.f; a3[e] = 0.f; }
    const float x = seed + (float)threadIdx.x, y = seed * 0.5f;
    for (int i = 0; i < n; ++i) {
        a0 = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, a0, 0, 0, 0);
        a1 = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, a1, 0, 0, 0);
        a2 = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, a2, 0, 0, 0);
        a3 = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, a3, 0, 0, 0);
    }
    keep_alive(a0, a1, a2, a3);
}

// ---- sum_over_broadcasted_axes (tenmo/sum_mean_reduction.mojo:185-211) fused with the
// Gradbox "+=" (tenmo/gradbox.mojo:1358-1364): dst[parent shape] += sum over the batch dims that
// the parent broadcast.  src is dense [batch_shape..., inner]; dst is dense at the parent's shape.
struct BroadcastReduceArgs {
    const float* src;
    float* dst;
    int64_t inner;           // elements of the trailing (non-batch) dims
    int64_t dst_batch;       // product of the parent's own batch dims
    int32_t rank;            // result batch rank
    int64_t shape[MAX_BATCH_RANK];     // result batch shape
    int64_t src_str[MAX_BATCH_RANK];   // dense strides of src batch dims (in units of `inner`)
    int32_t kept[MAX_BATCH_RANK];      // 1 where the parent has this dim with size > 1
    int64_t reduced_total;   // product of the reduced dims
};

__global__ void broadcast_reduce_add_kernel(const BroadcastReduceArgs g) {
    const int64_t total = g.dst_batch * g.inner;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t in = idx % g.inner;
        int64_t pb = idx / g.inner;
        // kept coordinates -> base offset in src
        int64_t base = 0;
        for (int d = g.rank - 1; d >= 0; --d) {
            if (g.kept[d]) { base += (pb % g.shape[d]) * g.src_str[d]; pb /= g.shape[d]; }
        }
        float acc = 0.f;
        for (int64_t r = 0; r < g.reduced_total; ++r) {
            int64_t rr = r, off = base;
            for (int d = g.rank - 1; d >= 0; --d) {
                if (!g.kept[d]) { off += (rr % g.shape[d]) * g.src_str[d]; rr /= g.shape[d]; }
            }
            acc += g.src[off * g.inner + in];
        }
        g.dst[idx] += acc;
    }
}

// The same with four consecutive inner elements per thread (inner % 4 == 0, both arrays 16-byte aligned) and the
// slices of four reduced batches in flight at a time; added in batch order, so the sum stays deterministic.
__global__ __launch_bounds__(256) void broadcast_reduce_add_vec_kernel(const BroadcastReduceArgs g) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    const int64_t inner4 = g.inner / 4, total4 = g.dst_batch * inner4;
    const f4* __restrict src4 = reinterpret_cast<const f4*>(g.src);
    f4* __restrict dst4 = reinterpret_cast<f4*>(g.dst);
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total4; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t in = idx % inner4;
        int64_t pb = idx / inner4;
        int64_t base = 0;
        for (int d = g.rank - 1; d >= 0; --d) {
            if (g.kept[d]) { base += (pb % g.shape[d]) * g.src_str[d]; pb /= g.shape[d]; }
        }
        auto slice = [&](int64_t r) {
            int64_t off = base;
            for (int d = g.rank - 1; d >= 0; --d) {
                if (!g.kept[d]) { off += (r % g.shape[d]) * g.src_str[d]; r /= g.shape[d]; }
            }
            return off * inner4 + in;
        };
        f4 acc = __builtin_nontemporal_load(dst4 + idx);
        for (int64_t r = 0; r < g.reduced_total; r += 4) {
            f4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = r + u < g.reduced_total ? __builtin_nontemporal_load(src4 + slice(r + u)) : f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int u = 0; u < 4; ++u) acc += v[u];
        }
        dst4[idx] = acc;
    }
}

// ---- outer-product gradients of mv / vm -------------------------------------------------------
// grad[b_parent][i][j] += sum over broadcast batches of  p[b][i] * q[b][j]
// (tenmo/matrixvector.mojo:87-139, tenmo/vectormatrix.mojo:145-201).  One thread per grad element;
// the loop over batches that map to the same parent element keeps the sum deterministic.
struct OuterArgs {
    const float* p; int64_t p_s;   // left factor, element stride; advanced by its offset
    const float* q; int64_t q_s;   // right factor
    float* grad;                   // dense [parent batch..., I, J]
    int64_t I, J;
    int64_t parent_batch;          // product of the parent's own batch dims
    int32_t rank;
    int64_t shape[MAX_BATCH_RANK];
    int64_t p_str[MAX_BATCH_RANK]; // batch strides of p, q (0 where broadcast)
    int64_t q_str[MAX_BATCH_RANK];
    int32_t kept[MAX_BATCH_RANK];  // 1 where the gradient's parent has this batch dim (> 1)
    int64_t reduced_total;
};

__global__ void outer_add_kernel(const OuterArgs g) {
    const int64_t total = g.parent_batch * g.I * g.J;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * blockDim.x) {
        const int64_t j = idx % g.J, i = (idx / g.J) % g.I;
        int64_t pb = idx / (g.J * g.I);
        int64_t pbase = 0, qbase = 0;
        for (int d = g.rank - 1; d >= 0; --d) {
            if (g.kept[d]) { const int64_t c = pb % g.shape[d]; pb /= g.shape[d]; pbase += c * g.p_str[d]; qbase += c * g.q_str[d]; }
        }
        float acc = 0.f;
        for (int64_t r = 0; r < g.reduced_total; ++r) {
            int64_t rr = r, po = pbase, qo = qbase;
            for (int d = g.rank - 1; d >= 0; --d) {
                if (!g.kept[d]) { const int64_t c = rr % g.shape[d]; rr /= g.shape[d]; po += c * g.p_str[d]; qo += c * g.q_str[d]; }
            }
            acc += g.p[po + i * g.p_s] * g.q[qo + j * g.q_s];
        }
        g.grad[idx] += acc;
    }
}

// The same with four consecutive j per thread (q_s == 1, J % 4 == 0, grad 16-byte aligned): 16-byte loads of q and of
// the gradient, four groups in flight, streaming stores — the update is a read-modify-write sweep over the gradient.
__global__ __launch_bounds__(256) void outer_add_vec_kernel(const OuterArgs g) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef float f4u __attribute__((ext_vector_type(4), aligned(4)));
    constexpr int U = 4;
    const int64_t J4 = g.J / 4, total4 = g.parent_batch * g.I * J4;
    f4* __restrict grad4 = reinterpret_cast<f4*>(g.grad);
    for (int64_t i0 = (int64_t)blockIdx.x * 256 * U + threadIdx.x; i0 < total4; i0 += (int64_t)gridDim.x * 256 * U) {
        f4 old[U], acc[U];
        bool ok[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int64_t idx = i0 + (int64_t)u * 256;
            ok[u] = idx < total4;
            acc[u] = f4{0.f, 0.f, 0.f, 0.f}; old[u] = acc[u];
            if (!ok[u]) continue;
            old[u] = __builtin_nontemporal_load(grad4 + idx);
            const int64_t j = 4 * (idx % J4), i = (idx / J4) % g.I;
            int64_t pb = idx / (J4 * g.I);
            int64_t pbase = 0, qbase = 0;
            for (int d = g.rank - 1; d >= 0; --d) {
                if (g.kept[d]) { const int64_t c = pb % g.shape[d]; pb /= g.shape[d]; pbase += c * g.p_str[d]; qbase += c * g.q_str[d]; }
            }
            for (int64_t r = 0; r < g.reduced_total; ++r) {
                int64_t rr = r, po = pbase, qo = qbase;
                for (int d = g.rank - 1; d >= 0; --d) {
                    if (!g.kept[d]) { const int64_t c = rr % g.shape[d]; rr /= g.shape[d]; po += c * g.p_str[d]; qo += c * g.q_str[d]; }
                }
                const f4 qv = *reinterpret_cast<const f4u*>(g.q + qo + j);
                acc[u] += g.p[po + i * g.p_s] * qv;
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (ok[u]) __builtin_nontemporal_store(old[u] + acc[u], grad4 + (i0 + (int64_t)u * 256));
    }
}

__global__ void fill_kernel(float* p, int64_t n, float value) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = value;
}

// ---- MLP harness stages -----------------------------------------------------------------------
// Fused class-index cross-entropy, mean reduction (tenmo/crossentropy.mojo:285-432) and its
// gradient (softmax - onehot) / valid_count (:775-793, :451-481).  One thread per row (C is tiny in
// the harness); per-row losses go to row_loss for the ordered sum.  When the whole batch fits one
// workgroup (gridDim.x == 1) and loss_out / db_out are given, the same launch also finishes the
// ordered mean and the bias gradient of the last layer (column sums of dz, rows ascending).
__global__ void cross_entropy_kernel(const float* __restrict logits, const int32_t* __restrict y, int64_t rows, int64_t C,
                                     float* __restrict dz, float* __restrict row_loss, float* __restrict loss_out, float* __restrict db_out) {
    const int64_t r = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r < rows) {
        const float* x = logits + r * C;
        float mx = -3.402823466e+38f;
        for (int64_t c = 0; c < C; ++c) mx = fmaxf(mx, x[c]);
        float sum_exp = 0.f;
        for (int64_t c = 0; c < C; ++c) sum_exp += expf(x[c] - mx);
        const float lse = logf(fmaxf(sum_exp, 1e-7f));
        const int32_t t = y[r];
        // a label outside [0, C) (the reference rejects it on the host, crossentropy.mojo:116-123) must
        // not turn into an out-of-bounds read: its loss is NaN, its row gets no one-hot term
        row_loss[r] = (t >= 0 && t < C) ? -(x[t] - mx - lse) : __builtin_nanf("");
        const float inv = 1.f / sum_exp, scale = 1.f / (float)rows;
        for (int64_t c = 0; c < C; ++c) dz[r * C + c] = (expf(x[c] - mx) * inv - (c == t ? 1.f : 0.f)) * scale;
    }
    if (gridDim.x == 1 && (loss_out || db_out)) {
        __syncthreads(); // this workgroup wrote every row
        if (loss_out && threadIdx.x == 0) {
            float s = 0.f;
            for (int64_t q = 0; q < rows; ++q) s += row_loss[q];
            *loss_out = s / (float)rows;
        }
        if (db_out) {
            for (int64_t c = threadIdx.x; c < C; c += blockDim.x) {
                float s = 0.f;
                for (int64_t q = 0; q < rows; ++q) s += dz[q * C + c];
                db_out[c] = s;
            }
        }
    }
}

// ---- the small end of an MLP training step in ONE launch ------------------------------------------------------------
// For a network whose last two Linear layers are small (the MNIST example's 128 -> 32 -> 10 at batch 64,
// examples/mnist.mojo:150-162): both layers forward (bias, ReLU between them), the class-index cross-entropy (mean) with
// its gradient, both layers backward (weight and bias gradients, ReLU masks), the gradient handed to the layer below with
// that layer's ReLU mask and bias gradient, and the SGD update of both layers — by one workgroup with every operand in
// LDS.  Run op by op these are eight dependent launches of a few microseconds each, which is what such a step costs; the
// reference names the same cause for its GPU time (docs/from-bytes-to-gradients.md:454).
constexpr int MLP_TAIL_THREADS = 256;
constexpr int MLP_TAIL_MAX_B = 64, MLP_TAIL_MAX_D0 = 128, MLP_TAIL_MAX_D1 = 64, MLP_TAIL_MAX_C = 32;
struct MlpTailArgs {
    const float* h0;      // [B, D0] output of the layer below (after its ReLU)
    const int32_t* y;     // [B]
    float *W1, *b1;       // [D0, D1], [D1]: updated in place
    float *W2, *b2;       // [D1, C], [C]
    float *dW1, *db1, *dW2, *db2;
    float *h1, *logits;   // [B, D1], [B, C]: the two layers' outputs, kept as the op-by-op path keeps them
    float* g0;            // [B, D0]: gradient for the layer below, already multiplied by its ReLU gradient (h0 > 0)
    float* db0;           // [D0]: that layer's bias gradient (column sums of g0)
    float* row_loss;      // [B]
    float* loss_out;      // [1]
    float lr;
    int32_t B, D0, D1, C;
};

// C[M][N] = A[M][K] . B[K][N] on LDS operands with arbitrary element strides; every thread of the workgroup takes blocks of 2
// rows x 4 columns (the columns a quarter of the width apart, so that neighbouring lanes read neighbouring columns); rows and
// columns beyond the extents are clamped for the loads and skipped by `emit(m, n, value)`.
template <class Emit>
__device__ __forceinline__ void lds_product(int M, int N, int K, const float* A, int a_rs, int a_cs, const float* B, int b_rs, int b_cs, Emit&& emit) {
    const int nq = (N + 3) / 4, mh = (M + 1) / 2;
    for (int blk = threadIdx.x; blk < mh * nq; blk += MLP_TAIL_THREADS) {
        const int m0 = (blk / nq) * 2, q = blk % nq;
        const int m1 = min(m0 + 1, M - 1);
        int n[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) n[j] = min(q + j * nq, N - 1);
        float acc[2][4] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
        for (int k = 0; k < K; ++k) {
            const float a0 = A[m0 * a_rs + k * a_cs], a1 = A[m1 * a_rs + k * a_cs];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float b = B[k * b_rs + n[j] * b_cs];
                acc[0][j] += a0 * b;
                acc[1][j] += a1 * b;
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (q + j * nq >= N) continue;
            emit(m0, n[j], acc[0][j]);
            if (m0 + 1 < M) emit(m0 + 1, n[j], acc[1][j]);
        }
    }
}

// The same product on the matrix cores: the 32x32 blocks of C are dealt to the workgroup's four wavefronts (v_mfma_f32_32x32x2,
// operands read from LDS one element per lane and MFMA: 2 LDS reads per 2048 multiply-adds, where the vector form above
// needs 1536 and is bound by the LDS).  With fewer blocks than wavefronts K is cut among 4 / blocks wavefronts per block and
// the partial blocks are added through `scratch` (MLP_TAIL_THREADS * 16 floats) in a fixed order.  Every thread of the
// workgroup must call it (it synchronises when it cuts K).
template <class Emit>
__device__ __forceinline__ void lds_product_mfma(int M, int N, int K, const float* A, int a_rs, int a_cs, const float* B, int b_rs, int b_cs, float* scratch,
                                                 Emit&& emit) {
    constexpr int WAVES = MLP_TAIL_THREADS / 64;
    const int t = threadIdx.x, wave = t >> 6, lane = t & 63, half = lane >> 5, i = lane & 31;
    const int bn = (N + 31) / 32, nblk = ((M + 31) / 32) * bn;
    const int ks = nblk >= WAVES ? 1 : WAVES / nblk;          // wavefronts per block
    const int kpart = ((K + ks - 1) / ks + 1) & ~1;           // k per part, even (an MFMA takes two)
    for (int u = wave; u < nblk * ks; u += WAVES) {
        const int blk = u / ks, part = u - blk * ks;
        const int m0 = (blk / bn) * 32, n0 = (blk % bn) * 32;
        const int kb = part * kpart, ke = min(K, kb + kpart);
        const int m = min(m0 + i, M - 1), n = min(n0 + i, N - 1); // clamped: computed, never emitted
        f32x16 acc;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] = 0.f;
        for (int k = kb; k < ke; k += 2) {
            const int kk = k + half;
            const bool ok = kk < ke;
            const float av = ok ? A[m * a_rs + kk * a_cs] : 0.f;
            const float bv = ok ? B[kk * b_rs + n * b_cs] : 0.f;
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc, 0, 0, 0);
        }
        if (ks == 1) {
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int r = m0 + 8 * (e >> 2) + 4 * half + (e & 3), c = n0 + i;
                if (r < M && c < N) emit(r, c, acc[e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e) scratch[u * 1024 + e * 64 + lane] = acc[e]; // (u < WAVES here)
        }
    }
    if (ks > 1) {
        __syncthreads();
        for (int idx = t; idx < nblk * 1024; idx += MLP_TAIL_THREADS) {
            const int blk = idx >> 10, el = idx & 1023, e = el >> 6, l = el & 63;
            float sum = 0.f;
            for (int part = 0; part < ks; ++part) sum += scratch[(blk * ks + part) * 1024 + el];
            const int r = (blk / bn) * 32 + 8 * (e >> 2) + 4 * (l >> 5) + (e & 3), c = (blk % bn) * 32 + (l & 31);
            if (r < M && c < N) emit(r, c, sum);
        }
        __syncthreads(); // the scratch is free again
    }
}

__global__ __launch_bounds__(MLP_TAIL_THREADS) void mlp_tail_kernel(const MlpTailArgs a) {
    // odd pitches: a column walk never stays on one LDS bank
    constexpr int P0 = MLP_TAIL_MAX_D0 + 1, P1 = MLP_TAIL_MAX_D1 + 1, PC = MLP_TAIL_MAX_C + 1;
    __shared__ float h0[MLP_TAIL_MAX_B * P0];   // [B][D0]; becomes g0 at the end
    __shared__ float w1[MLP_TAIL_MAX_D0 * P1];  // [D0][D1]
    __shared__ float h1[MLP_TAIL_MAX_B * P1];   // [B][D1]
    __shared__ float g1[MLP_TAIL_MAX_B * P1];   // [B][D1]
    __shared__ float w2[MLP_TAIL_MAX_D1 * PC];  // [D1][C]
    __shared__ float z[MLP_TAIL_MAX_B * PC];    // [B][C]: logits, then their gradient
    __shared__ float bias1[MLP_TAIL_MAX_D1], bias2[MLP_TAIL_MAX_C];
    __shared__ float scratch[MLP_TAIL_THREADS * 16]; // partial blocks of the products that cut K among the wavefronts
    const int B = a.B, D0 = a.D0, D1 = a.D1, C = a.C, t = threadIdx.x;
    for (int i = t; i < B * D0; i += MLP_TAIL_THREADS) h0[(i / D0) * P0 + i % D0] = a.h0[i];
    for (int i = t; i < D0 * D1; i += MLP_TAIL_THREADS) w1[(i / D1) * P1 + i % D1] = a.W1[i];
    for (int i = t; i < D1 * C; i += MLP_TAIL_THREADS) w2[(i / C) * PC + i % C] = a.W2[i];
    for (int i = t; i < D1; i += MLP_TAIL_THREADS) bias1[i] = a.b1[i];
    for (int i = t; i < C; i += MLP_TAIL_THREADS) bias2[i] = a.b2[i];
    __syncthreads();
    // forward: h1 = relu(h0 . W1 + b1), logits = h1 . W2 + b2      (tenmo/net.mojo:193-201, tenmo/relu.mojo:99-118)
    lds_product_mfma(B, D1, D0, h0, P0, 1, w1, P1, 1, scratch, [&](int m, int n, float v) {
        v += bias1[n];
        v = v > 0.f ? v : 0.f;
        h1[m * P1 + n] = v;
        a.h1[m * D1 + n] = v;
    });
    __syncthreads();
    lds_product_mfma(B, C, D1, h1, P1, 1, w2, PC, 1, scratch, [&](int m, int n, float v) {
        v += bias2[n];
        z[m * PC + n] = v;
        a.logits[m * C + n] = v;
    });
    __syncthreads();
    // cross-entropy, mean over the batch, and its gradient (tenmo/crossentropy.mojo:285-432, :775-793): one thread per row
    if (t < B) {
        float* x = z + t * PC;
        float mx = -3.402823466e+38f;
        for (int c = 0; c < C; ++c) mx = fmaxf(mx, x[c]);
        float sum_exp = 0.f;
        for (int c = 0; c < C; ++c) sum_exp += expf(x[c] - mx);
        const float lse = logf(fmaxf(sum_exp, 1e-7f));
        const int32_t label = a.y[t];
        a.row_loss[t] = (label >= 0 && label < C) ? -(x[label] - mx - lse) : __builtin_nanf("");
        const float inv = 1.f / sum_exp, scale = 1.f / (float)B;
        for (int c = 0; c < C; ++c) x[c] = (expf(x[c] - mx) * inv - (c == label ? 1.f : 0.f)) * scale;
    }
    __syncthreads();
    if (t == 0) { // the reference's scalar loop order
        float s = 0.f;
        for (int r = 0; r < B; ++r) s += a.row_loss[r];
        *a.loss_out = s / (float)B;
    }
    if (t < C) { // db2 = column sums of the logits' gradient, rows ascending (tenmo/broadcast.mojo:81-87)
        float s = 0.f;
        for (int r = 0; r < B; ++r) s += z[r * PC + t];
        a.db2[t] = s;
        a.b2[t] = bias2[t] - a.lr * s;
    }
    // dW2 = h1^T . dz, g1 = (dz . W2^T) masked by h1 > 0      (tenmo/matmul.mojo:36-48, tenmo/relu.mojo:120-123)
    lds_product_mfma(D1, C, B, h1, 1, P1, z, PC, 1, scratch, [&](int m, int n, float v) {
        a.dW2[m * C + n] = v;
        a.W2[m * C + n] = w2[m * PC + n] - a.lr * v;
    });
    lds_product_mfma(B, D1, C, z, PC, 1, w2, 1, PC, scratch, [&](int m, int n, float v) { g1[m * P1 + n] = h1[m * P1 + n] > 0.f ? v : 0.f; });
    __syncthreads();
    if (t < D1) {
        float s = 0.f;
        for (int r = 0; r < B; ++r) s += g1[r * P1 + t];
        a.db1[t] = s;
        a.b1[t] = bias1[t] - a.lr * s;
    }
    // dW1 = h0^T . g1 (with the update of W1 in global memory; the LDS copy keeps the old weights for g0)
    lds_product_mfma(D0, D1, B, h0, 1, P0, g1, P1, 1, scratch, [&](int m, int n, float v) {
        a.dW1[m * D1 + n] = v;
        a.W1[m * D1 + n] = w1[m * P1 + n] - a.lr * v;
    });
    __syncthreads(); // h0 is overwritten below
    // g0 = (g1 . W1^T) masked by h0 > 0, in place of h0
    lds_product_mfma(B, D0, D1, g1, P1, 1, w1, 1, P1, scratch, [&](int m, int n, float v) {
        v = h0[m * P0 + n] > 0.f ? v : 0.f;
        h0[m * P0 + n] = v;
        a.g0[m * D0 + n] = v;
    });
    __syncthreads();
    if (t < D0) {
        float s = 0.f;
        for (int r = 0; r < B; ++r) s += h0[r * P0 + t];
        a.db0[t] = s;
    }
}

// The weight gradient of the network's first layer and that layer's SGD update in one launch, for the small batches of
// the launch above: dW = x^T . g (tenmo/matmul.mojo:46-48), W -= lr * dW, b -= lr * db (tenmo/optim.mojo:93-120).  A
// workgroup takes MLP_FIRST_ROWS input features (rows of W) and all O <= MLP_TAIL_MAX_D0 outputs: the gradient g [B, O] and
// the workgroup's columns of x lie in LDS, every thread sums one 2 x 4 block over the batch in ascending order.
constexpr int MLP_FIRST_ROWS = 16;
struct MlpFirstArgs {
    const float* x;   // [B, I] network input
    const float* g;   // [B, O] gradient of the layer's output (its ReLU gradient applied)
    const float* db;  // [O] column sums of g
    float *W, *b;     // [I, O], [O]: updated in place
    float* dW;        // [I, O]
    float lr;
    int32_t B, I, O;
};
__global__ __launch_bounds__(MLP_TAIL_THREADS) void mlp_first_layer_kernel(const MlpFirstArgs a) {
    constexpr int PX = MLP_TAIL_MAX_B + 1; // x strip held feature-major with an odd pitch
    __shared__ float gs[MLP_TAIL_MAX_B * MLP_TAIL_MAX_D0]; // [B][O], pitch O
    __shared__ float xs[MLP_FIRST_ROWS * PX];              // [row][B]
    const int B = a.B, I = a.I, O = a.O, t = threadIdx.x;
    const int k0 = blockIdx.x * MLP_FIRST_ROWS, rows = min(MLP_FIRST_ROWS, I - k0);
    for (int i = t; i < B * O; i += MLP_TAIL_THREADS) gs[i] = a.g[i];
    for (int i = t; i < B * MLP_FIRST_ROWS; i += MLP_TAIL_THREADS) {
        const int bb = i / MLP_FIRST_ROWS, r = i % MLP_FIRST_ROWS;
        xs[r * PX + bb] = r < rows ? a.x[(int64_t)bb * I + k0 + r] : 0.f;
    }
    __syncthreads();
    lds_product(rows, O, B, xs, PX, 1, gs, O, 1, [&](int m, int n, float v) {
        const int64_t at = (int64_t)(k0 + m) * O + n;
        a.dW[at] = v;
        a.W[at] = a.W[at] - a.lr * v;
    });
    if (blockIdx.x == 0)
        for (int i = t; i < O; i += MLP_TAIL_THREADS) a.b[i] = a.b[i] - a.lr * a.db[i];
}

// The first layer's forward for a small batch in ONE launch: h = relu(x . W + b) (tenmo/net.mojo:193-201) for a batch of a
// few dozen rows against a long input (784).  The ordinary path cuts such a product into K slices over many workgroups and
// adds them in a second launch; here a workgroup of 16 wavefronts owns one 32x32 block of h and cuts K among its OWN
// wavefronts — wavefront w takes the 8-wide k chunks w, w + 16, ... with operands straight from global memory (x: one
// 16-byte read per lane and chunk, W: four dword reads of 128 contiguous bytes per half wavefront) — and the 16 partial
// blocks are added through LDS in wavefront order, so the result does not depend on scheduling.
constexpr int MLP_FWD_THREADS = 1024, MLP_FWD_WAVES = MLP_FWD_THREADS / 64;
struct MlpFwdArgs {
    const float* x;  // [B, I]
    const float* W;  // [I, O]
    const float* b;  // [O]
    float* h;        // [B, O]
    int32_t B, I, O, relu;
};
__global__ __launch_bounds__(MLP_FWD_THREADS) void mlp_first_forward_kernel(const MlpFwdArgs a) {
    __shared__ float part[MLP_FWD_WAVES][16 * 64];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6, half = lane >> 5, i = lane & 31;
    const int I = a.I, O = a.O;
    const int row = min((int)blockIdx.y * 32 + i, a.B - 1), col = min((int)blockIdx.x * 32 + i, O - 1); // clamped: loaded, never stored
    const float* __restrict xr = a.x + (int64_t)row * I;
    const float* __restrict wc = a.W + col;
    f32x16 acc;
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[e] = 0.f;
    const int chunks = (I + 7) / 8;
    constexpr int U = 4; // chunks in flight per wavefront
    for (int c0 = wave; c0 < chunks; c0 += U * MLP_FWD_WAVES) {
        float fa[U][4], fb[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = 8 * (c0 + u * MLP_FWD_WAVES) + 4 * half; // this lane's four k of the chunk (MFMA steps 0..3)
            if (k + 3 < I) {
                const f32x4 v = *reinterpret_cast<const f32x4_u*>(xr + k);
                fa[u][0] = v.x; fa[u][1] = v.y; fa[u][2] = v.z; fa[u][3] = v.w;
#pragma unroll
                for (int s = 0; s < 4; ++s) fb[u][s] = wc[(int64_t)(k + s) * O];
            } else {
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    const bool ok = k + s < I;
                    fa[u][s] = ok ? xr[k + s] : 0.f;
                    fb[u][s] = ok ? wc[(int64_t)(k + s) * O] : 0.f;
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[u][s], fb[u][s], acc, 0, 0, 0);
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) part[wave][e * 64 + lane] = acc[e];
    __syncthreads();
    // thread t adds element (e, l) = (t / 64, t % 64) of the 16 partial blocks: block row 8(e>>2) + 4(l>>5) + (e&3), column l & 31
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < MLP_FWD_WAVES; ++w) sum += part[w][t];
    const int e = t >> 6;
    const int r = (int)blockIdx.y * 32 + 8 * (e >> 2) + 4 * half + (e & 3), c = (int)blockIdx.x * 32 + i;
    if (r < a.B && c < O) {
        sum += a.b[c];
        a.h[(int64_t)r * O + c] = a.relu && !(sum > 0.f) ? 0.f : sum;
    }
}

// loss = (sum of row losses in row order) / rows — the order of the reference's scalar loop
__global__ void ordered_mean_kernel(const float* __restrict row_loss, int64_t rows, float* __restrict out) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        float s = 0.f;
        for (int64_t r = 0; r < rows; ++r) s += row_loss[r];
        *out = s / (float)rows;
    }
}

// db[c] = sum_r g[r][c], rows ascending (tenmo/broadcast.mojo:81-87)
__global__ void column_sum_kernel(const float* __restrict g, int64_t rows, int64_t cols, float* __restrict db) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    float s = 0.f;
    for (int64_t r = 0; r < rows; ++r) s += g[r * cols + c];
    db[c] = s;
}

// p -= lr * g   (tenmo/optim.mojo:93-120, no momentum, no weight decay) for up to SGD_MAX_TENSORS
// parameter tensors in one launch (blockIdx.y = tensor)
constexpr int SGD_MAX_TENSORS = 16;
struct SgdArgs {
    float* p[SGD_MAX_TENSORS];
    const float* g[SGD_MAX_TENSORS];
    int64_t n[SGD_MAX_TENSORS];
    int32_t count;
};
__global__ void sgd_multi_kernel(const SgdArgs a, float lr) {
    const int k = blockIdx.y;
    float* __restrict p = a.p[k];
    const float* __restrict g = a.g[k];
    const int64_t n = a.n[k];
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) p[i] = p[i] - lr * g[i];
}

// One optimiser step on one tensor, with the options of the reference's two SGD kernels
// (tenmo/kernels/sgd_kernel.mojo:8-26 without, :29-53 with momentum): g += wd * p when wd > 0;
// with a velocity buffer v = momentum * v + g and p -= lr * v, else p -= lr * g.
__device__ __forceinline__ void sgd_update(float& p, float g, float* v, float lr, float momentum, float weight_decay) {
    if (weight_decay > 0.f) g += p * weight_decay;
    if (v) {
        *v = momentum * *v + g;
        p = p - lr * *v;
    } else {
        p = p - lr * g;
    }
}
// VEC: all three arrays start on 16-byte boundaries; the tail of n % 4 elements is done by thread 0
template <bool VEC>
__global__ void sgd_step_kernel(float* __restrict p, const float* __restrict g, float* __restrict vel, int64_t n, float lr, float momentum, float weight_decay) {
    const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x, stride = (int64_t)gridDim.x * blockDim.x;
    if constexpr (VEC) {
        typedef float f4 __attribute__((ext_vector_type(4)));
        f4* __restrict p4 = reinterpret_cast<f4*>(p);
        const f4* __restrict g4 = reinterpret_cast<const f4*>(g);
        f4* __restrict v4 = reinterpret_cast<f4*>(vel);
        constexpr int U = 4; // groups in flight per thread
        const int64_t n4 = n / 4;
        for (int64_t i0 = (int64_t)blockIdx.x * blockDim.x * U + threadIdx.x; i0 < n4; i0 += stride * U) {
            f4 pp[U], gg[U], vv[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t i = i0 + (int64_t)u * blockDim.x;
                pp[u] = f4{0.f, 0.f, 0.f, 0.f}; gg[u] = pp[u]; vv[u] = pp[u];
                if (i < n4) {
                    pp[u] = __builtin_nontemporal_load(p4 + i);
                    gg[u] = __builtin_nontemporal_load(g4 + i);
                    if (vel) vv[u] = __builtin_nontemporal_load(v4 + i);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int64_t i = i0 + (int64_t)u * blockDim.x;
                if (i >= n4) continue;
                float pa[4] = {pp[u].x, pp[u].y, pp[u].z, pp[u].w};
                const float ga[4] = {gg[u].x, gg[u].y, gg[u].z, gg[u].w};
                if (vel) {
                    float va[4] = {vv[u].x, vv[u].y, vv[u].z, vv[u].w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) sgd_update(pa[e], ga[e], &va[e], lr, momentum, weight_decay);
                    __builtin_nontemporal_store(f4{va[0], va[1], va[2], va[3]}, v4 + i);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) sgd_update(pa[e], ga[e], nullptr, lr, momentum, weight_decay);
                }
                __builtin_nontemporal_store(f4{pa[0], pa[1], pa[2], pa[3]}, p4 + i);
            }
        }
        if (tid == 0)
            for (int64_t i = n / 4 * 4; i < n; ++i) sgd_update(p[i], g[i], vel ? vel + i : nullptr, lr, momentum, weight_decay);
    } else {
        for (int64_t i = tid; i < n; i += stride) sgd_update(p[i], g[i], vel ? vel + i : nullptr, lr, momentum, weight_decay);
    }
}

// Sums the k_splits partial results into C (plain or accumulating), slices in a fixed order, then
// applies the fused epilogue.  One thread per output; eight slice loads in flight per thread.
// (extra_*: a second, small set of slices added the same way onto extra_out — the column sums of B that a launch with
// GemmArgs::bsum leaves per K slice; extra_n = 0 without)
__global__ void splitk_reduce_kernel(const float* __restrict partial, float* __restrict C, int64_t n, int splits, int accumulate,
                                     const float* __restrict bias, const float* __restrict mask, int relu, int64_t N,
                                     const float* __restrict extra_partial = nullptr, float* __restrict extra_out = nullptr, int64_t extra_n = 0) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (int64_t j = i; j < extra_n; j += stride) {
        float s = extra_out[j];
        for (int p = 0; p < splits; ++p) s += extra_partial[(int64_t)p * extra_n + j];
        extra_out[j] = s;
    }
    for (; i < n; i += stride) {
        float s = accumulate ? C[i] : 0.f;
        int p = 0;
        for (; p + 8 <= splits; p += 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = partial[(int64_t)(p + u) * n + i];
#pragma unroll
            for (int u = 0; u < 8; ++u) s += v[u];
        }
        for (; p < splits; ++p) s += partial[(int64_t)p * n + i];
        if (bias || mask || relu) s = epilogue_value(s, bias, mask, relu, i, i % N);
        C[i] = s;
    }
}

// Offset tables of the implicit im2col (tenmo/cnn.mojo:308-507 walks the same indices in loops):
// patch element k = (ci, ky, kx) of output position p = (y, x) of one padded image [C_in, H_pad, W_pad]
// lies at by_k[k] + by_pos[p] with
//   by_k[k]   = ci*H_pad*W_pad + ky*dilation*W_pad + kx*dilation,   by_pos[p] = y*stride*W_pad + x*stride.
struct ConvGeometry {
    int32_t c_in, h_pad, w_pad, kh, kw, h_out, w_out, stride, dilation;
};
__global__ void conv_tables_kernel(const ConvGeometry c, int32_t* __restrict by_k, int32_t* __restrict by_pos) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    const int nk = c.c_in * c.kh * c.kw, np = c.h_out * c.w_out;
    if (i < nk) {
        const int ci = i / (c.kh * c.kw), r = i % (c.kh * c.kw), ky = r / c.kw, kx = r % c.kw;
        by_k[i] = ci * c.h_pad * c.w_pad + ky * c.dilation * c.w_pad + kx * c.dilation;
    }
    if (i < np) {
        const int y = i / c.w_out, x = i % c.w_out;
        by_pos[i] = y * c.stride * c.w_pad + x * c.stride;
    }
}

// Upstream gradient [planes, h_out, w_out] spread out for the input-gradient convolution: element (y, x) goes
// to (off_y + y*stride, off_x + x*stride) of a zero-filled [planes, h_dst, w_dst] array.  A workgroup per plane
// (grid-stride over the planes), 32-bit index arithmetic inside it: with one flat 64-bit index the three
// divisions per element made the kernel arithmetic-bound (65 us for 170 MB of traffic).
__global__ void conv_dilate_pad_kernel(const float* __restrict src, float* __restrict dst, int64_t planes, int h_out, int w_out,
                                       int h_dst, int w_dst, int stride, int off_y, int off_x) {
    const int per_plane = h_dst * w_dst;
    for (int64_t plane = blockIdx.x; plane < planes; plane += gridDim.x) {
        const float* __restrict s = src + plane * h_out * w_out;
        float* __restrict d = dst + plane * per_plane;
        for (int i = threadIdx.x; i < per_plane; i += blockDim.x) {
            const int yy = i / w_dst, xx = i - yy * w_dst;
            const int ry = yy - off_y, rx = xx - off_x;
            float v = 0.f;
            if (ry >= 0 && rx >= 0) {
                const int y = ry / stride, x = rx / stride;
                if (y * stride == ry && x * stride == rx && y < h_out && x < w_out) v = s[y * w_out + x];
            }
            d[i] = v;
        }
    }
}

// kernel [c_out, c_in, kh, kw] -> [c_in, c_out, th, tw]: channel axes swapped, and of each spatial axis the taps
// last, last - step, last - 2*step, ... (th / tw of them).  th = kh, tw = kw, last = kh-1 / kw-1, step = 1 is the
// whole kernel with both spatial axes reversed.
__global__ void conv_flip_taps_kernel(const float* __restrict src, float* __restrict dst, int c_out, int c_in, int kh, int kw,
                                      int th, int tw, int last_y, int last_x, int step) {
    const int total = c_out * c_in * th * tw;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int tx = i % tw, ty = (i / tw) % th, co = (i / (tw * th)) % c_out, ci = i / (tw * th * c_out);
    dst[i] = src[((co * c_in + ci) * kh + (last_y - ty * step)) * kw + (last_x - tx * step)];
}

// dst[plane, py + stride*i, px + stride*j] (+)= src[plane, i, j] for i < hs, j < ws: one phase of a strided image
// gradient put in place.  src == nullptr writes zeros (a phase no kernel tap reaches).  A workgroup per plane.
__global__ void conv_scatter_phase_kernel(const float* __restrict src, float* __restrict dst, int64_t planes, int h, int w, int hs, int ws,
                                          int py, int px, int stride, int accumulate) {
    const int per_plane = hs * ws;
    for (int64_t plane = blockIdx.x; plane < planes; plane += gridDim.x) {
        const float* __restrict s = src ? src + plane * per_plane : nullptr;
        float* __restrict dp = dst + plane * h * w;
        for (int i = threadIdx.x; i < per_plane; i += blockDim.x) {
            const int r = i / ws, j = i - r * ws;
            float* d = dp + (py + stride * r) * w + px + stride * j;
            const float v = s ? s[i] : 0.f;
            *d = accumulate ? *d + v : v;
        }
    }
}

} // namespace tenmo
