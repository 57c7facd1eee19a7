// Memory-bound products for gfx950: matrix x vector, (few rows) x matrix, dot.
// Every kernel streams the matrix exactly once with 16-byte-per-lane loads and reduces inside the
// wavefront; none of them can use the matrix cores profitably (<= 8 flop per byte of HBM traffic).
//
// Replaces matrix_vector_nd (tenmo/kernels/matrixvector_kernel.mojo:13-77), vector_matmul_nd
// (tenmo/kernels/vectormatrix_kernel.mojo:13-77) and dot_product (tenmo/kernels/dotproduct_kernel.mojo:19-110).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>
#include "gemm_mfma.hpp"

namespace tenmo {

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) x += __shfl_down(x, off, 64);
    return x;
}

struct GemvArgs {
    const float* Mx;  // advanced by the view offset
    const float* v;
    float* out;
    int64_t m_rs, m_cs, v_s;
    int64_t rows, k;       // row kernel: out has `rows` entries per batch, k = reduction length
    int32_t accumulate;
    int64_t batch0;        // batch index of blockIdx.y == 0 (a grid dimension holds 65535 batches; more go in several launches)
    BatchDesc batch;       // a_str: matrix batch strides, b_str: vector batch strides
};

// ---- rows kernel: unit stride along the reduction (row-major matrix . vector) ----------------
// A unit of WPR wavefronts (1, or the 4 of a workgroup) owns RPW consecutive rows.  It walks the
// reduction in batches of UNROLL 16-byte steps per lane: the vector's values of a batch are loaded
// once into registers, then each of the RPW rows contributes one contiguous burst of WPR x UNROLL KiB
// with all its loads in flight.  Measured on 16384^2 (fractions of the 8 TB/s HBM peak): workgroup
// per 4 rows with the vector in registers 0.90; one row per unit 0.83-0.85 (the vector's loads then
// compete with the matrix's); several rows interleaved load by load in one wavefront 0.65-0.80.
// WPR = 1 is for rows too short to give four wavefronts a full batch each.
constexpr int MV_WAVES = 4;
template <int WPR, int RPW, int UNROLL, bool V_UNIT>
__global__ __launch_bounds__(64 * MV_WAVES) void mv_rows_kernel(const GemvArgs g) {
    static_assert(WPR == 1 || WPR == MV_WAVES, "one wavefront or the whole workgroup per row");
    __shared__ float part[MV_WAVES][RPW];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tid = WPR == 1 ? lane : (int)threadIdx.x;           // index inside the unit
    const int64_t unit = WPR == 1 ? (int64_t)blockIdx.x * MV_WAVES + wave : (int64_t)blockIdx.x;
    const int64_t row0 = unit * RPW;
    if (row0 >= g.rows) return; // WPR == 4: uniform over the workgroup
    const int64_t batch = g.batch0 + blockIdx.y;
    int64_t m_off, v_off;
    batch_offsets(g.batch, batch, m_off, v_off);
    const float* __restrict vb = g.v + v_off;
    const int64_t k = g.k;
    constexpr int STEP = 64 * WPR * 4;

    auto vec4 = [&](int64_t kx) -> f32x4 {
        if constexpr (V_UNIT) return *reinterpret_cast<const f32x4_u*>(vb + kx);
        else return f32x4{vb[kx * g.v_s], vb[(kx + 1) * g.v_s], vb[(kx + 2) * g.v_s], vb[(kx + 3) * g.v_s]};
    };
    const float* rowp[RPW]; // rows past the end repeat the last one; their sums are dropped
    float acc[RPW];
#pragma unroll
    for (int j = 0; j < RPW; ++j) { rowp[j] = g.Mx + m_off + min(row0 + j, g.rows - 1) * g.m_rs; acc[j] = 0.f; }
    auto fma4 = [](float a, const f32x4& m, const f32x4& x) {
        a = fmaf(m.x, x.x, a); a = fmaf(m.y, x.y, a); a = fmaf(m.z, x.z, a); return fmaf(m.w, x.w, a);
    };

    int64_t kk = (int64_t)tid * 4;
    for (; kk + (int64_t)(UNROLL - 1) * STEP + 3 < k; kk += (int64_t)UNROLL * STEP) { // full batches
        f32x4 x[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) x[u] = vec4(kk + (int64_t)u * STEP);
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            f32x4 m[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) m[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(rowp[j] + kk + (int64_t)u * STEP));
            __builtin_amdgcn_sched_barrier(0); // every load of the row is issued before the first use
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) acc[j] = fma4(acc[j], m[u], x[u]);
        }
    }
    if (__any(kk + 3 < k)) { // the last, partial batch: the whole groups of 4 that remain
        f32x4 x[UNROLL];
        bool ok[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const int64_t kx = kk + (int64_t)u * STEP;
            ok[u] = kx + 3 < k;
            x[u] = f32x4{0.f, 0.f, 0.f, 0.f};
            if (ok[u]) x[u] = vec4(kx);
        }
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            f32x4 m[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                m[u] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (ok[u]) m[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(rowp[j] + kk + (int64_t)u * STEP));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) acc[j] = fma4(acc[j], m[u], x[u]);
        }
    }
    if (tid < (int)(k & 3)) { // the last k % 4 elements, one per lane
        const int64_t kx = (k & ~(int64_t)3) + tid;
        const float xe = vb[kx * g.v_s];
#pragma unroll
        for (int j = 0; j < RPW; ++j) acc[j] = fmaf(rowp[j][kx], xe, acc[j]);
    }
    float* __restrict ob = g.out + batch * g.rows + row0;
    if constexpr (WPR == 1) {
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            const float s = wave_sum(acc[j]);
            if (lane == 0 && row0 + j < g.rows) ob[j] = g.accumulate ? ob[j] + s : s;
        }
    } else {
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            const float s = wave_sum(acc[j]);
            if (lane == 0) part[wave][j] = s;
        }
        __syncthreads();
        if (threadIdx.x < RPW && row0 + threadIdx.x < g.rows) {
            float s = 0.f;
#pragma unroll
            for (int w = 0; w < MV_WAVES; ++w) s += part[w][threadIdx.x];
            ob[threadIdx.x] = g.accumulate ? ob[threadIdx.x] + s : s;
        }
    }
}

// ---- columns kernel: unit stride across the outputs ((R x k) . (k x n), R <= 8) ---------------
// out[r][j] = sum_k X[r][k] * Mx[k][j].  A workgroup owns 1024 consecutive columns (one 16-byte
// load per lane per k row: 1 KiB bursts per wavefront; dword loads when rows are not 16-byte
// aligned) and one slice of k; the R x slice block of
// X is staged in LDS and broadcast.  Partial sums of the k slices go to `partial` and are added by
// colsplit_reduce_kernel, so the result does not depend on scheduling.
struct ColsArgs {
    const float* X;   // (R x k) left operand: vector(s); element (r,k) = X[r*x_rs + k*x_ks]
    const float* Mx;  // (k x n) right operand, unit stride along n, row pitch m_rs
    float* out;       // dense [batch][R][n]  (or partial [splits][batch][R][n])
    int64_t x_rs, x_ks, m_rs;
    int64_t k, n;
    int32_t rows;     // actual row count (<= R)
    int32_t accumulate;
    int32_t k_splits;
    int64_t k_per_split;
    int64_t batch0;      // batch index of blockIdx.z == 0 (more than 65535 batches go in several launches)
    int64_t batch_total; // batches of the whole product: the partial sums are laid out [k_splits][batch_total][R][n]
    BatchDesc batch;  // a_str: X batch strides, b_str: Mx batch strides
    // K slices added inside the launch (the JOIN instantiations): the dense result [batch][R][n], and one arrival counter per
    // column block and batch of the launch, all zero between launches
    float* joined;
    uint32_t* arrivals;
};

constexpr int COLS_THREADS = 256;
constexpr int COLS_STAGE_FLOATS = 2048; // R x (2048 / R) left-operand values are staged in LDS per refill
constexpr int COLS_KSLICE_MIN = 32; // granularity of the K slices handed to workgroups

// The K slices of one column block added by the workgroup that finishes last, inside the streaming launch: every
// workgroup stores its partial sums, makes them visible to the device (fence) and counts itself in on the block's
// counter; the one that sees all others' arrivals reads the k_splits partial sums of the block back — slices in ascending
// order, on top of the old value when accumulating: the order of splitk_reduce_kernel, so the result is the same to the bit
// and independent of scheduling — and puts the counter back to zero for the next launch.  Nobody waits for anybody.
// Columns [first, first + width) of every row; 32 loads in flight per thread.
__device__ __forceinline__ void cols_join_slices(const ColsArgs& g, int64_t batch, int64_t first, int width) {
    __shared__ uint32_t last_to_arrive;
    __threadfence();
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t* counter = g.arrivals + (int64_t)blockIdx.z * gridDim.x + blockIdx.x;
        const bool last = atomicAdd(counter, 1u) == (uint32_t)g.k_splits - 1u;
        if (last) *counter = 0u;
        last_to_arrive = last ? 1u : 0u;
    }
    __syncthreads();
    if (!last_to_arrive) return;
    __threadfence(); // nothing below may be served from before the other workgroups' arrival
    const int64_t plane = (int64_t)g.rows * g.n, slice_stride = g.batch_total * plane;
    const float* part = g.out + batch * plane;
    float* dst = g.joined + batch * plane;
    const int64_t live = min((int64_t)width, g.n - first); // columns of this block inside the row
    const int items = (int)(g.rows * live);
    constexpr int IU = 4, SU = 8;
    for (int i0 = threadIdx.x; i0 < items; i0 += IU * COLS_THREADS) {
        int64_t at[IU];
        float sum[IU];
#pragma unroll
        for (int u = 0; u < IU; ++u) {
            const int i = min(i0 + u * COLS_THREADS, items - 1); // surplus threads repeat the last item and do not store
            at[u] = (int64_t)(i / (int)live) * g.n + first + i % (int)live;
            sum[u] = g.accumulate ? dst[at[u]] : 0.f;
        }
        int p = 0;
        for (; p + SU <= g.k_splits; p += SU) {
            float v[IU][SU];
#pragma unroll
            for (int u = 0; u < IU; ++u)
#pragma unroll
                for (int q = 0; q < SU; ++q) v[u][q] = part[(p + q) * slice_stride + at[u]];
#pragma unroll
            for (int u = 0; u < IU; ++u)
#pragma unroll
                for (int q = 0; q < SU; ++q) sum[u] += v[u][q];
        }
        for (; p < g.k_splits; ++p)
#pragma unroll
            for (int u = 0; u < IU; ++u) sum[u] += part[p * slice_stride + at[u]];
#pragma unroll
        for (int u = 0; u < IU; ++u)
            if (i0 + u * COLS_THREADS < items) dst[at[u]] = sum[u];
    }
}

// ALIGNED: every row of the matrix starts on a 16-byte boundary -> a lane owns 4 consecutive columns
// and moves them with one 16-byte load.  Otherwise (row pitch not a multiple of 4 floats, e.g.
// N = 50257) 16-byte loads would straddle and run at half rate, so a lane owns 4 columns 256 apart
// and uses dword loads, each still one contiguous 256-byte burst per wavefront.
template <int R, bool ALIGNED, bool JOIN = false> // JOIN: k_splits > 1 and the slices are added inside the launch (cols_join_slices)
__global__ __launch_bounds__(COLS_THREADS) void cols_kernel(const ColsArgs g) {
    constexpr int COLS_KCHUNK = COLS_STAGE_FLOATS / R; // k rows per LDS refill
    __shared__ float xs[R][COLS_KCHUNK];
    const int t = threadIdx.x;
    const int64_t col0 = (int64_t)blockIdx.x * COLS_THREADS * 4 + (ALIGNED ? 4 * t : t);
    constexpr int CSTEP = ALIGNED ? 1 : COLS_THREADS; // distance between a lane's 4 columns
    const int64_t batch = g.batch0 + blockIdx.z;
    int64_t x_off, m_off;
    batch_offsets(g.batch, batch, x_off, m_off);
    const float* __restrict Xb = g.X + x_off;
    const float* __restrict Mb = g.Mx + m_off;

    const int64_t k_begin = (int64_t)blockIdx.y * g.k_per_split;
    const int64_t k_end = min(g.k, k_begin + g.k_per_split);
    const bool full = (col0 + 3 * CSTEP < g.n);
    const bool any = (col0 < g.n);
    // whether every lane of this wavefront has its four columns inside the row (wave-uniform)
    const bool wave_full = (col0 + (63 - (t & 63)) * (ALIGNED ? 4 : 1) + 3 * CSTEP < g.n);

    f32x4 acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load_full = [&](const float* __restrict p) -> f32x4 {
        if constexpr (ALIGNED) return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
        else return f32x4{__builtin_nontemporal_load(p), __builtin_nontemporal_load(p + CSTEP),
                          __builtin_nontemporal_load(p + 2 * CSTEP), __builtin_nontemporal_load(p + 3 * CSTEP)};
    };
    // Ragged wavefront (the row ends inside it): columns past the end are moved onto the last valid
    // one, so the loads stay unconditional and as many are in flight as on the fast path; what they
    // bring is never stored.
    int64_t coff[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) coff[e] = min(col0 + e * CSTEP, g.n - 1) - col0;
    auto load_clamped = [&](const float* __restrict p) -> f32x4 {
        return f32x4{__builtin_nontemporal_load(p + coff[0]), __builtin_nontemporal_load(p + coff[1]),
                     __builtin_nontemporal_load(p + coff[2]), __builtin_nontemporal_load(p + coff[3])};
    };
    // U independent row loads in flight per lane; the last batch of a chunk re-reads row len-1 for
    // the rows it lacks and drops them.
    constexpr int U = R <= 2 ? 16 : 8;
    auto stream = [&](const float* __restrict p, int first, int len, auto load4) { // rows [first, len), first % U == 0
        int kk = first;
        for (; kk + U <= len; kk += U) {
            f32x4 m[U];
#pragma unroll
            for (int u = 0; u < U; ++u) m[u] = load4(p + (int64_t)(kk + u) * g.m_rs);
            __builtin_amdgcn_sched_barrier(0); // all U loads are issued before the first use
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r] += m[u] * xs[r][kk + u];
        }
        if (kk < len) {
            f32x4 m[U];
#pragma unroll
            for (int u = 0; u < U; ++u) m[u] = load4(p + (int64_t)min(kk + u, len - 1) * g.m_rs);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (kk + u >= len) m[u] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int r = 0; r < R; ++r) acc[r] += m[u] * xs[r][kk + u];
            }
        }
    };
    // Workgroups start at different eighths of their K slices and wrap around: slices that lie a power
    // of two apart in memory would otherwise walk the same memory channels in step.
    const int rotation = (int)((blockIdx.y * 5 + blockIdx.x * 3) & 7);

    for (int64_t kc = k_begin; kc < k_end; kc += COLS_KCHUNK) {
        const int len = (int)min((int64_t)COLS_KCHUNK, k_end - kc);
        __syncthreads();
        for (int idx = t; idx < R * COLS_KCHUNK; idx += COLS_THREADS) {
            const int r = idx / COLS_KCHUNK, kk = idx % COLS_KCHUNK;
            xs[r][kk] = (r < g.rows && kk < len) ? Xb[(int64_t)r * g.x_rs + (kc + kk) * g.x_ks] : 0.f;
        }
        __syncthreads();
        const float* __restrict p = Mb + kc * g.m_rs + col0;
        const int first = len >= 16 * U ? len / 8 * rotation / U * U : 0; // short slices are not worth a second ragged batch
        if (wave_full) { stream(p, first, len, load_full); stream(p, 0, first, load_full); }
        else if (any) { stream(p, first, len, load_clamped); stream(p, 0, first, load_clamped); }
    }
    if constexpr (!JOIN) {
        if (!any) return;
    }
    if (!JOIN || any) {
        const bool to_partial = g.k_splits > 1;
        float* __restrict ob = g.out + ((to_partial ? (int64_t)blockIdx.y * g.batch_total : 0) + batch) * g.rows * g.n;
        const bool accumulate = g.accumulate && !to_partial;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (r >= g.rows) break;
            float* o = ob + (int64_t)r * g.n + col0;
            if (ALIGNED && full) {
                f32x4 v = acc[r];
                if (accumulate) v += *reinterpret_cast<const f32x4_u*>(o);
                *reinterpret_cast<f32x4_u*>(o) = v;
            } else {
                const float a[4] = {acc[r].x, acc[r].y, acc[r].z, acc[r].w};
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col0 + e * CSTEP < g.n) o[e * CSTEP] = accumulate ? o[e * CSTEP] + a[e] : a[e];
            }
        }
    }
    if constexpr (JOIN) cols_join_slices(g, batch, (int64_t)blockIdx.x * COLS_THREADS * 4, COLS_THREADS * 4);
}

// ---- columns kernel for rows that do not start on 16-byte boundaries ---------------------------
// Same job as cols_kernel, for a matrix whose first row IS 16-byte aligned but whose row pitch is
// not a multiple of 4 floats (N = 50257): row r then starts m(r) = (r * pitch) % 4 elements past a
// 16-byte boundary, and m depends only on r % 4.  Every lane still moves one ALIGNED 16-byte group
// per row — the group that starts m(r) elements before its nominal columns — and keeps one
// accumulator set per r % 4, so that a set always holds the same four columns.  At the end the four
// sets are shifted back by their m through LDS and added.  Because a set's columns reach up to three
// to the left of the nominal ones, a workgroup produces COLS_SHIFT_WIDTH = 1020 outputs from 1024
// loaded columns.  The last row of the matrix is read element by element (an aligned group there
// could end past the allocation); groups of other rows that run past the row end read the next
// row's first elements, which are discarded.
constexpr int COLS_SHIFT_WIDTH = COLS_THREADS * 4 - 4;

template <int R, bool JOIN = false>
__global__ __launch_bounds__(COLS_THREADS) void cols_shift_kernel(const ColsArgs g) {
    constexpr int COLS_KCHUNK = COLS_STAGE_FLOATS / R; // k rows per LDS refill
    __shared__ float xs[R][COLS_KCHUNK];
    __shared__ float outs[R][COLS_THREADS * 4 + 4];
    const int t = threadIdx.x;
    const int64_t block0 = (int64_t)blockIdx.x * COLS_SHIFT_WIDTH; // first output column of the workgroup
    const int64_t batch = g.batch0 + blockIdx.z;
    int64_t x_off, m_off;
    batch_offsets(g.batch, batch, x_off, m_off);
    const float* __restrict Xb = g.X + x_off;
    const float* __restrict Mb = g.Mx + m_off; // 16-byte aligned (the host checks)
    const int64_t k_begin = (int64_t)blockIdx.y * g.k_per_split; // a multiple of 4
    const int64_t k_end = min(g.k, k_begin + g.k_per_split);
    const int64_t k_vec_end = min(k_end, g.k - 1);                // the matrix's last row is done apart
    int mj[4]; // misalignment of the rows with r % 4 == j
#pragma unroll
    for (int j = 0; j < 4; ++j) mj[j] = (int)((j * (g.m_rs & 3)) & 3);

    f32x4 acc[4][R];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < R; ++r) acc[j][r] = f32x4{0.f, 0.f, 0.f, 0.f};
    // First column of this lane's group for class j.  A group that lies wholly beyond the row is
    // moved back by whole groups onto the last one that starts inside it: the load stays unconditional
    // and in bounds, and what it brings lands in output columns >= n, which are never stored.
    int64_t c0[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        c0[j] = block0 - mj[j] + 4 * t;
        if (c0[j] >= g.n) c0[j] -= 4 * ((c0[j] - g.n) / 4 + 1);
    }

    for (int64_t kc = k_begin; kc < k_end; kc += COLS_KCHUNK) {
        const int len = (int)min((int64_t)COLS_KCHUNK, k_end - kc);
        const int vlen = (int)max((int64_t)0, min((int64_t)len, k_vec_end - kc));
        __syncthreads();
        for (int idx = t; idx < R * COLS_KCHUNK; idx += COLS_THREADS) {
            const int r = idx / COLS_KCHUNK, kk = idx % COLS_KCHUNK;
            xs[r][kk] = (r < g.rows && kk < len) ? Xb[(int64_t)r * g.x_rs + (kc + kk) * g.x_ks] : 0.f;
        }
        __syncthreads();
        int kk = 0;
        constexpr int U = 8;
        const float* __restrict pc = Mb + kc * g.m_rs;
        for (; kk + U <= vlen; kk += U) { // kc + kk is a multiple of 4: row kk + u has class u % 4
            f32x4 m[U];
#pragma unroll
            for (int u = 0; u < U; ++u)
                m[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pc + (int64_t)(kk + u) * g.m_rs + c0[u & 3]));
            __builtin_amdgcn_sched_barrier(0); // all U loads are issued before the first use
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int r = 0; r < R; ++r) acc[u & 3][r] += m[u] * xs[r][kk + u];
        }
        if (kk < vlen) { // last batch of the chunk: the rows it lacks re-read the chunk's first row and are dropped
            f32x4 m[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const bool ok = kk + u < vlen;
                m[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(pc + (int64_t)(ok ? kk + u : 0) * g.m_rs + (ok ? c0[u & 3] : c0[0])));
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // (skipped, not multiplied by zero: xs[.][vlen] is the vector's real last value when the matrix's last row is
                // done apart below, and 0 x inf would put a NaN where the reference has an infinity)
                if (kk + u < vlen) {
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[u & 3][r] += m[u] * xs[r][kk + u];
                }
            }
        }
        if (vlen < len) { // the matrix's last row: element by element, bounds-checked
            const int kl = vlen;
            const int j = (int)((kc + kl) & 3);
            const float* __restrict row = pc + (int64_t)kl * g.m_rs;
            const int64_t c = block0 - mj[j] + 4 * t;
            f32x4 m0 = {0.f, 0.f, 0.f, 0.f};
            if (c >= 0 && c < g.n) m0.x = row[c];
            if (c + 1 >= 0 && c + 1 < g.n) m0.y = row[c + 1];
            if (c + 2 >= 0 && c + 2 < g.n) m0.z = row[c + 2];
            if (c + 3 >= 0 && c + 3 < g.n) m0.w = row[c + 3];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj)
                if (jj == j)
#pragma unroll
                    for (int r = 0; r < R; ++r) acc[jj][r] += m0 * xs[r][kl];
        }
    }
    // shift the four sets back and add them: set j's element e of lane t is column block0 - mj + 4t + e
    for (int idx = t; idx < R * (COLS_THREADS * 4 + 4); idx += COLS_THREADS) (&outs[0][0])[idx] = 0.f;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            float* o = &outs[r][4 * t + 3 - mj[j]]; // local column + 3
            o[0] += acc[j][r].x; o[1] += acc[j][r].y; o[2] += acc[j][r].z; o[3] += acc[j][r].w;
        }
        __syncthreads();
    }
    const bool to_partial = g.k_splits > 1;
    float* __restrict ob = g.out + ((to_partial ? (int64_t)blockIdx.y * g.batch_total : 0) + batch) * g.rows * g.n;
    const bool accumulate = g.accumulate && !to_partial;
    for (int r = 0; r < R; ++r) {
        if (r >= g.rows) break;
        for (int c = t; c < COLS_SHIFT_WIDTH; c += COLS_THREADS) {
            const int64_t col = block0 + c;
            if (col < g.n) {
                float* o = ob + (int64_t)r * g.n + col;
                *o = accumulate ? *o + outs[r][c + 3] : outs[r][c + 3];
            }
        }
    }
    if constexpr (JOIN) cols_join_slices(g, batch, block0, COLS_SHIFT_WIDTH);
}

// ---- generic kernel: any strides, one thread per output (correct, not fast) -------------------
__global__ void mv_generic_kernel(const GemvArgs g) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= g.rows) return;
    const int64_t batch = g.batch0 + blockIdx.y;
    int64_t m_off, v_off;
    batch_offsets(g.batch, batch, m_off, v_off);
    const float* Mb = g.Mx + m_off + i * g.m_rs;
    const float* vb = g.v + v_off;
    float acc = 0.f;
    for (int64_t j = 0; j < g.k; ++j) acc = fmaf(Mb[j * g.m_cs], vb[j * g.v_s], acc);
    float* o = g.out + batch * g.rows + i;
    *o = g.accumulate ? *o + acc : acc;
}

// ---- dot ---------------------------------------------------------------------------------------
constexpr int DOT_THREADS = 256;
__device__ __forceinline__ float block_sum(float x) {
    __shared__ float part[DOT_THREADS / 64];
    x = wave_sum(x);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = x;
    __syncthreads();
    float s = 0.f;
    if (threadIdx.x == 0)
        for (int w = 0; w < DOT_THREADS / 64; ++w) s += part[w];
    return s; // valid on thread 0
}

__global__ __launch_bounds__(DOT_THREADS) void dot_partial_kernel(const float* __restrict a, int64_t a_s, const float* __restrict b, int64_t b_s,
                                                                  int64_t n, float* __restrict partial) {
    float acc = 0.f;
    const int64_t stride = (int64_t)gridDim.x * DOT_THREADS;
    for (int64_t i = (int64_t)blockIdx.x * DOT_THREADS + threadIdx.x; i < n; i += stride) acc = fmaf(a[i * a_s], b[i * b_s], acc);
    const float s = block_sum(acc);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

// Unit strides: 16-byte streaming loads, U groups of each vector in flight per thread, every workgroup side by side in one
// window that moves through the arrays (the element-at-a-time kernel above reaches 4 TB/s on 2 GB; this form 6.5+).
// The n % 4 last elements are added by the first threads of workgroup 0.  Fixed partition: the result is deterministic.
template <int U>
__global__ __launch_bounds__(DOT_THREADS) void dot_partial_vec_kernel(const float* __restrict a, const float* __restrict b, int64_t n, float* __restrict partial) {
    const int64_t n4 = n / 4, stride = (int64_t)gridDim.x * DOT_THREADS;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    int64_t i = (int64_t)blockIdx.x * DOT_THREADS + threadIdx.x;
    for (; i + (U - 1) * stride < n4; i += U * stride) {
        f32x4 x[U], y[U];
#pragma unroll
        for (int u = 0; u < U; ++u) x[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(a) + i + u * stride);
#pragma unroll
        for (int u = 0; u < U; ++u) y[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4_u*>(b) + i + u * stride);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; ++u) acc += x[u] * y[u];
    }
    for (; i < n4; i += stride) acc += reinterpret_cast<const f32x4_u*>(a)[i] * reinterpret_cast<const f32x4_u*>(b)[i];
    float s = (acc.x + acc.y) + (acc.z + acc.w);
    if (blockIdx.x == 0 && 4 * n4 + threadIdx.x < n) s = fmaf(a[4 * n4 + threadIdx.x], b[4 * n4 + threadIdx.x], s);
    s = block_sum(s);
    if (threadIdx.x == 0) partial[blockIdx.x] = s;
}

__global__ __launch_bounds__(DOT_THREADS) void dot_final_kernel(const float* __restrict partial, int nparts, float* __restrict out) {
    float acc = 0.f;
    for (int i = threadIdx.x; i < nparts; i += DOT_THREADS) acc += partial[i];
    const float s = block_sum(acc);
    if (threadIdx.x == 0) *out = s;
}

} // namespace tenmo
