// fp32 GEMM for gfx950 on v_mfma_f32_32x32x2_f32, LDS-tiled, views resolved in the global->LDS stage.
//
// C[b][M,N] (dense) (+)= A[b][M,K] . B[b][K,N] where A and B are arbitrary strided views.
// Replaces matmul_2d_tiled + MatmulNdGpu.launch (tenmo/kernels/matmul_kernel.mojo:38-120,:128-283).
//
// Workgroup: 256 threads = 4 wavefronts (2x2), one BM x BN tile of C, K walked in steps of BK=16
// through a double-buffered LDS stage (one barrier per step; the next step's global loads are in
// flight in registers while the current one feeds the matrix cores).
//
// Each operand is staged in the LDS layout that matches its memory order, so the global->LDS copy
// is always a straight 16-byte-per-lane copy and a transposed view costs nothing extra:
//   K-major  (unit stride along K: row-major A, transposed-view B):  tile[row][k], row pitch BK+4
//   MN-major (unit stride along M/N: transposed-view A, row-major B): tile[k][row]
// Any other striding (both strides non-unit, zero or overlapping) takes the element-wise
// "generic" loader into the K-major layout.
//
// MFMA operand order.  v_mfma_f32_32x32x2 consumes, per lane l, A[i=l%32][k=l/32] and
// B[k=l/32][j=l%32].  The sum over k is order-free, so within every 8-wide k chunk the kernel
// assigns MFMA step s (0..3) and lane half h=l/32 the index k = 4h + s.  A K-major operand then
// fetches its four steps with ONE 16-byte LDS read per 32x32 block (4 consecutive k of one row);
// an MN-major operand fetches, per step, one read of MB (or NB) consecutive rows which feed its
// MB blocks at once — block b of the wave tile owns rows {MB*i + b}, an interleave that is undone
// for free when C is stored (a lane then holds NB consecutive columns of a row: one vector store).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tenmo {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// vector types with element alignment: global loads/stores of these may start at any dword
typedef float f32x2_u __attribute__((ext_vector_type(2), aligned(4)));
typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));

constexpr int GEMM_BK = 16;
constexpr int GEMM_LDK = GEMM_BK + 4; // K-major row pitch: conflict-free 16-byte reads
constexpr int GEMM_THREADS = 256;
constexpr int MAX_BATCH_RANK = 6;

enum OperandMode : int { KMAJOR_VEC = 0, MNMAJOR_VEC = 1, KMAJOR_GEN = 2 };

struct BatchDesc {
    int32_t rank;
    int64_t shape[MAX_BATCH_RANK];
    int64_t a_str[MAX_BATCH_RANK];
    int64_t b_str[MAX_BATCH_RANK];
};

struct GemmArgs {
    const float* A; // already advanced by the view offset
    const float* B;
    float* C;
    int64_t a_rs, a_cs, b_rs, b_cs;
    int64_t M, N, K;
    int32_t accumulate;
    int32_t tiles_m, tiles_n;
    int32_t k_splits;     // >1: blockIdx.y selects a K range and partial tiles go to `partial`
    int64_t batch_count;
    int64_t k_per_split;  // multiple of GEMM_BK
    float* partial;       // [k_splits][batch*M*N] when k_splits > 1
    BatchDesc batch;
};

__device__ __forceinline__ void batch_offsets(const BatchDesc& bd, int64_t b, int64_t& a_off, int64_t& b_off) {
    a_off = 0; b_off = 0;
    for (int d = bd.rank - 1; d >= 0; --d) {
        int64_t c = b % bd.shape[d];
        b /= bd.shape[d];
        a_off += c * bd.a_str[d];
        b_off += c * bd.b_str[d];
    }
}

// ---- global -> registers -> LDS for one operand tile of ROWS x BK ----------------------------
// `row` indexes M for A and N for B; element(row, k) = base[row*rs + k*ks].
template <int ROWS, int MODE>
struct TileLoader {
    static constexpr int NCH = ROWS / 64; // 16-byte chunks per thread
    f32x4 r[NCH];

    __device__ __forceinline__ void load(const float* __restrict base, int64_t rs, int64_t ks,
                                         int64_t row0, int64_t k0, int64_t R, int64_t K, bool interior, int t) {
        if constexpr (MODE == KMAJOR_VEC) {
            const int kq = t & 3;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int64_t row = row0 + (t >> 2) + 64 * i;
                const int64_t k = k0 + 4 * kq;
                if (interior) {
                    r[i] = *reinterpret_cast<const f32x4_u*>(base + row * rs + k);
                } else {
                    f32x4 v = {0.f, 0.f, 0.f, 0.f};
                    if (row < R) {
                        const float* p = base + row * rs + k;
                        if (k + 3 < K) v = *reinterpret_cast<const f32x4_u*>(p);
                        else {
                            if (k + 0 < K) v.x = p[0];
                            if (k + 1 < K) v.y = p[1];
                            if (k + 2 < K) v.z = p[2];
                        }
                    }
                    r[i] = v;
                }
            }
        } else if constexpr (MODE == MNMAJOR_VEC) {
            constexpr int QPR = ROWS / 4; // chunks per k row
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int c = t + GEMM_THREADS * i;
                const int64_t k = k0 + c / QPR;
                const int64_t row = row0 + 4 * (c % QPR);
                if (interior) {
                    r[i] = *reinterpret_cast<const f32x4_u*>(base + k * ks + row);
                } else {
                    f32x4 v = {0.f, 0.f, 0.f, 0.f};
                    if (k < K) {
                        const float* p = base + k * ks + row;
                        if (row + 3 < R) v = *reinterpret_cast<const f32x4_u*>(p);
                        else {
                            if (row + 0 < R) v.x = p[0];
                            if (row + 1 < R) v.y = p[1];
                            if (row + 2 < R) v.z = p[2];
                        }
                    }
                    r[i] = v;
                }
            }
        } else { // KMAJOR_GEN: element loads, any strides
            const int kq = t & 3;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int64_t row = row0 + (t >> 2) + 64 * i;
                const int64_t k = k0 + 4 * kq;
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (row < R) {
                    const float* p = base + row * rs + k * ks;
                    if (k + 0 < K) v.x = p[0];
                    if (k + 1 < K) v.y = p[ks];
                    if (k + 2 < K) v.z = p[2 * ks];
                    if (k + 3 < K) v.w = p[3 * ks];
                }
                r[i] = v;
            }
        }
    }

    __device__ __forceinline__ void store(float* __restrict lds, int t) const {
        if constexpr (MODE == MNMAJOR_VEC) {
            constexpr int QPR = ROWS / 4;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int c = t + GEMM_THREADS * i;
                *reinterpret_cast<f32x4*>(lds + (c / QPR) * ROWS + 4 * (c % QPR)) = r[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < NCH; ++i)
                *reinterpret_cast<f32x4*>(lds + ((t >> 2) + 64 * i) * GEMM_LDK + 4 * (t & 3)) = r[i];
        }
    }
};

template <int ROWS, int MODE>
constexpr int lds_floats() { return MODE == MNMAJOR_VEC ? GEMM_BK * ROWS : ROWS * GEMM_LDK; }

// ---- LDS -> MFMA operand registers for one 8-wide k chunk ------------------------------------
// f[b][s]: operand of block b at MFMA step s.  `wave_row0` is the wave's first row in the tile.
template <int ROWS, int MODE, int NBLK>
__device__ __forceinline__ void load_fragments(const float* __restrict lds, int wave_row0, int kc, int lane, float (&f)[NBLK][4]) {
    const int h = lane >> 5, i = lane & 31;
    if constexpr (MODE == MNMAJOR_VEC) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const float* p = lds + (kc * 8 + 4 * h + s) * ROWS + wave_row0 + NBLK * i;
            if constexpr (NBLK == 4) {
                f32x4 v = *reinterpret_cast<const f32x4*>(p);
                f[0][s] = v.x; f[1][s] = v.y; f[2][s] = v.z; f[3][s] = v.w;
            } else if constexpr (NBLK == 2) {
                f32x2 v = *reinterpret_cast<const f32x2*>(p);
                f[0][s] = v.x; f[1][s] = v.y;
            } else {
                f[0][s] = p[0];
            }
        }
    } else {
#pragma unroll
        for (int b = 0; b < NBLK; ++b) {
            f32x4 v = *reinterpret_cast<const f32x4*>(lds + (wave_row0 + 32 * b + i) * GEMM_LDK + kc * 8 + 4 * h);
            f[b][0] = v.x; f[b][1] = v.y; f[b][2] = v.z; f[b][3] = v.w;
        }
    }
}

// position inside the wave tile of MFMA index x (0..31) of block b
template <int MODE, int NBLK>
__device__ __forceinline__ int tile_pos(int b, int x) { return MODE == MNMAJOR_VEC ? NBLK * x + b : 32 * b + x; }

// XCD-aware, L2-friendly block order.  Hardware deals consecutive workgroup ids round-robin to
// the 8 XCDs (each with its own L2); give every XCD a contiguous run of tiles, and walk the
// tiles of a run in groups of GROUP_M tile-rows so that concurrently resident tiles share
// A rows and B columns.
__device__ __forceinline__ int64_t xcd_remap(int64_t pid, int64_t n) {
    constexpr int XCDS = 8;
    const int64_t q = n / XCDS, rem = n % XCDS;
    const int64_t xcd = pid % XCDS, local = pid / XCDS;
    const int64_t base = xcd < rem ? xcd * (q + 1) : rem * (q + 1) + (xcd - rem) * q;
    return base + local;
}

template <int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_mfma_kernel(const GemmArgs g) {
    constexpr int TM = BM / 2, TN = BN / 2;     // wave tile (2x2 waves)
    constexpr int MB = TM / 32, NB = TN / 32;   // 32x32 MFMA blocks per wave tile
    constexpr int A_FLOATS = lds_floats<BM, AMODE>();
    constexpr int B_FLOATS = lds_floats<BN, BMODE>();
    __shared__ __attribute__((aligned(16))) float lds[2 * (A_FLOATS + B_FLOATS)];

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- which tile ----
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    int64_t pid = xcd_remap(blockIdx.x, gridDim.x);
    const int64_t batch = pid / tiles;
    const int64_t tid = pid % tiles;
    constexpr int GROUP_M = 8;
    const int64_t per_group = (int64_t)GROUP_M * g.tiles_n;
    const int64_t first_m = (tid / per_group) * GROUP_M;
    const int64_t gsz = min((int64_t)g.tiles_m - first_m, (int64_t)GROUP_M);
    const int64_t tile_m = first_m + (tid % per_group) % gsz;
    const int64_t tile_n = (tid % per_group) / gsz;
    const int64_t m0 = tile_m * BM, n0 = tile_n * BN;

    int64_t a_boff, b_boff;
    batch_offsets(g.batch, batch, a_boff, b_boff);
    const float* __restrict Ab = g.A + a_boff;
    const float* __restrict Bb = g.B + b_boff;

    // operand strides in (row, k) form
    const int64_t a_row_s = g.a_rs, a_k_s = g.a_cs;   // A(m,k)
    const int64_t b_row_s = g.b_cs, b_k_s = g.b_rs;   // B(n,k) = Bmem[k*b_rs + n*b_cs]

    int64_t k_begin = 0, k_end = g.K;
    if (g.k_splits > 1) {
        k_begin = (int64_t)blockIdx.y * g.k_per_split;
        k_end = min(g.K, k_begin + g.k_per_split);
    }
    const int64_t nk = (k_end > k_begin) ? (k_end - k_begin + GEMM_BK - 1) / GEMM_BK : 0;
    const bool rows_interior = (m0 + BM <= g.M) && (n0 + BN <= g.N);

    f32x16 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    TileLoader<BM, AMODE> la;
    TileLoader<BN, BMODE> lb;

    if (nk > 0) {
        const bool in0 = rows_interior && (k_begin + GEMM_BK <= k_end);
        la.load(Ab, a_row_s, a_k_s, m0, k_begin, g.M, k_end, in0, t);
        lb.load(Bb, b_row_s, b_k_s, n0, k_begin, g.N, k_end, in0, t);
        la.store(lds, t);
        lb.store(lds + A_FLOATS, t);
    }
    __syncthreads();

    for (int64_t it = 0; it < nk; ++it) {
        const int cur = (int)(it & 1);
        const float* __restrict As = lds + cur * (A_FLOATS + B_FLOATS);
        const float* __restrict Bs = As + A_FLOATS;
        const bool more = (it + 1 < nk);
        if (more) {
            const int64_t k0 = k_begin + (it + 1) * GEMM_BK;
            const bool interior = rows_interior && (k0 + GEMM_BK <= k_end);
            la.load(Ab, a_row_s, a_k_s, m0, k0, g.M, k_end, interior, t);
            lb.load(Bb, b_row_s, b_k_s, n0, k0, g.N, k_end, interior, t);
        }
#pragma unroll
        for (int kc = 0; kc < GEMM_BK / 8; ++kc) {
            float fa[MB][4], fb[NB][4];
            load_fragments<BM, AMODE, MB>(As, wm * TM, kc, lane, fa);
            load_fragments<BN, BMODE, NB>(Bs, wn * TN, kc, lane, fb);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int i = 0; i < MB; ++i)
#pragma unroll
                    for (int j = 0; j < NB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
        }
        if (more) {
            float* nxt = lds + (cur ^ 1) * (A_FLOATS + B_FLOATS);
            la.store(nxt, t);
            lb.store(nxt + A_FLOATS, t);
        }
        __syncthreads();
    }

    // ---- epilogue ----
    float* __restrict Cb;
    bool accumulate = g.accumulate != 0;
    if (g.k_splits > 1) {
        Cb = g.partial + ((int64_t)blockIdx.y * g.batch_count + batch) * g.M * g.N;
        accumulate = false;
    } else {
        Cb = g.C + batch * g.M * g.N;
    }
    const int h = lane >> 5, x = lane & 31;
#pragma unroll
    for (int i = 0; i < MB; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int ip = 8 * (e >> 2) + 4 * h + (e & 3); // MFMA row of accumulator element e
            const int64_t row = m0 + wm * TM + tile_pos<AMODE, MB>(i, ip);
            if (row >= g.M) continue;
            float* crow = Cb + row * g.N;
            if constexpr (BMODE == MNMAJOR_VEC && NB > 1) {
                const int64_t col = n0 + wn * TN + NB * x;
                if (col + NB <= g.N) {
                    if constexpr (NB == 4) {
                        f32x4 v = {acc[i][0][e], acc[i][1][e], acc[i][2][e], acc[i][3][e]};
                        if (accumulate) v += *reinterpret_cast<const f32x4_u*>(crow + col);
                        *reinterpret_cast<f32x4_u*>(crow + col) = v;
                    } else {
                        f32x2 v = {acc[i][0][e], acc[i][1][e]};
                        if (accumulate) v += *reinterpret_cast<const f32x2_u*>(crow + col);
                        *reinterpret_cast<f32x2_u*>(crow + col) = v;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < NB; ++j)
                        if (col + j < g.N) crow[col + j] = accumulate ? crow[col + j] + acc[i][j][e] : acc[i][j][e];
                }
            } else {
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const int64_t col = n0 + wn * TN + tile_pos<BMODE, NB>(j, x);
                    if (col < g.N) crow[col] = accumulate ? crow[col] + acc[i][j][e] : acc[i][j][e];
                }
            }
        }
    }
}

// Sums the k_splits partial results into C (plain or accumulating).
__global__ void splitk_reduce_kernel(const float* __restrict partial, float* __restrict C, int64_t n, int splits, int accumulate) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) {
        float s = accumulate ? C[i] : 0.f;
        for (int p = 0; p < splits; ++p) s += partial[(int64_t)p * n + i];
        C[i] = s;
    }
}

} // namespace tenmo
