// fp32 GEMM for gfx950 on v_mfma_f32_32x32x2_f32, LDS-tiled, views resolved in the global->LDS stage.
//
// C[b][M,N] (dense) (+)= A[b][M,K] . B[b][K,N] where A and B are arbitrary strided views.
// Replaces matmul_2d_tiled + MatmulNdGpu.launch (tenmo/kernels/matmul_kernel.mojo:38-120,:128-283).
//
// Workgroup: 256 threads = 4 wavefronts (2x2), one BM x BN tile of C, K walked in steps of BK=16.
// Two or more workgroups share a CU (<= 256 VGPRs per lane, <= 72 KiB LDS each), but the inner
// loop does not depend on that: every LDS read and memory load sits between two MFMAs of the same
// wavefront, so one wavefront per SIMD already keeps the matrix pipe busy.
//
// Each operand is staged in the LDS layout that matches its memory order, so the global->LDS copy
// is always a straight 16-byte-per-lane copy and a transposed view costs nothing extra:
//   K-major  (unit stride along K: row-major A, transposed-view B): tile[row][16 k], the four
//            16-byte chunks of a row XOR-swizzled by (row>>2)&3 so that both the row-wise copy-in
//            and the column-wise operand fetch are free of bank conflicts without padding
//   MN-major (unit stride along M/N: transposed-view A, row-major B): tile[k][row]
// Any other striding (both strides non-unit, zero or overlapping) takes the element-wise
// "generic" loader into the K-major layout.
//
// The main path is a three-stage LDS ring filled by direct global->LDS loads
// (global_load_lds_dwordx4 with scalar base + 32-bit lane offset: no staging registers, no vector
// address arithmetic, two K steps in flight).  The operand fetch of the next half step and the
// direct loads are issued one at a time behind the MFMAs of the current half step and carried
// across the workgroup barrier, so the matrix pipe does not drain.  Tiles that hang over the last
// row or column take the same path with clamped rows.  The K tail and operands the direct path
// cannot take (misaligned, generic strides) use register-staged, bounds-checked loads into two
// stages of the same ring.
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
#include <type_traits>
#include <stdint.h>

#include "gemm_index.hpp"
#include "gfx950_asm.hpp"

namespace tenmo {

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// vector types with element alignment: global loads/stores of these may start at any dword
typedef float f32x2_u __attribute__((ext_vector_type(2), aligned(4)));
typedef float f32x4_u __attribute__((ext_vector_type(4), aligned(4)));

constexpr int GEMM_BK = 16;
constexpr int GEMM_THREADS = 256;

enum OperandMode : int { KMAJOR_VEC = 0, MNMAJOR_VEC = 1, KMAJOR_GEN = 2 };

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
    // fused epilogue, applied to the finished sums (by the slice reduction when k_splits > 1):
    const float* bias;    // + bias[col], or null                         (Linear: x.W + b)
    const float* mask;    // dense like C: result zeroed where mask <= 0, or null   (ReLU backward on dX)
    int32_t relu;         // max(.,0) after the bias                      (ReLU forward)
    int32_t bias_rows;    // the bias is indexed by the row of C instead of the column (convolution: one per filter)
    float* colsum;        // [batch][N] or null: receives the column sums of the finished C (after the epilogue above); only for
                          // a launch whose tile holds every row (tiles_m == 1), one K slice, one of the tiles up to 128x64
                          // (the bias gradient of a hidden layer, out of the GEMM that produces that layer's gradient)
    // Gathered B (implicit im2col): when set, B(n, k) = B[b_gather_row[n] + b_gather_k[k]] instead of
    // B[k*b_rs + n*b_cs]; loaded through registers.  Launched as an MN-major B it takes 16-byte loads where four
    // consecutive n are contiguous in memory (b_gather_row strictly increasing), launched as a K-major B where
    // four consecutive k are (b_gather_k strictly increasing).
    const int32_t* b_gather_row; // [N]
    const int32_t* b_gather_k;   // [K]
    BatchDesc batch;
};

// The column sums of B beside the product (the BSUM instantiations of the kernels; a kernel argument of its own, so that
// the other instantiations keep their argument layout): out[n] += sum_k B(k, n) — the bias gradient of a Linear layer (the
// upstream gradient summed over its rows, tenmo/broadcast.mojo:66-88) out of the launch that computes the weight gradient
// X^T . dY, which streams dY as its B anyway.  One matrix (batch_count == 1); the workgroups of the first tile row do it.
struct BsumArgs {
    float* out;      // [N]
    float* partial;  // one-workgroup-per-tile launch with k_splits > 1: [k_splits][N], the sums of each K slice, added by the
                     // slice reduction; stream-K launch: [2 * workgroups][BN], the sums over each piece of a shared tile,
                     // added by the fix-up in the order of the tile's partial sums
};

// bias, ReLU and ReLU-backward mask on one finished element (i = flat index into the dense C)
__device__ __forceinline__ float epilogue_value(float v, const float* __restrict bias, const float* __restrict mask, int relu, int64_t i, int64_t col) {
    if (bias) v += bias[col];
    if (relu && !(v > 0.f)) v = 0.f;
    if (mask && !(mask[i] > 0.f)) v = 0.f;
    return v;
}

// tells the compiler that a pointer is the same in every lane (keeps it in scalar registers)
__device__ __forceinline__ const float* uniform_ptr(const float* p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (const float*)(uintptr_t)(((uint64_t)hi << 32) | lo);
}

// ---- one operand tile of ROWS x BK: global -> LDS ---------------------------------------------
// `row` indexes M for A and N for B; element(row, k) = base[row*rs + k*ks].
template <int ROWS, int MODE>
struct TileLoader {
    static constexpr int NCH = ROWS / 64; // 16-byte chunks per thread == direct loads per wavefront
    static constexpr int QPR = ROWS / 4;  // MN-major: chunks per k row
    static constexpr int KROWS_PER_WAVELOAD = 256 / ROWS > 0 ? 256 / ROWS : 1;
    f32x4 r[NCH];        // staging registers of the checked path
    // direct path: source of wave-load j = `origin` (same in every lane, lives in scalar registers)
    // + `lane_off[j]` bytes; one K step advances the origin by GEMM_BK * kstep elements
    const float* origin;
    uint32_t lane_off[NCH];
    int64_t kstep;

    // largest row pitch (K-major) / k pitch (MN-major), in elements, whose lane offsets fit 32 bits
    static constexpr int64_t MAX_DIRECT_PITCH = MODE == MNMAJOR_VEC ? (int64_t(1) << 25) : (int64_t(1) << 21);

    // Rows at or beyond the extent R are clamped onto valid rows: their products are never stored,
    // they only have to be readable.  (An MN-major operand moves 4 rows per 16-byte chunk, so a
    // ragged extent there needs R % 4 == 0; the caller checks, and that 0 <= pitch <= MAX_DIRECT_PITCH.)
    __device__ __forceinline__ void init_direct(const float* __restrict base, int64_t rs, int64_t ks, int64_t row0, int64_t k_begin, int64_t R, int lane, int wave) {
        if constexpr (MODE == MNMAJOR_VEC) {
#pragma unroll
            for (int j = 0; j < NCH; ++j) lane_off[j] = direct_lane_off_mnmajor<ROWS>(ks, row0, R, lane, wave * NCH + j);
            origin = uniform_ptr(base + k_begin * ks + row0);
            kstep = ks;
        } else {
#pragma unroll
            for (int j = 0; j < NCH; ++j) lane_off[j] = direct_lane_off_kmajor<ROWS>(rs, row0, R, lane, wave * NCH + j);
            origin = uniform_ptr(base + row0 * rs + k_begin);
            kstep = 1;
        }
    }

    // lane offsets of the last K step of a K that is no multiple of 16 (`k_valid` of its 16 k exist): see gemm_index.hpp
    __device__ __forceinline__ void tail_offsets(int64_t rs, int64_t ks, int64_t row0, int64_t R, int lane, int wave, int k_valid, uint32_t (&off)[NCH]) const {
#pragma unroll
        for (int j = 0; j < NCH; ++j)
            off[j] = MODE == MNMAJOR_VEC ? direct_lane_off_mnmajor<ROWS>(ks, row0, R, lane, wave * NCH + j, k_valid)
                                         : direct_lane_off_kmajor<ROWS>(rs, row0, R, lane, wave * NCH + j, k_valid);
    }

    // Wave-load j of the tile at K offset koff -> LDS tile `lds`, straight from global memory (direct_load_16B,
    // gfx950_asm.hpp: lane L writes bytes [16L, 16L+16) of that load's 1 KiB LDS block).  The callers wait for these
    // loads explicitly with s_waitcnt vmcnt(n).
    __device__ __forceinline__ void load_direct(float* lds, int64_t koff, int wave, int j) const { load_direct_at(lds, koff, wave, j, lane_off[j]); }
    // the same with the lane's byte offset given (the last K step of a ragged K uses tail_offsets)
    __device__ __forceinline__ void load_direct_at(float* lds, int64_t koff, int wave, int j, uint32_t lane_byte_off) const {
        static_assert(MODE != KMAJOR_GEN, "the generic loader has no direct path");
        direct_load_16B(lds, (uint32_t)((wave * NCH + j) * 1024), lane_byte_off, origin + koff * kstep);
    }

    // ---- register-staged path (generic strides, gathered operands, ragged MN-major tiles) --------
    // Per-thread source of chunk i as a 32-bit element offset from the operand's base, fixed for the
    // whole tile: the K loop only adds the step's offset.  Rows past the extent R are clamped onto the
    // last valid row (K-major forms: their products are never stored); an MN-major chunk moves 4 rows at
    // once and cannot be clamped, so `staged_ok` is false for a tile that has such a chunk — or whose
    // offsets do not fit 31 bits — and that tile takes the checked loads.
    // (Only the two vector forms take it: issuing a generic operand's 8-16 element loads together costs
    // 20-35 more registers, which spills next to the 256x128 accumulators and lowers the occupancy of
    // the 128-row tiles; measured slower than the checked loads, which issue one chunk at a time.)
    static constexpr bool STAGED_FAST = MODE != KMAJOR_GEN;
    uint32_t soff[NCH];
    uint32_t vec_mask;     // gathered MN-major: bit i = the 4 rows of chunk i are contiguous in memory
    bool staged_ok;

    __device__ __forceinline__ void init_staged(int64_t rs, int64_t ks, int64_t row0, int64_t R, int t, const int32_t* __restrict gather_row) {
        vec_mask = ~0u;
        if constexpr (!STAGED_FAST) {
            staged_ok = false;
        } else if constexpr (MODE == MNMAJOR_VEC) {
            staged_ok = row0 + ROWS <= R && R <= 0x7fffffffLL; // uniform over the workgroup
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int64_t row = row0 + 4 * ((t + GEMM_THREADS * i) % QPR);
                soff[i] = (uint32_t)row;
                if (staged_ok && gather_row) {
                    const int32_t o0 = gather_row[row];
                    if (gather_row[row + 3] - o0 != 3) vec_mask &= ~(1u << i); // offsets increase: a span of 3 means contiguous
                    soff[i] = (uint32_t)o0;
                }
            }
        } else if (gather_row) { // K-major gather: element (row, k) at base[gather_row[row] + gather_k[k]], rows clamped
            staged_ok = true;
#pragma unroll
            for (int i = 0; i < NCH; ++i) soff[i] = (uint32_t)gather_row[min(row0 + (t >> 2) + 64 * i, R - 1)];
        } else {
            staged_ok = rs >= 0 && (R - 1) * rs + 16 <= 0x7fffffffLL;
#pragma unroll
            for (int i = 0; i < NCH; ++i) soff[i] = (uint32_t)(min(row0 + (t >> 2) + 64 * i, R - 1) * rs + 4 * (t & 3));
        }
    }

    // One whole K step (k0 .. k0+15 all valid), no bounds checks.
    __device__ __forceinline__ void load_staged(const float* __restrict base, int64_t ks, int64_t row0, int64_t k0,
                                                const int32_t* __restrict gather_row, const int32_t* __restrict gather_k, int t) {
        if constexpr (!STAGED_FAST) {
            return;
        } else if constexpr (MODE == KMAJOR_VEC) {
            if (gather_row) {
                // this thread's four k of the step; gather_k is increasing, so a span of 3 means contiguous in memory
                const int32_t* __restrict gk = gather_k + k0 + 4 * (t & 3);
                const int32_t g0 = gk[0], g1 = gk[1], g2 = gk[2], g3 = gk[3];
                if (g3 - g0 == 3) {
#pragma unroll
                    for (int i = 0; i < NCH; ++i) r[i] = *reinterpret_cast<const f32x4_u*>(base + soff[i] + g0);
                } else {
#pragma unroll
                    for (int i = 0; i < NCH; ++i) {
                        const float* __restrict p = base + soff[i];
                        r[i] = f32x4{p[g0], p[g1], p[g2], p[g3]};
                    }
                }
                return;
            }
            const float* __restrict b0 = base + k0;
#pragma unroll
            for (int i = 0; i < NCH; ++i) r[i] = *reinterpret_cast<const f32x4_u*>(b0 + soff[i]);
        } else if constexpr (MODE == MNMAJOR_VEC) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int64_t k = k0 + (t + GEMM_THREADS * i) / QPR;
                if (gather_row) {
                    const float* pk = base + gather_k[k] + soff[i];
                    if (vec_mask >> i & 1) r[i] = *reinterpret_cast<const f32x4_u*>(pk);
                    else {
                        const int64_t row = row0 + 4 * ((t + GEMM_THREADS * i) % QPR);
                        const int32_t o0 = gather_row[row];
                        r[i] = f32x4{pk[0], pk[gather_row[row + 1] - o0], pk[gather_row[row + 2] - o0], pk[gather_row[row + 3] - o0]};
                    }
                } else {
                    r[i] = *reinterpret_cast<const f32x4_u*>(base + k * ks + soff[i]);
                }
            }
        }
    }

    // register-staged loads with every element checked against the extents (edge tiles, K tail,
    // generic strides)
    __device__ __forceinline__ void load_checked(const float* __restrict base, int64_t rs, int64_t ks,
                                                 int64_t row0, int64_t k0, int64_t R, int64_t K, int t,
                                                 const int32_t* __restrict gather_row = nullptr, const int32_t* __restrict gather_k = nullptr) {
        if constexpr (MODE == KMAJOR_VEC) {
            const int kq = t & 3;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int64_t row = row0 + (t >> 2) + 64 * i;
                const int64_t k = k0 + 4 * kq;
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (row < R && gather_row) { // K-major gather, element by element
                    const float* p = base + gather_row[row];
                    if (k + 0 < K) v.x = p[gather_k[k]];
                    if (k + 1 < K) v.y = p[gather_k[k + 1]];
                    if (k + 2 < K) v.z = p[gather_k[k + 2]];
                    if (k + 3 < K) v.w = p[gather_k[k + 3]];
                } else if (row < R) {
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
        } else if constexpr (MODE == MNMAJOR_VEC) {
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int c = t + GEMM_THREADS * i;
                const int64_t k = k0 + c / QPR;
                const int64_t row = row0 + 4 * (c % QPR);
                f32x4 v = {0.f, 0.f, 0.f, 0.f};
                if (k < K && gather_row) {
                    // element (row, k) at base[gather_row[row] + gather_k[k]]; gather_row is increasing, so four
                    // rows whose offsets span exactly 3 are contiguous in memory (one output row, stride 1)
                    const float* pk = base + gather_k[k];
                    if (row + 3 < R) {
                        const int32_t o0 = gather_row[row], o3 = gather_row[row + 3];
                        if (o3 - o0 == 3) v = *reinterpret_cast<const f32x4_u*>(pk + o0);
                        else v = f32x4{pk[o0], pk[gather_row[row + 1]], pk[gather_row[row + 2]], pk[o3]};
                    } else {
                        if (row + 0 < R) v.x = pk[gather_row[row]];
                        if (row + 1 < R) v.y = pk[gather_row[row + 1]];
                        if (row + 2 < R) v.z = pk[gather_row[row + 2]];
                    }
                } else if (k < K) {
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
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                const int c = t + GEMM_THREADS * i;
                *reinterpret_cast<f32x4*>(lds + (c / QPR) * ROWS + 4 * (c % QPR)) = r[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < NCH; ++i)
                *reinterpret_cast<f32x4*>(lds + kmajor_off((t >> 2) + 64 * i, t & 3)) = r[i];
        }
    }
};

// ---- LDS -> MFMA operand registers for one 8-wide k chunk ------------------------------------
// f[b][s]: operand of block b at MFMA step s.  `wave_row0` is the wave's first row in the tile.
// The fetch of one operand is frag_parts() LDS instructions; part p is one of them, so that the
// kernel can place them one by one between its MFMAs.
template <int MODE, int NBLK>
__device__ __forceinline__ constexpr int frag_parts() { return MODE == MNMAJOR_VEC ? 4 : NBLK; }

template <int ROWS, int MODE, int NBLK>
__device__ __forceinline__ void load_fragment_part(const float* __restrict lds, int wave_row0, int kc, int lane, float (&f)[NBLK][4], int p) {
    if constexpr (MODE == MNMAJOR_VEC) { // part = MFMA step s: one read feeds all NBLK blocks
        const int s = p;
        const float* q = lds + frag_off_mnmajor(ROWS, NBLK, wave_row0, kc, lane, s);
        if constexpr (NBLK == 4) {
            f32x4 v = *reinterpret_cast<const f32x4*>(q);
            f[0][s] = v.x; f[1][s] = v.y; f[2][s] = v.z; f[3][s] = v.w;
        } else if constexpr (NBLK == 2) {
            f32x2 v = *reinterpret_cast<const f32x2*>(q);
            f[0][s] = v.x; f[1][s] = v.y;
        } else {
            f[0][s] = q[0];
        }
    } else { // part = block b: one 16-byte read feeds its four MFMA steps
        const int b = p;
        f32x4 v = *reinterpret_cast<const f32x4*>(lds + frag_off_kmajor(wave_row0, kc, lane, b));
        f[b][0] = v.x; f[b][1] = v.y; f[b][2] = v.z; f[b][3] = v.w;
    }
}

template <int ROWS, int MODE, int NBLK>
__device__ __forceinline__ void load_fragments(const float* __restrict lds, int wave_row0, int kc, int lane, float (&f)[NBLK][4]) {
#pragma unroll
    for (int p = 0; p < frag_parts<MODE, NBLK>(); ++p) load_fragment_part<ROWS, MODE, NBLK>(lds, wave_row0, kc, lane, f, p);
}

// position inside the wave tile of MFMA index x (0..31) of block b
template <int MODE, int NBLK>
__device__ __forceinline__ int tile_pos(int b, int x) { return wave_tile_pos(MODE == MNMAJOR_VEC, NBLK, b, x); }

// s_waitcnt vmcnt(n) only (expcnt / lgkmcnt left unconstrained), gfx9 encoding
__device__ __forceinline__ constexpr int vmcnt_imm(int n) { return (n & 0xF) | (0x7 << 4) | (0xF << 8) | ((n >> 4) << 14); }

// workgroup barrier without the memory fence of __syncthreads(): the callers order their LDS
// traffic themselves (the direct loads are waited for with vmcnt, the reads happen after it)
__device__ __forceinline__ void bare_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// position of tile number `tid` (0 .. tiles_m*tiles_n-1) in the tile grid.
// Workgroup ids are dealt round-robin to the 8 XCDs (checked with HW_REG_XCC_ID), so with groups
// of 8 tile-rows each XCD keeps one tile-row of A hot in its L2 and streams B past it.
__device__ __forceinline__ void tile_coords(const GemmArgs& g, int64_t tile_id, int64_t& tile_m, int64_t& tile_n) {
    // tile ids are below 2^31: 32-bit divisions (a 64-bit one costs hundreds of instructions)
    constexpr uint32_t GROUP_M = 8;
    const uint32_t tid = (uint32_t)tile_id;
    // Fewer than 8 tile-rows: the tiles of one column block all go to the same XCD (ids that are equal mod 8), so
    // that a panel of B is fetched from memory by one L2 instead of by up to `tiles_m` of them (A, with so few
    // rows, is small).  The columns beyond the last multiple of 8 keep the plain column-major order.
    if ((uint32_t)g.tiles_m < GROUP_M && g.tiles_m > 1) {
        const uint32_t gsz = (uint32_t)g.tiles_m, cols8 = (uint32_t)g.tiles_n & ~7u, main_tiles = gsz * cols8;
        if (tid < main_tiles) {
            const uint32_t xcd = tid % 8, j = tid / 8, c = j / gsz;
            tile_m = j - c * gsz;
            tile_n = c * 8 + xcd;
        } else {
            const uint32_t r = tid - main_tiles, c = r / gsz;
            tile_m = r - c * gsz;
            tile_n = cols8 + c;
        }
        return;
    }
    const uint64_t per_group64 = (uint64_t)GROUP_M * (uint32_t)g.tiles_n;
    const uint32_t per_group = per_group64 > 0xffffffffull ? 0xffffffffu : (uint32_t)per_group64; // clamped: then group 0 holds every tile
    const uint32_t group = tid / per_group, in_group = tid - group * per_group;
    const uint32_t first_m = group * GROUP_M;
    const uint32_t gsz = min((uint32_t)g.tiles_m - first_m, GROUP_M);
    const uint32_t col = in_group / gsz;
    tile_m = first_m + (in_group - col * gsz);
    tile_n = col;
}

// The same for the one-workgroup-per-tile launch of the 256x128 tile, whose 64 resident workgroups per
// XCD (2 per CU) then form one block of 2 x 32 (or 4 x 16) tiles: the XCD's L2 fetches 2 (4) panels of A
// and 32 (16) of B per round instead of 1 and 64.  Measured at 8192^3: L2-miss traffic 9.2 GB -> 5.9 GB
// (6.2 GB for 4 x 16), run time unchanged (the kernel is bound by the matrix pipe); an 8 x 8 block has
// the least traffic on paper but measured 11.5 GB — eight A panels at a power-of-two row pitch thrash a
// few L2 sets.  Tile grids that do not divide into such blocks keep the order above.
template <int BM, int BN>
__device__ __forceinline__ void tile_coords_blocked(const GemmArgs& g, int64_t tid, int64_t& tile_m, int64_t& tile_n) {
    if constexpr (BM == 256 && BN == 128) {
        const uint32_t rn = g.tiles_n % 32 == 0 ? 32 : 16, rm = 64 / rn; // powers of two
        const uint32_t bm_count = (uint32_t)g.tiles_m / rm, bn_count = (uint32_t)g.tiles_n / rn;
        if (g.tiles_m % rm == 0 && g.tiles_n % rn == 0 && (bm_count * bn_count) % 8 == 0) {
            const uint32_t t32 = (uint32_t)tid;
            const uint32_t xcd = t32 % 8, j = t32 / 8, round = j / 64, q = j % 64;
            const uint32_t block = round * 8 + xcd; // the 8 XCDs work on 8 neighbouring blocks at a time
            const uint32_t block_m = block / bn_count;
            tile_m = block_m * rm + q % rm;
            tile_n = (block - block_m * bn_count) * rn + q / rm;
            return;
        }
    }
    tile_coords(g, tid, tile_m, tile_n);
}

// where a finished tile goes: element (row, col) of the product is written to
// base[(row - row0) * ld + (col - col0)]
struct TileDest {
    float* base;
    int64_t ld, row0, col0;
    bool accumulate; // += instead of =
    bool fused;      // apply g.bias / g.relu / g.mask (never together with accumulate)
};

// BSUM kernels: where the sum over a gemm_tile call's K range of B(k, col) goes: out[col - col0] (out null: nowhere)
struct BsumDest {
    float* out;
    int64_t col0;
    bool add; // += instead of =
};

// One tile of C over the K range [k_begin, k_end) (k_begin a multiple of GEMM_BK), by the whole
// workgroup.  The three LDS stages are the caller's; on return every wavefront has left them.
template <int BM, int BN, int AMODE, int BMODE, bool BSUM = false>
__device__ __forceinline__ void gemm_tile(const GemmArgs& g, float* stage0, float* stage1, float* stage2,
                                          int64_t batch, int64_t tile_m, int64_t tile_n, int64_t k_begin, int64_t k_end, const TileDest dst,
                                          const int64_t a_extra = 0, const int64_t b_extra = 0, // (element offsets on top of the batch's)
                                          const BsumDest bsum = BsumDest{nullptr, 0, false}) {
    constexpr int TM = BM / 2, TN = BN / 2;     // wave tile (2x2 waves)
    constexpr int MB = TM / 32, NB = TN / 32;   // 32x32 MFMA blocks per wave tile
    constexpr int A_FLOATS = BM * GEMM_BK;
    constexpr bool DIRECT = (AMODE != KMAJOR_GEN) && (BMODE != KMAJOR_GEN);

    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int64_t m0 = tile_m * BM, n0 = tile_n * BN;

    int64_t a_boff, b_boff;
    batch_offsets(g.batch, batch, a_boff, b_boff);
    const float* __restrict Ab = g.A + a_boff + a_extra;
    const float* __restrict Bb = g.B + b_boff + b_extra;

    // operand strides in (row, k) form
    const int64_t a_row_s = g.a_rs, a_k_s = g.a_cs;   // A(m,k)
    const int64_t b_row_s = g.b_cs, b_k_s = g.b_rs;   // B(n,k) = Bmem[k*b_rs + n*b_cs]

    const int64_t nk = (k_end > k_begin) ? (k_end - k_begin + GEMM_BK - 1) / GEMM_BK : 0;

    f32x16 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    TileLoader<BM, AMODE> la;
    TileLoader<BN, BMODE> lb;

    // BSUM: every B fragment that feeds the MFMAs is also added up per lane — a lane always holds the same columns
    // (block j, column lane & 31; the two halves of the wavefront hold different k), so the sums stay in registers for
    // the whole K range and are combined once, in the epilogue.  Every wavefront does it (no branch in the K loop; the
    // vector ALU is idle beside the MFMAs), the ones of the first wave row store.
    float bs[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) bs[j] = 0.f;
    auto add_b_fragments = [&](const float (&fb)[NB][4]) {
        if constexpr (BSUM) {
#pragma unroll
            for (int j = 0; j < NB; ++j)
#pragma unroll
                for (int s = 0; s < 4; ++s) bs[j] += fb[j][s];
        }
    };

    auto mfma_chunk = [&](const float (&fa)[MB][4], const float (&fb)[NB][4]) {
        add_b_fragments(fb);
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
    };
    auto compute = [&](const float* __restrict st) {
#pragma unroll
        for (int kc = 0; kc < GEMM_BK / 8; ++kc) {
            float fa[MB][4], fb[NB][4];
            load_fragments<BM, AMODE, MB>(st, wm * TM, kc, lane, fa);
            load_fragments<BN, BMODE, NB>(st + A_FLOATS, wn * TN, kc, lane, fb);
            mfma_chunk(fa, fb);
        }
    };

    int64_t done = 0; // K steps finished by the direct pipeline
    if constexpr (DIRECT) {
        // ---- three-stage direct-to-LDS ring --------------------------------------------------
        // Ragged tiles stay on this path as long as clamping rows is enough; row / k pitches must be
        // non-negative and small enough for 32-bit lane offsets.
        using LA = TileLoader<BM, AMODE>;
        using LB = TileLoader<BN, BMODE>;
        const int64_t a_pitch = AMODE == KMAJOR_VEC ? a_row_s : a_k_s, b_pitch = BMODE == KMAJOR_VEC ? b_row_s : b_k_s;
        const bool a_ok = ((m0 + BM <= g.M) || AMODE == KMAJOR_VEC || (g.M % 4 == 0 && g.M >= 4)) && a_pitch >= 0 && a_pitch <= LA::MAX_DIRECT_PITCH;
        const bool b_ok = ((n0 + BN <= g.N) || BMODE == KMAJOR_VEC || (g.N % 4 == 0 && g.N >= 4)) && b_pitch >= 0 && b_pitch <= LB::MAX_DIRECT_PITCH;
        const int64_t nfast = (a_ok && b_ok && !g.b_gather_row) ? (k_end - k_begin) / GEMM_BK : 0; // a gathered B is register-staged
        if (nfast > 0) {
            constexpr int NLA = LA::NCH, NL = LA::NCH + LB::NCH;  // direct loads per wave per K step
            constexpr int PA = frag_parts<AMODE, MB>(), PB = frag_parts<BMODE, NB>(); // LDS reads per chunk
            constexpr int NMFMA = 4 * MB * NB;                    // MFMAs per chunk
            constexpr int PER_SLOT = (PA + PB + NL + NMFMA - 1) / NMFMA;
            la.init_direct(Ab, a_row_s, a_k_s, m0, k_begin, g.M, lane, wave);
            lb.init_direct(Bb, b_row_s, b_k_s, n0, k_begin, g.N, lane, wave);
            // direct load number j (A's first, then B's) of K step `it` into stage `st`
            auto issue_one = [&](float* st, int64_t it, int j) {
                if (j < NLA) la.load_direct(st, it * GEMM_BK, wave, j);
                else lb.load_direct(st + A_FLOATS, it * GEMM_BK, wave, j - NLA);
            };
            auto issue = [&](float* st, int64_t it) {
#pragma unroll
                for (int j = 0; j < NL; ++j) issue_one(st, it, j);
            };
            // operand fetch number p (A's parts first, then B's) of chunk kc of stage `st`
            auto fetch_one = [&](const float* st, int kc, float (&fa)[MB][4], float (&fb)[NB][4], int p) {
                if (p < PA) load_fragment_part<BM, AMODE, MB>(st, wm * TM, kc, lane, fa, p);
                else load_fragment_part<BN, BMODE, NB>(st + A_FLOATS, wn * TN, kc, lane, fb, p - PA);
            };
            float fa0[MB][4], fb0[NB][4], fa1[MB][4], fb1[NB][4];
            issue(stage0, 0);
            if (nfast > 1) {
                issue(stage1, 1);
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(NL));
            } else {
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            }
            bare_barrier();
            load_fragments<BM, AMODE, MB>(stage0, wm * TM, 0, lane, fa0);
            load_fragments<BN, BMODE, NB>(stage0 + A_FLOATS, wn * TN, 0, lane, fb0);

            // The MFMAs of one chunk with the other instructions of the pipeline placed between
            // them: after MFMA n, `slot(n * PER_SLOT + u)` runs for u < PER_SLOT.  A wavefront then
            // never leaves the matrix pipe idle for longer than one LDS or memory instruction takes
            // to issue, so the loop runs at full rate even with a single wavefront per SIMD
            // (measured at 8192^3: all loads and fetches ahead of the MFMAs 142 TFLOP/s, interleaved 153).
            auto mfma_interleaved = [&](const float (&fa)[MB][4], const float (&fb)[NB][4], auto&& slot) {
                add_b_fragments(fb);
                int n = 0;
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int i = 0; i < MB; ++i)
#pragma unroll
                        for (int j = 0; j < NB; ++j) {
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int u = 0; u < PER_SLOT; ++u) slot(n * PER_SLOT + u);
                            __builtin_amdgcn_sched_barrier(0);
                            ++n;
                        }
            };
            // One K step: `cur` holds step it, `nxt` step it+1 (in flight), `ld` receives step it+2.
            // `full` = std::true_type in the steady state (both later steps exist: no conditions in
            // the body, so the wait counts the compiler derives are exact); std::false_type for the
            // last steps.
            auto step = [&](auto full, float* cur, float* nxt, float* ld, int64_t it) {
                constexpr bool FULL = decltype(full)::value;
                const bool have_ld = FULL || it + 2 < nfast, have_next = FULL || it + 1 < nfast;
                // chunk 0; behind its MFMAs the operand fetch of chunk 1 and the direct loads of step it+2
                mfma_interleaved(fa0, fb0, [&](int p) {
                    if (p < PA + PB) fetch_one(cur, 1, fa1, fb1, p);
                    else if (p < PA + PB + NL && have_ld) issue_one(ld, it + 2, p - PA - PB);
                });
                if (have_next) {
                    if (have_ld) __builtin_amdgcn_s_waitcnt(vmcnt_imm(NL)); // step it+1 has landed
                    else __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
                    bare_barrier();
                }
                __builtin_amdgcn_sched_barrier(0);
                // chunk 1; behind its MFMAs the operand fetch of the next step's chunk 0
                mfma_interleaved(fa1, fb1, [&](int p) {
                    if (p < PA + PB && have_next) fetch_one(nxt, 0, fa0, fb0, p);
                });
            };
            int64_t it = 0;
            for (; it + 4 < nfast; it += 3) { // steps it .. it+2 all have two successors
                step(std::true_type{}, stage0, stage1, stage2, it);
                step(std::true_type{}, stage1, stage2, stage0, it + 1);
                step(std::true_type{}, stage2, stage0, stage1, it + 2);
            }
            for (; it < nfast; it += 3) { // the last one to four steps
                step(std::false_type{}, stage0, stage1, stage2, it);
                if (it + 1 >= nfast) break;
                step(std::false_type{}, stage1, stage2, stage0, it + 1);
                if (it + 2 >= nfast) break;
                step(std::false_type{}, stage2, stage0, stage1, it + 2);
            }
            done = nfast;
            __syncthreads(); // every wave has left the ring before the tail reuses stage0/stage1
        }
    }

    // ---- edge tiles, the K tail, generic strides: register-staged checked loads, two stages ----
    if (done < nk) {
        constexpr bool STAGED_FAST = TileLoader<BM, AMODE>::STAGED_FAST && TileLoader<BN, BMODE>::STAGED_FAST;
        if constexpr (STAGED_FAST) {
            la.init_staged(a_row_s, a_k_s, m0, g.M, t, nullptr);
            lb.init_staged(b_row_s, b_k_s, n0, g.N, t, g.b_gather_row);
        }
        // a whole K step goes through the unchecked loads; the K tail and ragged MN-major tiles through the checked ones
        auto load_a_into = [&](TileLoader<BM, AMODE>& l, int64_t k0) {
            if (STAGED_FAST && l.staged_ok && k0 + GEMM_BK <= k_end) l.load_staged(Ab, a_k_s, m0, k0, nullptr, nullptr, t);
            else l.load_checked(Ab, a_row_s, a_k_s, m0, k0, g.M, k_end, t);
        };
        auto load_b_into = [&](TileLoader<BN, BMODE>& l, int64_t k0) {
            if (STAGED_FAST && l.staged_ok && k0 + GEMM_BK <= k_end) l.load_staged(Bb, b_k_s, n0, k0, g.b_gather_row, g.b_gather_k, t);
            else l.load_checked(Bb, b_row_s, b_k_s, n0, k0, g.N, k_end, t, g.b_gather_row, g.b_gather_k);
        };
        auto load_a = [&](int64_t k0) { load_a_into(la, k0); };
        auto load_b = [&](int64_t k0) { load_b_into(lb, k0); };
        if constexpr (BM * BN <= 64 * 64 && STAGED_FAST) {
            // (64x64 only: the second register set costs the 128x64 tile a resident workgroup per CU, measured a loss there)
            // Two LDS stages and two sets of staging registers: the loads of step it+2 are issued at the top of step it
            // and go to LDS in the middle of step it+1, so that they have a step and a half to land (a gathered operand
            // needs a table lookup and then the load: with one set, in flight for half a step only, the small tiles were
            // bound by that latency).  The barrier sits in the middle of a step as in the direct ring: behind the first
            // half's MFMAs the operand fetch of the second half, then the next step's registers go to the other stage,
            // barrier, and behind the second half's MFMAs the operand fetch of the next step's first half.
            constexpr int PA2 = frag_parts<AMODE, MB>(), PB2 = frag_parts<BMODE, NB>();
            constexpr int NMFMA2 = 4 * MB * NB;
            constexpr int PER_SLOT2 = (PA2 + PB2 + NMFMA2 - 1) / NMFMA2;
            auto fetch2 = [&](const float* st, int kc, float (&fa)[MB][4], float (&fb)[NB][4], int p) {
                if (p < PA2) load_fragment_part<BM, AMODE, MB>(st, wm * TM, kc, lane, fa, p);
                else if (p < PA2 + PB2) load_fragment_part<BN, BMODE, NB>(st + A_FLOATS, wn * TN, kc, lane, fb, p - PA2);
            };
            auto mfma2 = [&](const float (&fa)[MB][4], const float (&fb)[NB][4], auto&& slot) {
                add_b_fragments(fb);
                int n = 0;
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int i = 0; i < MB; ++i)
#pragma unroll
                        for (int j = 0; j < NB; ++j) {
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int u = 0; u < PER_SLOT2; ++u) slot(n * PER_SLOT2 + u);
                            __builtin_amdgcn_sched_barrier(0);
                            ++n;
                        }
            };
            TileLoader<BM, AMODE> la2; // the same per-thread offsets, a second set of staging registers
            TileLoader<BN, BMODE> lb2;
            la2.init_staged(a_row_s, a_k_s, m0, g.M, t, nullptr);
            lb2.init_staged(b_row_s, b_k_s, n0, g.N, t, g.b_gather_row);
            float ga0[MB][4], gb0[NB][4], ga1[MB][4], gb1[NB][4];
            const int64_t kb = k_begin + done * GEMM_BK;
            load_a_into(la, kb);
            load_b_into(lb, kb);
            la.store(stage0, t);
            lb.store(stage0 + A_FLOATS, t);
            if (done + 1 < nk) { load_a_into(la, kb + GEMM_BK); load_b_into(lb, kb + GEMM_BK); } // step 1 into the first set
            __syncthreads();
            load_fragments<BM, AMODE, MB>(stage0, wm * TM, 0, lane, ga0);
            load_fragments<BN, BMODE, NB>(stage0 + A_FLOATS, wn * TN, 0, lane, gb0);
            // one K step: `held` holds step it+1 (loaded a step ago), `ahead` receives step it+2
            auto step = [&](TileLoader<BM, AMODE>& a_held, TileLoader<BN, BMODE>& b_held, TileLoader<BM, AMODE>& a_ahead, TileLoader<BN, BMODE>& b_ahead,
                            float* cur, float* nxt, int64_t it) {
                const bool more = it + 1 < nk;
                if (it + 2 < nk) {
                    const int64_t k0 = k_begin + (it + 2) * GEMM_BK;
                    load_a_into(a_ahead, k0);
                    load_b_into(b_ahead, k0);
                }
                mfma2(ga0, gb0, [&](int p) { fetch2(cur, 1, ga1, gb1, p); });
                if (more) {
                    a_held.store(nxt, t);
                    b_held.store(nxt + A_FLOATS, t);
                    __syncthreads();
                }
                mfma2(ga1, gb1, [&](int p) { if (more) fetch2(nxt, 0, ga0, gb0, p); });
            };
            int64_t it = done;
            for (; it + 1 < nk; it += 2) {
                step(la, lb, la2, lb2, stage0, stage1, it);
                step(la2, lb2, la, lb, stage1, stage0, it + 1);
            }
            if (it < nk) step(la, lb, la2, lb2, stage0, stage1, it);
            __syncthreads();
        } else if constexpr (BM * BN <= 128 * 128 && STAGED_FAST) {
            // Two LDS stages; the barrier sits in the middle of a step (as in the direct ring): behind the first half's
            // MFMAs the operand fetch of the second half, then the next step's registers go to the other stage, barrier,
            // and behind the second half's MFMAs the operand fetch of the next step's first half.
            constexpr int PA2 = frag_parts<AMODE, MB>(), PB2 = frag_parts<BMODE, NB>();
            constexpr int NMFMA2 = 4 * MB * NB;
            constexpr int PER_SLOT2 = (PA2 + PB2 + NMFMA2 - 1) / NMFMA2;
            auto fetch2 = [&](const float* st, int kc, float (&fa)[MB][4], float (&fb)[NB][4], int p) {
                if (p < PA2) load_fragment_part<BM, AMODE, MB>(st, wm * TM, kc, lane, fa, p);
                else if (p < PA2 + PB2) load_fragment_part<BN, BMODE, NB>(st + A_FLOATS, wn * TN, kc, lane, fb, p - PA2);
            };
            auto mfma2 = [&](const float (&fa)[MB][4], const float (&fb)[NB][4], auto&& slot) {
                add_b_fragments(fb);
                int n = 0;
#pragma unroll
                for (int s = 0; s < 4; ++s)
#pragma unroll
                    for (int i = 0; i < MB; ++i)
#pragma unroll
                        for (int j = 0; j < NB; ++j) {
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i][s], fb[j][s], acc[i][j], 0, 0, 0);
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int u = 0; u < PER_SLOT2; ++u) slot(n * PER_SLOT2 + u);
                            __builtin_amdgcn_sched_barrier(0);
                            ++n;
                        }
            };
            float ga0[MB][4], gb0[NB][4], ga1[MB][4], gb1[NB][4];
            load_a(k_begin + done * GEMM_BK);
            load_b(k_begin + done * GEMM_BK);
            la.store(stage0, t);
            lb.store(stage0 + A_FLOATS, t);
            __syncthreads();
            load_fragments<BM, AMODE, MB>(stage0, wm * TM, 0, lane, ga0);
            load_fragments<BN, BMODE, NB>(stage0 + A_FLOATS, wn * TN, 0, lane, gb0);
            for (int64_t it = done; it < nk; ++it) {
                float* cur = ((it - done) & 1) ? stage1 : stage0;
                float* nxt = ((it - done) & 1) ? stage0 : stage1;
                const bool more = (it + 1 < nk);
                if (more) {
                    const int64_t k0 = k_begin + (it + 1) * GEMM_BK;
                    load_a(k0);
                    load_b(k0);
                }
                mfma2(ga0, gb0, [&](int p) { fetch2(cur, 1, ga1, gb1, p); });
                if (more) {
                    la.store(nxt, t);
                    lb.store(nxt + A_FLOATS, t);
                    __syncthreads();
                }
                mfma2(ga1, gb1, [&](int p) { if (more) fetch2(nxt, 0, ga0, gb0, p); });
            }
            __syncthreads();
        } else { // plain two-stage loop: the 256x128 accumulators leave no registers for a second set of operand fragments,
                 // and the element loads of a generic operand need the whole step to land (measured 15 % slower with the
                 // barrier mid-step)
            load_a(k_begin + done * GEMM_BK);
            load_b(k_begin + done * GEMM_BK);
            la.store(stage0, t);
            lb.store(stage0 + A_FLOATS, t);
            __syncthreads();
            for (int64_t it = done; it < nk; ++it) {
                float* cur = ((it - done) & 1) ? stage1 : stage0;
                float* nxt = ((it - done) & 1) ? stage0 : stage1;
                const bool more = (it + 1 < nk);
                if (more) {
                    const int64_t k0 = k_begin + (it + 1) * GEMM_BK;
                    load_a(k0);
                    load_b(k0);
                }
                compute(cur);
                if (more) {
                    la.store(nxt, t);
                    lb.store(nxt + A_FLOATS, t);
                }
                __syncthreads();
            }
        }
    }

    // ---- epilogue ----
    const bool accumulate = dst.accumulate;
    const bool fused = dst.fused && (g.bias != nullptr || g.mask != nullptr || g.relu != 0);
    const float* __restrict mask = g.mask ? g.mask + batch * g.M * g.N : nullptr;
    const int h = lane >> 5, x = lane & 31;
    constexpr bool COLSUM = BM * BN <= 128 * 64; // the larger tiles have no registers to spare for it
    const bool colsum = COLSUM && g.colsum != nullptr && dst.fused;
    float cs[NB]; // this lane's part of the column sums
#pragma unroll
    for (int j = 0; j < NB; ++j) cs[j] = 0.f;
#pragma unroll
    for (int i = 0; i < MB; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int ip = 8 * (e >> 2) + 4 * h + (e & 3); // MFMA row of accumulator element e
            const int64_t row = m0 + wm * TM + tile_pos<AMODE, MB>(i, ip);
            if (row >= g.M) continue;
            float* crow = dst.base + (row - dst.row0) * dst.ld - dst.col0;
            float val[NB]; // the finished sums of this row, fused epilogue applied (never combined with accumulate)
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                val[j] = acc[i][j][e];
                if (fused) {
                    const int64_t col = n0 + wn * TN + tile_pos<BMODE, NB>(j, x);
                    if (col < g.N) val[j] = epilogue_value(val[j], g.bias, mask, g.relu, row * g.N + col, g.bias_rows ? row : col);
                }
                if constexpr (COLSUM) { if (colsum) cs[j] += val[j]; }
            }
            if constexpr (BMODE == MNMAJOR_VEC && NB > 1) {
                const int64_t col = n0 + wn * TN + NB * x;
                if (col + NB <= g.N) {
                    if constexpr (NB == 4) {
                        f32x4 v = {val[0], val[1], val[2], val[3]};
                        if (accumulate) v += *reinterpret_cast<const f32x4_u*>(crow + col);
                        *reinterpret_cast<f32x4_u*>(crow + col) = v;
                    } else {
                        f32x2 v = {val[0], val[1]};
                        if (accumulate) v += *reinterpret_cast<const f32x2_u*>(crow + col);
                        *reinterpret_cast<f32x2_u*>(crow + col) = v;
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < NB; ++j)
                        if (col + j < g.N) crow[col + j] = accumulate ? crow[col + j] + val[j] : val[j];
                }
            } else {
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const int64_t col = n0 + wn * TN + tile_pos<BMODE, NB>(j, x);
                    if (col < g.N) crow[col] = accumulate ? crow[col] + val[j] : val[j];
                }
            }
        }
    }
    if constexpr (BSUM) {
        if (bsum.out != nullptr) { // uniform over the workgroup
#pragma unroll
            for (int j = 0; j < NB; ++j) bs[j] += __shfl_xor(bs[j], 32); // the two halves of a wavefront hold different k
            if (wm == 0 && h == 0) {
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const int64_t col = n0 + wn * TN + tile_pos<BMODE, NB>(j, x);
                    if (col < g.N) {
                        float* p = bsum.out + (col - bsum.col0);
                        *p = bsum.add ? *p + bs[j] : bs[j];
                    }
                }
            }
        }
    }
    if constexpr (COLSUM) {
        if (colsum) { // uniform over the workgroup; the LDS stages are free: every wave has left the K loop
            float* red = stage0;
#pragma unroll
            for (int j = 0; j < NB; ++j) cs[j] += __shfl_xor(cs[j], 32); // the two halves of a wavefront hold different rows
            if (wm == 1 && h == 0) {
#pragma unroll
                for (int j = 0; j < NB; ++j) red[wn * TN + tile_pos<BMODE, NB>(j, x)] = cs[j];
            }
            __syncthreads();
            if (wm == 0 && h == 0) {
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    const int local = wn * TN + tile_pos<BMODE, NB>(j, x);
                    if (n0 + local < g.N) g.colsum[batch * g.N + n0 + local] = cs[j] + red[local];
                }
            }
        }
    }
}

// One workgroup per tile (and per K slice when g.k_splits > 1): tile number `pid` (batches included) and K slice `slice`.
template <int BM, int BN, int AMODE, int BMODE, bool BSUM = false>
__device__ __forceinline__ void gemm_workgroup(const GemmArgs& g, float* stage0, float* stage1, float* stage2, uint32_t pid, uint32_t slice,
                                               const BsumArgs bsum = BsumArgs{}) {
    const uint32_t tiles = (uint32_t)g.tiles_m * (uint32_t)g.tiles_n; // the grid, batches included, is below 2^31
    uint32_t batch32;
    int64_t tile_m, tile_n;
    // With 8 or more batches each XCD (workgroup id mod 8) takes whole batches, so that a batch's operands are
    // fetched by one L2 only (attention P.V: V is otherwise read by all eight); the batches beyond the last
    // multiple of 8 keep the plain order.
    const uint32_t by_xcd = ((uint32_t)g.batch_count & ~7u) * tiles;
    if (pid < by_xcd) {
        const uint32_t xcd = pid % 8, j = pid / 8, bl = j / tiles;
        batch32 = bl * 8 + xcd;
        tile_coords(g, j - bl * tiles, tile_m, tile_n);
    } else {
        batch32 = pid / tiles;
        tile_coords_blocked<BM, BN>(g, pid - batch32 * tiles, tile_m, tile_n);
    }
    const int64_t batch = batch32;

    int64_t k_begin = 0, k_end = g.K;
    TileDest dst;
    dst.ld = g.N; dst.row0 = 0; dst.col0 = 0;
    if (g.k_splits > 1) { // partial sums of this K slice; the slice reduction finishes them
        k_begin = (int64_t)slice * g.k_per_split;
        k_end = min(g.K, k_begin + g.k_per_split);
        dst.base = g.partial + ((int64_t)slice * g.batch_count + batch) * g.M * g.N;
        dst.accumulate = false; dst.fused = false;
    } else {
        dst.base = g.C + batch * g.M * g.N;
        dst.accumulate = g.accumulate != 0; dst.fused = true;
    }
    if constexpr (BSUM) {
        BsumDest bd{nullptr, 0, false};
        if (tile_m == 0 && batch == 0) { // the first tile row sees every element of its columns of B once
            if (g.k_splits > 1) { bd.out = bsum.partial + (int64_t)slice * g.N; bd.add = false; }
            else { bd.out = bsum.out; bd.add = true; }
        }
        gemm_tile<BM, BN, AMODE, BMODE, true>(g, stage0, stage1, stage2, batch, tile_m, tile_n, k_begin, k_end, dst, 0, 0, bd);
    } else {
        gemm_tile<BM, BN, AMODE, BMODE>(g, stage0, stage1, stage2, batch, tile_m, tile_n, k_begin, k_end, dst);
    }
}

template <int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_mfma_kernel(const GemmArgs g) {
    constexpr int STAGE_FLOATS = (BM + BN) * GEMM_BK;
    constexpr bool DIRECT = (AMODE != KMAJOR_GEN) && (BMODE != KMAJOR_GEN);
    // three separate objects: the compiler can then tell that a direct load into one stage does
    // not alias the operand fetch from another
    __shared__ __attribute__((aligned(1024))) float stage0[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage1[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage2[DIRECT ? STAGE_FLOATS : 4];
    gemm_workgroup<BM, BN, AMODE, BMODE>(g, stage0, stage1, stage2, blockIdx.x, blockIdx.y);
}

// The same launch with the column sums of B added up beside the product (BsumArgs; vector operand forms).
template <int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_mfma_bsum_kernel(const GemmArgs g, const BsumArgs bsum) {
    constexpr int STAGE_FLOATS = (BM + BN) * GEMM_BK;
    __shared__ __attribute__((aligned(1024))) float stage0[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage1[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage2[STAGE_FLOATS];
    gemm_workgroup<BM, BN, AMODE, BMODE, true>(g, stage0, stage1, stage2, blockIdx.x, blockIdx.y, bsum);
}

// Batch dimensions that a product is SUMMED over (the gradient of a parent that was broadcast along them,
// tenmo/matmul.mojo:115-135 with sum_over_broadcasted_axes).  `dims` holds the reduced dimensions only.
struct BatchReduce {
    BatchDesc dims;
    int64_t count; // product of dims.shape
};

// C[kept batch] (+)= sum over the reduced batch dimensions of A[kept, reduced] . B[kept, reduced]: one workgroup per tile of
// a kept batch (g.batch and g.batch_count describe the kept dimensions only; one K slice, no fused epilogue).  The
// workgroup runs the tile once per index of the reduced dimensions, each round adding onto what the round before stored
// (the same lanes touch the same elements, which stay in the L2): the gradient of a broadcast parent without a batched
// intermediate, without a reduction pass, and summed in a fixed order.
template <int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_reduce_kernel(const GemmArgs g, const BatchReduce red) {
    constexpr int STAGE_FLOATS = (BM + BN) * GEMM_BK;
    __shared__ __attribute__((aligned(1024))) float stage0[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage1[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage2[STAGE_FLOATS];
    const uint32_t tiles = (uint32_t)g.tiles_m * (uint32_t)g.tiles_n;
    const uint32_t batch32 = blockIdx.x / tiles;
    int64_t tile_m, tile_n;
    tile_coords(g, blockIdx.x - batch32 * tiles, tile_m, tile_n);
    const int64_t batch = batch32;
    TileDest dst;
    dst.ld = g.N; dst.row0 = 0; dst.col0 = 0;
    dst.base = g.C + batch * g.M * g.N;
    dst.fused = false;
    const uint32_t rounds = (uint32_t)red.count; // (below 2^31: it is a factor of the result's batch count)
    for (uint32_t r = 0; r < rounds; ++r) {
        int64_t a_roff, b_roff;
        batch_offsets(red.dims, r, a_roff, b_roff);
        dst.accumulate = r > 0 || g.accumulate != 0;
        gemm_tile<BM, BN, AMODE, BMODE>(g, stage0, stage1, stage2, batch, tile_m, tile_n, 0, g.K, dst, a_roff, b_roff);
    }
}

// Two independent products in one launch (both with one K slice and vector operand forms): workgroups below `first_count`
// work on g0, the others on g1.  For small products that a dependent-launch latency of about 5 us each would dominate
// (the weight gradient of a layer and the gradient passed to the layer below both consume the same upstream gradient).
template <int BM, int BN, int AMODE0, int BMODE0, int AMODE1, int BMODE1>
__global__ __launch_bounds__(GEMM_THREADS, 2) void gemm_pair_kernel(const GemmArgs g0, const GemmArgs g1, uint32_t first_count) {
    constexpr int STAGE_FLOATS = (BM + BN) * GEMM_BK;
    __shared__ __attribute__((aligned(1024))) float stage0[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage1[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage2[STAGE_FLOATS];
    if (blockIdx.x < first_count) gemm_workgroup<BM, BN, AMODE0, BMODE0>(g0, stage0, stage1, stage2, blockIdx.x, 0);
    else gemm_workgroup<BM, BN, AMODE1, BMODE1>(g1, stage0, stage1, stage2, blockIdx.x - first_count, 0);
}

// ---- stream-K --------------------------------------------------------------------------------
// A persistent grid.  The first `dp_tiles` tiles (a multiple of the grid size) are taken whole, one
// per workgroup and round: workgroup w works on tile round * grid + w, so the workgroups that run side
// by side work on neighbouring tiles and share operand panels in L2, exactly as in the one-tile-per-
// workgroup launch.  The work of the remaining tiles is cut into K steps ("iterations": tile-major,
// K-minor) and every workgroup takes an equal contiguous run of them, so the chip stays full whatever
// the tile count.  A workgroup whose run covers a whole tile stores it as usual; the pieces of a tile
// that is shared between workgroups go to compact partial tiles (two slots per workgroup: slot 2w for
// a piece that starts inside the tile, 2w+1 for one that starts at its beginning) and
// streamk_fixup_kernel adds them in workgroup order — deterministic, no spinning.
struct StreamKArgs {
    int64_t dp_tiles; // tiles (batches included) stored whole, round-robin over the grid
    int64_t total;    // iterations of the shared part = (tiles - dp_tiles) * nks
    int64_t per_wg;   // iterations per workgroup
    int64_t nks;      // K steps per tile
    float* partial;   // [2 * workgroups][BM * BN]
};

// (the small tiles must keep to the registers of four workgroups per CU, as their one-tile-per-workgroup kernels do)
template <int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(GEMM_THREADS, (BM * BN <= 128 * 64 ? 4 : 2)) void gemm_streamk_kernel(const GemmArgs g, const StreamKArgs sk) {
    constexpr int STAGE_FLOATS = (BM + BN) * GEMM_BK;
    constexpr bool DIRECT = (AMODE != KMAJOR_GEN) && (BMODE != KMAJOR_GEN);
    __shared__ __attribute__((aligned(1024))) float stage0[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage1[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage2[DIRECT ? STAGE_FLOATS : 4];
    const uint32_t tiles = (uint32_t)g.tiles_m * (uint32_t)g.tiles_n; // tile ids, batches included, are below 2^31
    // (every count of the schedule is below 2^31 — the host refuses larger ones — and is kept in 32 bits: the persistent
    // loop's state lives in scalar registers beside the tile function's, which are nearly all in use)
    const uint32_t w = blockIdx.x, nks = (uint32_t)sk.nks, dp_tiles = (uint32_t)sk.dp_tiles;
    uint32_t whole = blockIdx.x; // next tile of the data-parallel part
    uint32_t it = w * (uint32_t)sk.per_wg;
    const uint32_t end = min((uint32_t)sk.total, it + (uint32_t)sk.per_wg);
    for (;;) { // one call site for gemm_tile: the function is large
        uint32_t gt, k0, k1;
        if (whole < dp_tiles) {
            gt = whole; k0 = 0; k1 = nks;
            whole += gridDim.x;
        } else if (it < end) {
            const uint32_t st = it / nks; // shared tile number
            k0 = it - st * nks;
            k1 = min(nks, k0 + (end - it));
            gt = dp_tiles + st;
            it += k1 - k0;
        } else {
            break;
        }
        const uint32_t batch32 = gt / tiles;
        const int64_t batch = batch32;
        int64_t tile_m, tile_n;
        tile_coords_blocked<BM, BN>(g, gt - batch32 * tiles, tile_m, tile_n); // one numbering for both parts and the fix-up
        TileDest dst;
        if (k0 == 0 && k1 == nks) {
            dst.base = g.C + batch * g.M * g.N; dst.ld = g.N; dst.row0 = 0; dst.col0 = 0;
            dst.accumulate = g.accumulate != 0; dst.fused = true;
        } else {
            dst.base = sk.partial + (uint64_t)(2 * w + (k0 == 0 ? 1 : 0)) * (uint64_t)(BM * BN); dst.ld = BN;
            dst.row0 = tile_m * BM; dst.col0 = tile_n * BN;
            dst.accumulate = false; dst.fused = false;
        }
        gemm_tile<BM, BN, AMODE, BMODE>(g, stage0, stage1, stage2, batch, tile_m, tile_n, (int64_t)k0 * GEMM_BK, min(g.K, (int64_t)k1 * GEMM_BK), dst);
    }
}

// The same launch with the column sums of B added up beside the product (BsumArgs; vector operand forms; one matrix).  A
// tile of the first tile row that a workgroup computes whole adds its sums straight onto bsum.out; a piece of a shared tile
// leaves them in the slot of bsum.partial that matches its slot of sk.partial, for the fix-up.
template <int BM, int BN, int AMODE, int BMODE>
__global__ __launch_bounds__(GEMM_THREADS, (BM * BN <= 128 * 64 ? 4 : 2)) void gemm_streamk_bsum_kernel(const GemmArgs g, const StreamKArgs sk, const BsumArgs bsum) {
    constexpr int STAGE_FLOATS = (BM + BN) * GEMM_BK;
    __shared__ __attribute__((aligned(1024))) float stage0[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage1[STAGE_FLOATS];
    __shared__ __attribute__((aligned(1024))) float stage2[STAGE_FLOATS];
    const uint32_t tiles = (uint32_t)g.tiles_m * (uint32_t)g.tiles_n;
    const int64_t w = blockIdx.x;
    uint32_t whole = blockIdx.x;
    int64_t it = w * sk.per_wg;
    const int64_t end = min(sk.total, it + sk.per_wg);
    for (;;) {
        uint32_t gt;
        int64_t k0, k1;
        if (whole < (uint32_t)sk.dp_tiles) {
            gt = whole; k0 = 0; k1 = sk.nks;
            whole += gridDim.x;
        } else if (it < end) {
            const int64_t st = it / sk.nks;
            k0 = it - st * sk.nks;
            k1 = min(sk.nks, k0 + (end - it));
            gt = (uint32_t)(sk.dp_tiles + st);
            it += k1 - k0;
        } else {
            break;
        }
        int64_t tile_m, tile_n;
        tile_coords_blocked<BM, BN>(g, gt % tiles, tile_m, tile_n); // (one matrix: the tile id is the tile's number in it)
        const bool complete = k0 == 0 && k1 == sk.nks;
        const int64_t slot = 2 * w + (k0 == 0 ? 1 : 0);
        TileDest dst;
        if (complete) {
            dst.base = g.C; dst.ld = g.N; dst.row0 = 0; dst.col0 = 0;
            dst.accumulate = g.accumulate != 0; dst.fused = true;
        } else {
            dst.base = sk.partial + slot * (int64_t)(BM * BN); dst.ld = BN;
            dst.row0 = tile_m * BM; dst.col0 = tile_n * BN;
            dst.accumulate = false; dst.fused = false;
        }
        BsumDest bd{nullptr, 0, false};
        if (tile_m == 0) { // the first tile row sees every element of its columns of B once
            if (complete) { bd.out = bsum.out; bd.add = true; }
            else { bd.out = bsum.partial + slot * (int64_t)BN; bd.col0 = tile_n * BN; }
        }
        gemm_tile<BM, BN, AMODE, BMODE, true>(g, stage0, stage1, stage2, 0, tile_m, tile_n, k0 * GEMM_BK, min(g.K, k1 * GEMM_BK), dst, 0, 0, bd);
    }
}

// A tile that was shared between workgroups is the sum of their partial tiles (ascending workgroup
// order), finished with accumulate / the fused epilogue.  blockIdx.x = shared tile, blockIdx.y = one
// of gridDim.y equal parts of the tile, so that a launch with few tiles still fills the chip.
template <int BM, int BN>
__global__ void streamk_fixup_kernel(const GemmArgs g, const StreamKArgs sk, const BsumArgs bsum) {
    const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
    const int64_t gt = sk.dp_tiles + blockIdx.x;
    const int64_t it0 = (int64_t)blockIdx.x * sk.nks, it1 = it0 + sk.nks;
    const int64_t w_first = it0 / sk.per_wg, w_last = (it1 - 1) / sk.per_wg;
    if (w_first == w_last) return; // one workgroup had the whole tile and stored it
    const int64_t batch = gt / tiles;
    int64_t tile_m, tile_n;
    tile_coords_blocked<BM, BN>(g, gt % tiles, tile_m, tile_n);
    float* __restrict Cb = g.C + batch * g.M * g.N;
    const float* __restrict mask = g.mask ? g.mask + batch * g.M * g.N : nullptr;
    const bool fused = g.bias != nullptr || g.mask != nullptr || g.relu != 0;
    // the first contributor's piece starts at the tile's beginning (slot 2w+1) exactly when its run
    // began at or before the tile; every later contributor's piece starts inside the tile (slot 2w)
    const float* __restrict first = sk.partial + (2 * w_first + (w_first * sk.per_wg <= it0 ? 1 : 0)) * (int64_t)(BM * BN);
    // the column sums of B over the tile's pieces (BSUM launches: a tile of the first tile row), same slots, same order
    if (bsum.out != nullptr && tile_m == 0 && batch == 0 && blockIdx.y == 0) {
        for (int c = threadIdx.x; c < BN; c += blockDim.x) {
            const int64_t col = tile_n * BN + c;
            if (col >= g.N) continue;
            float s = bsum.out[col] + bsum.partial[(2 * w_first + (w_first * sk.per_wg <= it0 ? 1 : 0)) * (int64_t)BN + c];
            for (int64_t w = w_first + 1; w <= w_last; ++w) s += bsum.partial[(2 * w) * (int64_t)BN + c];
            bsum.out[col] = s;
        }
    }
    constexpr int PER_TILE = BM * BN / 4; // float4 positions
    const int part = PER_TILE / gridDim.y;
    for (int q4 = blockIdx.y * part + threadIdx.x; q4 < (int)(blockIdx.y + 1) * part; q4 += blockDim.x) {
        const int e = 4 * q4, r = e / BN, c = e % BN;
        const int64_t row = tile_m * BM + r, col = tile_n * BN + c;
        if (row >= g.M || col >= g.N) continue;
        f32x4 s = *reinterpret_cast<const f32x4*>(first + e);
        int64_t w = w_first + 1;
        for (; w + 3 <= w_last; w += 4) { // four loads in flight, added in workgroup order
            const float* __restrict p = sk.partial + (2 * w) * (int64_t)(BM * BN) + e;
            const f32x4 v0 = *reinterpret_cast<const f32x4*>(p);
            const f32x4 v1 = *reinterpret_cast<const f32x4*>(p + 2 * (int64_t)(BM * BN));
            const f32x4 v2 = *reinterpret_cast<const f32x4*>(p + 4 * (int64_t)(BM * BN));
            const f32x4 v3 = *reinterpret_cast<const f32x4*>(p + 6 * (int64_t)(BM * BN));
            s += v0; s += v1; s += v2; s += v3;
        }
        for (; w <= w_last; ++w) s += *reinterpret_cast<const f32x4*>(sk.partial + (2 * w) * (int64_t)(BM * BN) + e);
        const float v[4] = {s.x, s.y, s.z, s.w};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (col + q >= g.N) break;
            const int64_t i = row * g.N + col + q;
            float o = v[q];
            if (g.accumulate) o += Cb[i];
            if (fused) o = epilogue_value(o, g.bias, mask, g.relu, i, g.bias_rows ? row : col + q);
            Cb[i] = o;
        }
    }
}

} // namespace tenmo
