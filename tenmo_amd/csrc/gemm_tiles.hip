// The instantiations of gemm_mfma_kernel (and, for four of the tiles, gemm_streamk_kernel) for ONE
// workgroup tile, selected with -DTENMO_TILE_BM / -DTENMO_TILE_BN.  -DTENMO_TILE_STREAMK=0 compiles the
// one-workgroup-per-tile kernels, =1 the stream-K kernels of that tile.  tenmo_amd/build.py compiles
// this file once per (tile, part), in parallel.
#include "gemm_launch.hpp"

#ifndef TENMO_TILE_BM
#error "compile with -DTENMO_TILE_BM=<rows> -DTENMO_TILE_BN=<cols>"
#endif
#define TENMO_PASTE3(a, b, c, d) a##b##c##d
#define TENMO_NAME(prefix, bm, bn) TENMO_PASTE3(prefix, bm, x, bn)

namespace tenmo {

#if !TENMO_TILE_STREAMK
bool TENMO_NAME(launch_gemm_, TENMO_TILE_BM, TENMO_TILE_BN)(const GemmArgs& g, dim3 grid, int amode, int bmode, hipStream_t stream, const BsumArgs* bsum) {
    constexpr int BM = TENMO_TILE_BM, BN = TENMO_TILE_BN;
    if (bsum != nullptr) { // the column sums of B beside the product: the one operand form the weight gradient of a Linear layer has
        if (amode != MNMAJOR_VEC || bmode != MNMAJOR_VEC) return false;
        hipLaunchKernelGGL((gemm_mfma_bsum_kernel<BM, BN, MNMAJOR_VEC, MNMAJOR_VEC>), grid, dim3(GEMM_THREADS), 0, stream, g, *bsum);
        return true;
    }
#define TENMO_CASE(A_, B_)                                                                                     \
    if (amode == A_ && bmode == B_) {                                                                          \
        hipLaunchKernelGGL((gemm_mfma_kernel<BM, BN, A_, B_>), grid, dim3(GEMM_THREADS), 0, stream, g);        \
        return true;                                                                                           \
    }
    TENMO_CASE(KMAJOR_VEC, KMAJOR_VEC) TENMO_CASE(KMAJOR_VEC, MNMAJOR_VEC) TENMO_CASE(KMAJOR_VEC, KMAJOR_GEN)
    TENMO_CASE(MNMAJOR_VEC, KMAJOR_VEC) TENMO_CASE(MNMAJOR_VEC, MNMAJOR_VEC) TENMO_CASE(MNMAJOR_VEC, KMAJOR_GEN)
    TENMO_CASE(KMAJOR_GEN, KMAJOR_VEC) TENMO_CASE(KMAJOR_GEN, MNMAJOR_VEC) TENMO_CASE(KMAJOR_GEN, KMAJOR_GEN)
#undef TENMO_CASE
    return false;
}
#if (TENMO_TILE_BM == 64 && TENMO_TILE_BN == 64) || (TENMO_TILE_BM == 128 && TENMO_TILE_BN == 128)
bool TENMO_NAME(launch_gemm_reduce_, TENMO_TILE_BM, TENMO_TILE_BN)(const GemmArgs& g, const BatchReduce& red, unsigned wgs, int amode, int bmode, hipStream_t stream) {
    constexpr int BM = TENMO_TILE_BM, BN = TENMO_TILE_BN;
#define TENMO_CASE(A_, B_)                                                                                               \
    if (amode == A_ && bmode == B_) {                                                                                    \
        hipLaunchKernelGGL((gemm_reduce_kernel<BM, BN, A_, B_>), dim3(wgs), dim3(GEMM_THREADS), 0, stream, g, red);     \
        return true;                                                                                                     \
    }
    TENMO_CASE(KMAJOR_VEC, KMAJOR_VEC) TENMO_CASE(KMAJOR_VEC, MNMAJOR_VEC) TENMO_CASE(MNMAJOR_VEC, KMAJOR_VEC) TENMO_CASE(MNMAJOR_VEC, MNMAJOR_VEC)
#if TENMO_TILE_BM == 64 // operands without a unit stride (views with steps, overlapping rows): the small tile only
    TENMO_CASE(KMAJOR_VEC, KMAJOR_GEN) TENMO_CASE(MNMAJOR_VEC, KMAJOR_GEN) TENMO_CASE(KMAJOR_GEN, KMAJOR_VEC) TENMO_CASE(KMAJOR_GEN, MNMAJOR_VEC)
    TENMO_CASE(KMAJOR_GEN, KMAJOR_GEN)
#endif
#undef TENMO_CASE
    return false;
}
#endif
#if TENMO_TILE_BM == 64 && TENMO_TILE_BN == 64
bool launch_gemm_pair_64x64(const GemmArgs& g0, const GemmArgs& g1, unsigned count0, unsigned count1, int amode0, int bmode0, int amode1, int bmode1,
                            hipStream_t stream) {
    // the one combination in use: X^T(view).G beside G.W^T(view)
    if (amode0 != MNMAJOR_VEC || bmode0 != MNMAJOR_VEC || amode1 != KMAJOR_VEC || bmode1 != KMAJOR_VEC) return false;
    hipLaunchKernelGGL((gemm_pair_kernel<64, 64, MNMAJOR_VEC, MNMAJOR_VEC, KMAJOR_VEC, KMAJOR_VEC>), dim3(count0 + count1), dim3(GEMM_THREADS), 0, stream,
                       g0, g1, count0);
    return true;
}
#endif
#else
bool TENMO_NAME(launch_streamk_, TENMO_TILE_BM, TENMO_TILE_BN)(const GemmArgs& g, const StreamKArgs& sk, unsigned wgs, unsigned tiles,
                                                              unsigned fix_parts, int amode, int bmode, hipStream_t stream, const BsumArgs* bsum) {
    constexpr int BM = TENMO_TILE_BM, BN = TENMO_TILE_BN;
#define TENMO_CASE(A_, B_)                                                                                               \
    if (amode == A_ && bmode == B_)                                                                                      \
        hipLaunchKernelGGL((gemm_streamk_kernel<BM, BN, A_, B_>), dim3(wgs), dim3(GEMM_THREADS), 0, stream, g, sk);
    if (bsum != nullptr) { // (the 128x128 tile only: the others have no registers left for the sums without spilling inside their loops)
#if TENMO_TILE_BM == 128 && TENMO_TILE_BN == 128
        if (amode != MNMAJOR_VEC || bmode != MNMAJOR_VEC) return false;
        hipLaunchKernelGGL((gemm_streamk_bsum_kernel<BM, BN, MNMAJOR_VEC, MNMAJOR_VEC>), dim3(wgs), dim3(GEMM_THREADS), 0, stream, g, sk, *bsum);
#else
        return false;
#endif
    } else
    TENMO_CASE(KMAJOR_VEC, KMAJOR_VEC) else TENMO_CASE(KMAJOR_VEC, MNMAJOR_VEC) else TENMO_CASE(MNMAJOR_VEC, KMAJOR_VEC) else TENMO_CASE(MNMAJOR_VEC, MNMAJOR_VEC)
    else return false;
#undef TENMO_CASE
    if (fix_parts) hipLaunchKernelGGL((streamk_fixup_kernel<BM, BN>), dim3(tiles, fix_parts), dim3(256), 0, stream, g, sk, bsum ? *bsum : BsumArgs{});
    return true;
}
#endif

} // namespace tenmo
