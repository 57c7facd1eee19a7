// Products with a short reduction (K <= 64) and a large result: C[b][M,N] (+)= A[b][M,K] . B[b][K,N] with both
// operands K-major (row-major A, transposed-view B: attention's Q.K^T and dO.V^T, tenmo/matmul.mojo:36-38 on the
// backward side).  Such a launch is bound by its stores, not by the matrix pipe.  The vector memory operations of a
// wavefront complete in issue order, so in a kernel whose wavefronts both load and store, the loads of a tile wait
// for the acknowledgement of every store issued before them — under a saturated write path that is microseconds —
// and the run time approaches the SUM of MFMA time and store time (measured: attention Q.K^T 180 us against 100 us
// of MFMAs; with the stores removed 131 us, with the loads removed 124 us).
//
// Here the two kinds of traffic belong to different wavefronts of a persistent workgroup that walks 64x64 tiles:
//   * wavefronts 4-7 only load: they copy the operands of a WHOLE tile (all of K) into one of two LDS panels with
//     direct loads (global_load_lds), one tile ahead, and wait for them alone;
//   * wavefronts 0-3 (2x2, one 32x32 block each) fetch operands from the panel, run the MFMAs and store; they never
//     wait for a memory operation (an accumulating store loads the old values before the MFMAs).
// The result is written with non-temporal stores: it is far
// larger than the L2 and is not read again by this launch, while the operands are read many times; written
// normally, the result's lines push the operands out of the L2 (attention Q.K^T: 175 us, non-temporal 139 us).
// One workgroup barrier per tile hands panels over: behind it the panel of this tile is complete and the panel of
// the tile before is free for the tile after.
// A panel is the K steps of the ordinary kernel's LDS stage laid end to end ([K step][A rows | B rows][16 k],
// swizzled as there), so the loaders and the operand fetch are the ones of gemm_mfma.hpp.
#include <algorithm>

#include "gemm_launch.hpp"

namespace tenmo {

constexpr int SMALLK_THREADS = 512; // four computing wavefronts and four loading ones

// TileLoader::load_direct (one 16-row / 4-k part `part` of the tile at K offset koff) for the lanes with `ok` only:
// the others neither read memory nor write LDS.
template <class Loader>
__device__ __forceinline__ void load_direct_where(const Loader& l, float* lds, int64_t koff, int part, bool ok) {
    direct_load_16B_where(lds, (uint32_t)(part * 1024), l.lane_off[0], l.origin + koff * l.kstep, ok);
}

// AMODE / BMODE: KMAJOR_VEC or MNMAJOR_VEC (the LDS layouts and loaders of gemm_mfma.hpp).  NK = K steps of 16 that
// cover K; `col_major`: tiles are numbered column block by column block (few tile-rows: see the launcher).
template <int AMODE, int BMODE, int NK, int WGS_PER_CU, bool ACC>
__global__ __launch_bounds__(SMALLK_THREADS, WGS_PER_CU) void gemm_smallk_kernel(const GemmArgs g, const uint32_t total_tiles, const uint32_t xcds, const uint32_t chunk,
                                                                                 const int col_major) {
    constexpr int BM = 64, BN = 64;
    constexpr int A_FLOATS = BM * GEMM_BK, STAGE = (BM + BN) * GEMM_BK;
    using LA = TileLoader<BM, AMODE>;
    using LB = TileLoader<BN, BMODE>;
    static_assert(LA::NCH == 1 && LB::NCH == 1, "one direct load per operand, quarter tile and K step");
    __shared__ __attribute__((aligned(1024))) float panel0[STAGE * NK];
    __shared__ __attribute__((aligned(1024))) float panel1[STAGE * NK];

    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    // K not a multiple of 16: the loads of the last K step skip what lies beyond K (a K-major operand in 16-byte
    // chunks: the host admits K % 4 == 0 only), and those places of the panels, which no load ever writes, are
    // zeroed once here.
    const int k_tail = (int)g.K - (NK - 1) * GEMM_BK; // valid k of the last step, 1..16
    if (k_tail < GEMM_BK) {
        for (int i = t * 4; i < STAGE * NK; i += SMALLK_THREADS * 4) {
            *reinterpret_cast<f32x4*>(panel0 + i) = f32x4{0.f, 0.f, 0.f, 0.f};
            *reinterpret_cast<f32x4*>(panel1 + i) = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        __syncthreads();
    }
    const uint32_t tiles_n = (uint32_t)g.tiles_n, tiles_per_batch = (uint32_t)g.tiles_m * tiles_n;
    // Which tiles this workgroup takes.  Workgroup ids are dealt round-robin to the `xcds` XCDs (8, or 1 for a plain
    // round-robin over the grid); the workgroups of one XCD walk `chunk` consecutive tiles together (one batch),
    // then the chunk `xcds` further on: an XCD then reads the operands of its own batches only, where a plain
    // round-robin makes every L2 fetch every batch's operands (8 x the operand traffic, as much as the stores).
    const uint32_t per_xcd = gridDim.x / xcds, xcd = blockIdx.x % xcds;
    auto tile_at = [&](uint32_t q) { // q = position in this XCD's sequence; increasing in q; >= total_tiles: done
        const uint32_t c = q / chunk;
        const uint64_t tl = ((uint64_t)c * xcds + xcd) * chunk + (q - c * chunk);
        return (uint32_t)std::min<uint64_t>(tl, total_tiles);
    };
    uint32_t q = blockIdx.x / xcds;
    uint32_t tile = tile_at(q);
    if (tile >= total_tiles) return; // (every wavefront of the workgroup alike)
    auto advance = [&]() -> bool { // to this workgroup's next tile; false: there is none
        q += per_xcd;
        tile = tile_at(q);
        return tile < total_tiles;
    };
    // tiles are numbered row by row inside a batch: workgroups side by side share the A rows and stream B
    const uint32_t tiles_m = (uint32_t)g.tiles_m;
    auto tile_coords3 = [&](uint32_t tl, uint32_t& b, int64_t& m0, int64_t& n0) {
        b = tl / tiles_per_batch;
        const uint32_t r = tl - b * tiles_per_batch;
        uint32_t tm, tn;
        if (col_major) { tn = r / tiles_m; tm = r - tn * tiles_m; }
        else { tm = r / tiles_n; tn = r - tm * tiles_n; }
        m0 = (int64_t)tm * BM;
        n0 = (int64_t)tn * BN;
    };

    if (wave >= 4) {
        // ---- a loading wavefront: one of the four 16-row parts of the ordinary tile loader ----
        // (one wavefront for the whole panel was measured at about 110 ns per 1 KiB load: far too slow)
        const int w = wave - 4;
        // k (within a K step) of this lane's 16 bytes, as the loaders lay them out: a K-major load moves 4 consecutive k
        // of one row (chunk (lane & 3) ^ ((lane >> 4) & 3), the swizzle), an MN-major load one k of 4 rows
        auto last_ok = [&](int mode) {
            if (mode == KMAJOR_VEC) return 4 * ((lane & 3) ^ ((lane >> 4) & 3)) + 4 <= k_tail;
            return 4 * w + lane / 16 < k_tail;
        };
        const bool a_last_ok = last_ok(AMODE), b_last_ok = last_ok(BMODE);
        auto issue_tile = [&](float* panel, uint32_t tl) {
            uint32_t b;
            int64_t m0, n0, a_boff, b_boff;
            tile_coords3(tl, b, m0, n0);
            batch_offsets(g.batch, b, a_boff, b_boff);
            LA la;
            LB lb;
            la.init_direct(g.A + a_boff, g.a_rs, g.a_cs, m0, 0, g.M, lane, w);
            lb.init_direct(g.B + b_boff, g.b_cs, g.b_rs, n0, 0, g.N, lane, w);
#pragma unroll
            for (int it = 0; it < NK - 1; ++it) {
                la.load_direct(panel + it * STAGE, (int64_t)it * GEMM_BK, w, 0);
                lb.load_direct(panel + it * STAGE + A_FLOATS, (int64_t)it * GEMM_BK, w, 0);
            }
            // the last step: this lane's part of it may lie beyond K
            load_direct_where(la, panel + (NK - 1) * STAGE, (int64_t)(NK - 1) * GEMM_BK, w, a_last_ok);
            load_direct_where(lb, panel + (NK - 1) * STAGE + A_FLOATS, (int64_t)(NK - 1) * GEMM_BK, w, b_last_ok);
        };
        issue_tile(panel0, tile);
        for (;;) {
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); // panel0 is complete
            bare_barrier();                           // ... and every computing wavefront has left panel1
            if (!advance()) break;
            issue_tile(panel1, tile);
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            bare_barrier();
            if (!advance()) break;
            issue_tile(panel0, tile);
        }
        return;
    }

    // ---- the computing wavefronts ----
    const int wm = wave >> 1, wn = wave & 1;
    const int h = lane >> 5, x = lane & 31;
    const int64_t N = g.N;
    // Accumulator element e is row 8(e>>2) + 4h + (e&3), column x of the wavefront's 32x32 block.
    auto row_of = [](int e) { return 8 * (e >> 2) + (e & 3); };
    auto one_tile = [&](const float* __restrict panel) {
        uint32_t b;
        int64_t m0, n0;
        tile_coords3(tile, b, m0, n0);
        const int64_t row = m0 + wm * 32 + 4 * h, col = n0 + wn * 32 + x;
        float* __restrict dst = g.C + ((int64_t)b * g.M + row) * N + col; // element e at dst[row_of(e) * N]
        const bool whole = m0 + BM <= g.M && n0 + BN <= N;                 // the same for the whole workgroup
        const int rows_left = (int)std::min<int64_t>(g.M - row, 64);
        const bool col_ok = col < N;
        float old[16];
        if constexpr (ACC) { // the old values travel while the MFMAs run
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                old[e] = 0.f;
                if (whole || (col_ok && row_of(e) < rows_left)) old[e] = dst[(int64_t)row_of(e) * N];
            }
        }
        bare_barrier(); // the panel is complete
        f32x16 acc;
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[e] = 0.f;
        float fa[2][1][4], fb[2][1][4];
        load_fragments<BM, AMODE, 1>(panel, wm * 32, 0, lane, fa[0]);
        load_fragments<BN, BMODE, 1>(panel + A_FLOATS, wn * 32, 0, lane, fb[0]);
#pragma unroll
        for (int c = 0; c < 2 * NK; ++c) { // 8-wide chunks of K; the operand fetch runs one chunk ahead
            if (c + 1 < 2 * NK) {
                const float* st = panel + ((c + 1) >> 1) * STAGE;
                load_fragments<BM, AMODE, 1>(st, wm * 32, (c + 1) & 1, lane, fa[(c + 1) & 1]);
                load_fragments<BN, BMODE, 1>(st + A_FLOATS, wn * 32, (c + 1) & 1, lane, fb[(c + 1) & 1]);
            }
#pragma unroll
            for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[c & 1][0][s], fb[c & 1][0][s], acc, 0, 0, 0);
        }
        if (whole) {
#pragma unroll
            for (int e = 0; e < 16; ++e) __builtin_nontemporal_store(ACC ? acc[e] + old[e] : acc[e], &dst[(int64_t)row_of(e) * N]);
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e)
                if (col_ok && row_of(e) < rows_left) __builtin_nontemporal_store(ACC ? acc[e] + old[e] : acc[e], &dst[(int64_t)row_of(e) * N]);
        }
    };
    for (;;) {
        one_tile(panel0);
        if (!advance()) break;
        one_tile(panel1);
        if (!advance()) break;
    }
}

namespace {

struct SmallkLaunch {
    unsigned cus, total_tiles;
    bool by_batch;
    hipStream_t stream;
};

template <int AMODE, int BMODE, int NK, int WPC>
void launch_smallk(const GemmArgs& g, const SmallkLaunch& l) {
    const unsigned wgs = std::min(l.total_tiles, l.cus * WPC);
    const unsigned per_batch = (unsigned)g.tiles_m * (unsigned)g.tiles_n;
    // With 8 or more batches the workgroups of an XCD take whole batches; else, with fewer than 8 tile-rows, whole
    // column blocks (tiles numbered column block by column block): a panel of B is then fetched by one L2.
    unsigned xcds = 1, chunk = 1;
    int col_major = 0;
    if (wgs % 8 == 0) {
        if (l.by_batch && l.total_tiles / per_batch >= 8) { xcds = 8; chunk = per_batch; }
        else if (l.by_batch && g.tiles_m < 8 && g.tiles_n >= 64) { xcds = 8; chunk = (unsigned)g.tiles_m; col_major = 1; }
    }
    if (g.accumulate)
        hipLaunchKernelGGL((gemm_smallk_kernel<AMODE, BMODE, NK, WPC, true>), dim3(wgs), dim3(SMALLK_THREADS), 0, l.stream, g, l.total_tiles, xcds, chunk, col_major);
    else
        hipLaunchKernelGGL((gemm_smallk_kernel<AMODE, BMODE, NK, WPC, false>), dim3(wgs), dim3(SMALLK_THREADS), 0, l.stream, g, l.total_tiles, xcds, chunk, col_major);
}

// LDS per workgroup: two panels of 8 KiB per K step
template <int AMODE, int BMODE>
bool launch_smallk_modes(const GemmArgs& g, int nk, const SmallkLaunch& l) {
    switch (nk) {
        case 1: launch_smallk<AMODE, BMODE, 1, 4>(g, l); return true;
        case 2: launch_smallk<AMODE, BMODE, 2, 4>(g, l); return true;
        case 3: launch_smallk<AMODE, BMODE, 3, 2>(g, l); return true;
        case 4: launch_smallk<AMODE, BMODE, 4, 2>(g, l); return true;
        default: return false;
    }
}

} // namespace

bool launch_gemm_smallk_64x64(const GemmArgs& g, int amode, int bmode, unsigned cus, unsigned total_tiles, bool by_batch, hipStream_t stream) {
    const int nk = (int)((g.K + GEMM_BK - 1) / GEMM_BK);
    if (nk < 1 || nk > 4 || total_tiles == 0) return false; // (more K steps: one workgroup per CU, no gain; not instantiated)
    const SmallkLaunch l{cus, total_tiles, by_batch, stream};
    if (amode == KMAJOR_VEC && bmode == KMAJOR_VEC) return launch_smallk_modes<KMAJOR_VEC, KMAJOR_VEC>(g, nk, l);
    if (amode == KMAJOR_VEC && bmode == MNMAJOR_VEC) return launch_smallk_modes<KMAJOR_VEC, MNMAJOR_VEC>(g, nk, l);
    if (amode == MNMAJOR_VEC && bmode == KMAJOR_VEC) return launch_smallk_modes<MNMAJOR_VEC, KMAJOR_VEC>(g, nk, l);
    if (amode == MNMAJOR_VEC && bmode == MNMAJOR_VEC) return launch_smallk_modes<MNMAJOR_VEC, MNMAJOR_VEC>(g, nk, l);
    return false;
}

} // namespace tenmo
