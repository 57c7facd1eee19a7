// Products whose result is large next to their reduction (attention's Q.K^T and dO.V^T, tenmo/matmul.mojo:36-38 on the
// backward side; the CBOW logits [256,100].[100,50000] of examples/word2vec_cbow.mojo:531-553 and their gradient; any
// K up to a few hundred against thousands of tiles).  One workgroup per tile spends such a launch on things that are
// not MFMAs: every tile primes and drains its own K loop, and its stores — most of the traffic — go out after the last
// MFMA with nothing running beside them.
//
// Here a persistent workgroup treats the K steps of all its tiles as ONE stream:
//   * wavefronts 4-7 only load: K step after K step, tile after tile, they copy operand stages into a ring of NP LDS
//     stages with direct loads (global_load_lds), several steps ahead of the one being multiplied, so that a tile's
//     first operands are on their way while the tile before is still being multiplied;
//   * wavefronts 0-3 (2x2) multiply and store: they never wait for a load;
//   * one workgroup barrier per K step hands stages over: barrier number u tells the multiplying wavefronts that steps
//     u and u+1 have landed (so that the operand fetch of the next step's first half runs behind the MFMAs of this
//     step's second half), and tells the loading wavefronts that step u-1 has been read and its stage is free.
// A stage is the ordinary kernel's LDS stage ([A rows | B rows][16 k], K-major tiles swizzled), so the loaders and the
// operand fetch are those of gemm_mfma.hpp.  A K that is no multiple of 16: the lanes of the last step whose k do not
// exist re-read the step's first chunk (in bounds), and the multiplying wavefronts zero those operand registers.
//
// A tile's stores go out in one burst at its end, as non-temporal stores (the result is not read again by this launch and
// would push the operands out of the L2s); two workgroups share a CU, so that one multiplies while the other stores.
// `accumulate` (the gradbox +=) adds with one hardware fp32 atomic per element: each element of C is touched by exactly
// one lane of the launch, so the result is old + sum, in a fixed order.
//
// What bounds such a launch, measured on attention's Q.K^T ([8,12,1024,64], 82 us of MFMAs, 403 MB of result): the MFMAs
// alone (no loads, no stores) take 99 us in this kernel, with the loads 123 us, with the stores 156 us; the loads and the
// stores alone 76 us.  The stores do not overlap with the rest however they are issued — in a burst, paced with sleeps,
// or (a variant with two alternating sets of accumulators and the K steps unrolled) one by one behind the MFMAs of the
// whole next tile: 156-170 us every time.  A compute unit feeds ONE in-order vector-memory queue; while the memory
// system drains a CU's stores at its own pace (about 20 GB/s per CU when all 256 write), the loading wavefronts' next
// loads wait in that queue behind them (their issue was seen to stall for 2 us at a time) and the multiplying
// wavefronts starve.
#include <algorithm>

#include "gemm_launch.hpp"

namespace tenmo {

constexpr int PANEL_THREADS = 512; // four multiplying wavefronts and four loading ones

struct PanelArgs {
    uint32_t total_tiles, xcds, chunk; // the tile walk (gemm_index.hpp)
    int32_t col_major;                 // tiles numbered column block by column block
    int32_t nk;                        // K steps of 16 per tile
    int32_t k_tail;                    // k that exist in the last step: 1..16
};

// ring depth for two resident workgroups per CU (160 KiB of LDS; 16 wavefronts of at most 128 registers)
constexpr int panel_ring(int bm, int bn) { return (80 * 1024) / ((bm + bn) * GEMM_BK * 4) > 8 ? 8 : (80 * 1024) / ((bm + bn) * GEMM_BK * 4); }
constexpr int PANEL_WGS_PER_CU = 2;

// waits until at most `units` x LPU of this wavefront's loads are outstanding (the immediate must be a constant)
template <int LPU>
__device__ __forceinline__ void wait_loads_ahead(int units) {
    switch (units) {
        case 0: __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); break;
        case 1: __builtin_amdgcn_s_waitcnt(vmcnt_imm(1 * LPU)); break;
        case 2: __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * LPU)); break;
        case 3: __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * LPU)); break;
        case 4: __builtin_amdgcn_s_waitcnt(vmcnt_imm(4 * LPU)); break;
        default: __builtin_amdgcn_s_waitcnt(vmcnt_imm(5 * LPU)); break; // more would be allowed: waiting for fewer is safe
    }
}

// (the second launch bound is wavefronts per SIMD: a workgroup brings two to each)
template <int AMODE, int BMODE, int BM, int BN, bool ACC>
__global__ __launch_bounds__(PANEL_THREADS, 2 * PANEL_WGS_PER_CU) void gemm_panel_kernel(const GemmArgs g, const PanelArgs pa) {
    constexpr int NP = panel_ring(BM, BN);
    constexpr int TM = BM / 2, TN = BN / 2;   // wave tile (2x2 multiplying wavefronts)
    constexpr int MB = TM / 32, NB = TN / 32; // 32x32 blocks per wave tile
    constexpr int A_FLOATS = BM * GEMM_BK, STAGE = (BM + BN) * GEMM_BK;
    using LA = TileLoader<BM, AMODE>;
    using LB = TileLoader<BN, BMODE>;
    static_assert(NP >= 4 && NP <= 8, "ring of 4 to 8 stages");
    static_assert(5 * (LA::NCH + LB::NCH) < 64, "the load counter holds 63");
    __shared__ __attribute__((aligned(1024))) float ring[NP * STAGE];

    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    TileWalk walk;
    walk.start(blockIdx.x, gridDim.x, pa.total_tiles, pa.xcds, pa.chunk);
    if (walk.tile() >= pa.total_tiles) return; // (every wavefront of the workgroup alike)
    const int nk = pa.nk;
    const bool ragged_k = pa.k_tail < GEMM_BK;
    const uint32_t tiles_m = (uint32_t)g.tiles_m, tiles_n = (uint32_t)g.tiles_n;

    if (wave >= 4) {
        // ---- a loading wavefront: part `w` of every stage ----
        const int w = wave - 4;
        constexpr int NA = LA::NCH, NBL = LB::NCH, LPU = NA + NBL; // loads per K step and wavefront
        LA la;
        LB lb;
        uint32_t a_tail[NA], b_tail[NBL]; // lane offsets of the last K step when K is no multiple of 16
        auto init_tile = [&](uint32_t tile) {
            uint32_t b;
            int64_t m0, n0, a_boff, b_boff;
            tile_origin(tile, tiles_m, tiles_n, pa.col_major, BM, BN, b, m0, n0);
            batch_offsets(g.batch, b, a_boff, b_boff);
            la.init_direct(g.A + a_boff, g.a_rs, g.a_cs, m0, 0, g.M, lane, w);
            lb.init_direct(g.B + b_boff, g.b_cs, g.b_rs, n0, 0, g.N, lane, w);
            la.tail_offsets(g.a_rs, g.a_cs, m0, g.M, lane, w, pa.k_tail, a_tail);
            lb.tail_offsets(g.b_cs, g.b_rs, n0, g.N, lane, w, pa.k_tail, b_tail);
        };
        auto issue = [&](int slot, int ks) { // K step `ks` of the current tile into stage `slot` of the ring
            float* st = ring + slot * STAGE;
            const bool tail = ragged_k && ks == nk - 1;
#pragma unroll
            for (int j = 0; j < NA; ++j) la.load_direct_at(st, (int64_t)ks * GEMM_BK, w, j, tail ? a_tail[j] : la.lane_off[j]);
#pragma unroll
            for (int j = 0; j < NBL; ++j) lb.load_direct_at(st + A_FLOATS, (int64_t)ks * GEMM_BK, w, j, tail ? b_tail[j] : lb.lane_off[j]);
        };
        kstream_loader(walk, nk, NP, init_tile, issue, [&](int ahead) {
            wait_loads_ahead<LPU>(ahead);
            bare_barrier();
        });
        return;
    }

    // ---- a multiplying wavefront ----
    const int wm = wave >> 1, wn = wave & 1;
    const int h = lane >> 5, x = lane & 31;
    constexpr int PA = frag_parts<AMODE, MB>(), PB = frag_parts<BMODE, NB>(); // LDS reads per 8-wide k chunk
    constexpr int NMFMA = 4 * MB * NB;                                        // MFMAs per chunk
    constexpr int NSLOT = MB * 16;                                            // store slots of a tile: (block row i, accumulator element e)
    constexpr int PER_MFMA = (PA + PB + NMFMA - 1) / NMFMA;                   // operand fetches placed behind one MFMA: 1, or 2 for the 64x64 tile
    static_assert(PER_MFMA <= 2, "at most two operand fetches behind an MFMA");

    f32x16 acc[MB][NB];
    float fa[2][MB][4], fb[2][NB][4]; // operand registers of the two k chunks of a step

    // A store's address is a wave-uniform row pointer (the tile's corner in C plus a constant number of rows: scalar
    // arithmetic) plus ONE per-lane byte offset shared by every store of the lane.
    const uint32_t row_bytes = (uint32_t)g.N * 4u;
    const int lane_row = wm * TM + (AMODE == MNMAJOR_VEC ? MB : 1) * 4 * h;       // row of accumulator element 0 of block row 0
    const int lane_col = wn * TN + (BMODE == MNMAJOR_VEC ? NB * x : x);           // column of block column 0
    const uint32_t lane_byte = (uint32_t)lane_row * row_bytes + (uint32_t)lane_col * 4u;
    // store slot sl = (i, e) of the finished tile whose corner in C is `tile_base` and of which rows x cols exist:
    // row lane_row + c(i, e) with c a constant; NB values at columns lane_col + (MN-major: j, K-major: 32 j)
    auto store_slot = [&](auto whole_t, char* tile_base, int rows, int cols, int sl) {
        const f32x16 (&src)[MB][NB] = acc;
        constexpr bool WHOLE = decltype(whole_t)::value;
        const int i = sl / 16, e = sl % 16;
        const int c = AMODE == MNMAJOR_VEC ? MB * (8 * (e >> 2) + (e & 3)) + i : 32 * i + 8 * (e >> 2) + (e & 3);
        char* rowp = tile_base + (uint64_t)((uint32_t)c * row_bytes); // uniform
        float* p = reinterpret_cast<float*>(rowp + lane_byte);
        const bool row_ok = WHOLE || lane_row < rows - c;
        if constexpr (BMODE == MNMAJOR_VEC && NB == 2 && !ACC) {
            if (WHOLE || (row_ok && lane_col + 1 < cols)) {
                const f32x2 v = {src[i][0][e], src[i][1][e]};
                __builtin_nontemporal_store(v, reinterpret_cast<f32x2_u*>(p));
            } else if (row_ok && lane_col < cols) {
                __builtin_nontemporal_store(src[i][0][e], p);
            }
        } else {
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const int dc = BMODE == MNMAJOR_VEC ? j : 32 * j;
                if (WHOLE || (row_ok && lane_col + dc < cols)) {
                    if constexpr (ACC) unsafeAtomicAdd(p + dc, src[i][j][e]);
                    else __builtin_nontemporal_store(src[i][j][e], p + dc);
                }
            }
        }
    };

    auto fetch_part = [&](const float* st, int kc, int p) { // operand fetch number p (A's parts, then B's) of chunk kc
        if (p < PA) load_fragment_part<BM, AMODE, MB>(st, wm * TM, kc, lane, fa[kc], p);
        else if (p < PA + PB) load_fragment_part<BN, BMODE, NB>(st + A_FLOATS, wn * TN, kc, lane, fb[kc], p - PA);
    };
    // zero the operand registers of chunk kc whose k (8 kc + 4 h + s) is at or beyond `klimit`
    auto mask_tail = [&](int kc, int klimit) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bool ok = 8 * kc + 4 * h + s < klimit;
#pragma unroll
            for (int i = 0; i < MB; ++i) fa[kc][i][s] = ok ? fa[kc][i][s] : 0.f;
#pragma unroll
            for (int j = 0; j < NB; ++j) fb[kc][j][s] = ok ? fb[kc][j][s] : 0.f;
        }
    };
    // The MFMAs of chunk kc with `slot(n)` placed behind MFMA n.  (There is ONE such sequence per chunk in the kernel:
    // alternative sequences for different kinds of steps make the compiler keep the accumulators in two sets of
    // registers and copy between them every step, and a branch behind every MFMA costs more than the MFMA.)
    auto mfma_chunk = [&](int kc, auto&& slot) {
        int n = 0;
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int i = 0; i < MB; ++i)
#pragma unroll
                for (int j = 0; j < NB; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[kc][i][s], fb[kc][j][s], acc[i][j], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
                    slot(n);
                    __builtin_amdgcn_sched_barrier(0);
                    ++n;
                }
    };

    bool first = true;
    auto barrier = [&]() {
        bare_barrier();
        if (first) { // behind barrier 0: the first operands of step 0
            first = false;
#pragma unroll
            for (int p = 0; p < PA + PB; ++p) fetch_part(ring, 0, p);
        }
    };

        kstream_consumer(
            walk, nk, NP, barrier,
            [&](int slot, int next_slot, int ks, bool last_step, int) {
                const float* st = ring + slot * STAGE;
                const float* st_next = ring + next_slot * STAGE;
                if (ks == 0) {
#pragma unroll
                    for (int i = 0; i < MB; ++i)
#pragma unroll
                        for (int j = 0; j < NB; ++j)
#pragma unroll
                            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
                }
                const int klimit = ragged_k && last_step ? pa.k_tail : GEMM_BK;
                if (klimit < GEMM_BK) mask_tail(0, klimit);
                // chunk 0; behind its MFMAs the operand fetch of chunk 1
                mfma_chunk(0, [&](int n) {
#pragma unroll
                    for (int q = 0; q < PER_MFMA; ++q)
                        if (n * PER_MFMA + q < PA + PB) fetch_part(st, 1, n * PER_MFMA + q);
                });
                if (klimit > 8) {
                    if (klimit < GEMM_BK) mask_tail(1, klimit);
                    // chunk 1; behind its MFMAs the operand fetch of the next step's chunk 0 (harmless when there is no
                    // next step: the registers are not used)
                    mfma_chunk(1, [&](int n) {
#pragma unroll
                        for (int q = 0; q < PER_MFMA; ++q)
                            if (n * PER_MFMA + q < PA + PB) fetch_part(st_next, 0, n * PER_MFMA + q);
                    });
                } else {
#pragma unroll
                    for (int p = 0; p < PA + PB; ++p) fetch_part(st_next, 0, p);
                }
            },
            [&](uint32_t tile, int) {
                uint32_t b;
                int64_t m0, n0;
                tile_origin(tile, tiles_m, tiles_n, pa.col_major, BM, BN, b, m0, n0);
                char* tile_base = reinterpret_cast<char*>(g.C + ((int64_t)b * g.M + m0) * g.N + n0);
                const int rows = (int)min((int64_t)BM, g.M - m0), cols = (int)min((int64_t)BN, g.N - n0);
                if (rows == BM && cols == BN) {
#pragma unroll
                    for (int sl = 0; sl < NSLOT; ++sl) store_slot(std::true_type{}, tile_base, rows, cols, sl);
                } else { // a ragged tile (last tile-row or tile-column): lane by lane under its bounds
#pragma unroll
                    for (int sl = 0; sl < NSLOT; ++sl) store_slot(std::false_type{}, tile_base, rows, cols, sl);
                }
            });
}

namespace {

struct PanelLaunch {
    unsigned cus, total_tiles;
    bool by_batch;
    hipStream_t stream;
};

template <int AMODE, int BMODE, int BM, int BN>
void launch_panel(const GemmArgs& g, const PanelLaunch& l) {
    const TileWalkPlan plan = plan_tile_walk(l.total_tiles, (unsigned)g.tiles_m, (unsigned)g.tiles_n, l.cus, PANEL_WGS_PER_CU, l.by_batch);
    PanelArgs pa{};
    pa.total_tiles = l.total_tiles;
    pa.xcds = plan.xcds; pa.chunk = plan.chunk; pa.col_major = plan.col_major;
    pa.nk = (int32_t)((g.K + GEMM_BK - 1) / GEMM_BK);
    pa.k_tail = (int32_t)(g.K - (int64_t)(pa.nk - 1) * GEMM_BK);
    if (g.accumulate)
        hipLaunchKernelGGL((gemm_panel_kernel<AMODE, BMODE, BM, BN, true>), dim3(plan.grid), dim3(PANEL_THREADS), 0, l.stream, g, pa);
    else
        hipLaunchKernelGGL((gemm_panel_kernel<AMODE, BMODE, BM, BN, false>), dim3(plan.grid), dim3(PANEL_THREADS), 0, l.stream, g, pa);
}

template <int BM, int BN>
bool launch_panel_modes(const GemmArgs& g, int amode, int bmode, const PanelLaunch& l) {
    if (amode == KMAJOR_VEC && bmode == KMAJOR_VEC) launch_panel<KMAJOR_VEC, KMAJOR_VEC, BM, BN>(g, l);
    else if (amode == KMAJOR_VEC && bmode == MNMAJOR_VEC) launch_panel<KMAJOR_VEC, MNMAJOR_VEC, BM, BN>(g, l);
    else if (amode == MNMAJOR_VEC && bmode == KMAJOR_VEC) launch_panel<MNMAJOR_VEC, KMAJOR_VEC, BM, BN>(g, l);
    else if (amode == MNMAJOR_VEC && bmode == MNMAJOR_VEC) launch_panel<MNMAJOR_VEC, MNMAJOR_VEC, BM, BN>(g, l);
    else return false;
    return true;
}

} // namespace

bool launch_gemm_panel(const GemmArgs& g, int tile, int amode, int bmode, unsigned cus, unsigned total_tiles, bool by_batch, hipStream_t stream) {
    if (g.K < 1 || total_tiles == 0) return false;
    const PanelLaunch l{cus, total_tiles, by_batch, stream};
    if (tile == PANEL_TILE_128x128) return launch_panel_modes<128, 128>(g, amode, bmode, l);
    if (tile == PANEL_TILE_64x64) return launch_panel_modes<64, 64>(g, amode, bmode, l);
    return false;
}

} // namespace tenmo
