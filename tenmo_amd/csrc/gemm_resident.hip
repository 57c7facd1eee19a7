// Products of a SMALL left operand with a very wide right one: C[M,N] = A[M,K] . B[K,N] with M of a few tile rows, K up to
// 256 and N in the tens of thousands — the CBOW logits [256,100].[100,50000] of examples/word2vec_cbow.mojo:531-553 and
// the gradient A^T.dC [100,256].[256,50000] that tenmo/matmul.mojo:46-48 issues for them.  One workgroup per tile reads
// the same rows of A again for every one of hundreds of column tiles, and the K-stream kernel (gemm_panel.hip) still
// does: half of what its loading wavefronts move is A.
//
// Here a persistent workgroup keeps its tile row of A — ALL of K — in LDS for its whole life (a panel of K steps, each
// laid out as the A part of the ordinary kernel's LDS stage) and streams only B, K step after K step, column tile after
// column tile, through a ring of NP stages, exactly as gemm_panel.hip streams both operands:
//   * wavefronts 4-7 only load: first the A panel, then the B steps, up to NP-1 steps ahead of the one being multiplied —
//     with a short K that is a whole tile ahead, so the loads of the next tile are under way before this tile's stores
//     enter the CU's memory queue (the queue is in order: loads issued behind a burst of stores wait for it to drain);
//   * wavefronts 0-3 (2x2) multiply and store; they never wait for a load;
//   * one workgroup barrier per K step, the protocol of gemm_index.hpp (kstream_loader / kstream_consumer).
// The tile walk is the column-block walk of gemm_index.hpp (tiles numbered column block by column block, the workgroups of
// an XCD walking whole column blocks together) with a grid chosen so that every workgroup stays in ONE tile row: the
// launcher makes the number of workgroups per XCD a multiple of the number of tile rows.
// A K that is no multiple of 16: as in gemm_panel.hip (lanes whose k do not exist re-read the step's first chunk; the
// multiplying wavefronts zero those operand registers).  Plain stores only (non-temporal), one matrix (no batches).
#include <algorithm>

#include "gemm_launch.hpp"

namespace tenmo {

constexpr int RESIDENT_THREADS = 512; // four multiplying wavefronts and four loading ones

struct ResidentArgs {
    uint32_t total_tiles, xcds, chunk; // the tile walk (gemm_index.hpp), column-block numbering
    int32_t nk;                        // K steps of 16
    int32_t k_tail;                    // k that exist in the last step: 1..16
};

// NKMAX: K steps the A panel holds; NP: stages of the B ring; WPC: workgroups per CU the LDS allows
template <int AMODE, int BMODE, int BM, int BN, int NKMAX, int NP, int WPC>
__global__ __launch_bounds__(RESIDENT_THREADS, 2 * WPC) void gemm_resident_kernel(const GemmArgs g, const ResidentArgs ra) {
    constexpr int TM = BM / 2, TN = BN / 2;   // wave tile (2x2 multiplying wavefronts)
    constexpr int MB = TM / 32, NB = TN / 32; // 32x32 blocks per wave tile
    constexpr int A_FLOATS = BM * GEMM_BK, B_FLOATS = BN * GEMM_BK;
    using LA = TileLoader<BM, AMODE>;
    using LB = TileLoader<BN, BMODE>;
    constexpr int NA = LA::NCH, NBL = LB::NCH;
    static_assert(NP >= 4 && NP <= 8, "ring of 4 to 8 stages");
    static_assert(NKMAX * NA + (NP - 1) * NBL < 64, "the load counter holds 63");
    static_assert((NKMAX * A_FLOATS + NP * B_FLOATS) * 4 * WPC <= 160 * 1024, "LDS of a CU");
    __shared__ __attribute__((aligned(1024))) float apanel[NKMAX * A_FLOATS];
    __shared__ __attribute__((aligned(1024))) float ring[NP * B_FLOATS];

    const int t = threadIdx.x, lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
    TileWalk walk;
    walk.start(blockIdx.x, gridDim.x, ra.total_tiles, ra.xcds, ra.chunk);
    if (walk.tile() >= ra.total_tiles) return; // (every wavefront of the workgroup alike)
    const int nk = ra.nk;
    const bool ragged_k = ra.k_tail < GEMM_BK;
    const uint32_t tiles_m = (uint32_t)g.tiles_m, tiles_n = (uint32_t)g.tiles_n;

    if (wave >= 4) {
        // ---- a loading wavefront: part `w` of the A panel, then of every B stage ----
        const int w = wave - 4;
        LB lb;
        uint32_t b_tail[NBL]; // lane offsets of the last K step when K is no multiple of 16
        {
            uint32_t b;
            int64_t m0, n0;
            tile_origin(walk.tile(), tiles_m, tiles_n, 1, BM, BN, b, m0, n0);
            LA la;
            uint32_t a_tail[NA];
            la.init_direct(g.A, g.a_rs, g.a_cs, m0, 0, g.M, lane, w);
            la.tail_offsets(g.a_rs, g.a_cs, m0, g.M, lane, w, ra.k_tail, a_tail);
            for (int ks = 0; ks < nk; ++ks) {
                const bool tail = ragged_k && ks == nk - 1;
#pragma unroll
                for (int j = 0; j < NA; ++j) la.load_direct_at(apanel + ks * A_FLOATS, (int64_t)ks * GEMM_BK, w, j, tail ? a_tail[j] : la.lane_off[j]);
            }
        }
        auto init_tile = [&](uint32_t tile) {
            uint32_t b;
            int64_t m0, n0;
            tile_origin(tile, tiles_m, tiles_n, 1, BM, BN, b, m0, n0);
            lb.init_direct(g.B, g.b_cs, g.b_rs, n0, 0, g.N, lane, w);
            lb.tail_offsets(g.b_cs, g.b_rs, n0, g.N, lane, w, ra.k_tail, b_tail);
        };
        auto issue = [&](int slot, int ks) { // K step `ks` of the current tile's B into stage `slot` of the ring
            const bool tail = ragged_k && ks == nk - 1;
#pragma unroll
            for (int j = 0; j < NBL; ++j) lb.load_direct_at(ring + slot * B_FLOATS, (int64_t)ks * GEMM_BK, w, j, tail ? b_tail[j] : lb.lane_off[j]);
        };
        // the panel's loads are older than any stage's: a wait that certifies a stage certifies the panel
        kstream_loader(walk, nk, NP, init_tile, issue, [&](int ahead) {
            switch (ahead) { // at most `ahead` steps of NBL loads outstanding (the immediate must be a constant)
                case 0: __builtin_amdgcn_s_waitcnt(vmcnt_imm(0)); break;
                case 1: __builtin_amdgcn_s_waitcnt(vmcnt_imm(1 * NBL)); break;
                case 2: __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * NBL)); break;
                case 3: __builtin_amdgcn_s_waitcnt(vmcnt_imm(3 * NBL)); break;
                case 4: __builtin_amdgcn_s_waitcnt(vmcnt_imm(4 * NBL)); break;
                case 5: __builtin_amdgcn_s_waitcnt(vmcnt_imm(5 * NBL)); break;
                default: __builtin_amdgcn_s_waitcnt(vmcnt_imm(6 * NBL)); break; // more would be allowed: waiting for fewer is safe
            }
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
    constexpr int PER_MFMA = (PA + PB + NMFMA - 1) / NMFMA;                   // operand fetches placed behind one MFMA
    static_assert(PER_MFMA <= 2, "at most two operand fetches behind an MFMA");

    f32x16 acc[MB][NB];
    float fa[2][MB][4], fb[2][NB][4]; // operand registers of the two k chunks of a step

    const uint32_t row_bytes = (uint32_t)g.N * 4u;
    const int lane_row = wm * TM + (AMODE == MNMAJOR_VEC ? MB : 1) * 4 * h; // row of accumulator element 0 of block row 0
    const int lane_col = wn * TN + (BMODE == MNMAJOR_VEC ? NB * x : x);     // column of block column 0
    const uint32_t lane_byte = (uint32_t)lane_row * row_bytes + (uint32_t)lane_col * 4u;
    // store slot sl = (i, e) of the finished tile whose corner in C is `tile_base` and of which rows x cols exist
    auto store_slot = [&](auto whole_t, char* tile_base, int rows, int cols, int sl) {
        const f32x16 (&src)[MB][NB] = acc;
        constexpr bool WHOLE = decltype(whole_t)::value;
        const int i = sl / 16, e = sl % 16;
        const int c = AMODE == MNMAJOR_VEC ? MB * (8 * (e >> 2) + (e & 3)) + i : 32 * i + 8 * (e >> 2) + (e & 3);
        char* rowp = tile_base + (uint64_t)((uint32_t)c * row_bytes); // uniform
        float* p = reinterpret_cast<float*>(rowp + lane_byte);
        const bool row_ok = WHOLE || lane_row < rows - c;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
            const int dc = BMODE == MNMAJOR_VEC ? j : 32 * j;
            if (WHOLE || (row_ok && lane_col + dc < cols)) __builtin_nontemporal_store(src[i][j][e], p + dc);
        }
    };

    // operand fetch number p (A's parts, then B's) of chunk kc: A from its step of the panel, B from its stage of the ring
    auto fetch_part = [&](const float* a_step, const float* b_stage, int kc, int p) {
        if (p < PA) load_fragment_part<BM, AMODE, MB>(a_step, wm * TM, kc, lane, fa[kc], p);
        else if (p < PA + PB) load_fragment_part<BN, BMODE, NB>(b_stage, wn * TN, kc, lane, fb[kc], p - PA);
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
    // the MFMAs of chunk kc with `slot(n)` placed behind MFMA n (one such sequence per chunk: see gemm_panel.hip)
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
        if (first) { // behind barrier 0: the panel and stage 0 have landed; the first operands of step 0
            first = false;
#pragma unroll
            for (int p = 0; p < PA + PB; ++p) fetch_part(apanel, ring, 0, p);
        }
    };

    kstream_consumer(
        walk, nk, NP, barrier,
        [&](int slot, int next_slot, int ks, bool last_step, int) {
            const float* a_step = apanel + ks * A_FLOATS;
            const float* a_next = last_step ? apanel : a_step + A_FLOATS; // the next tile starts over on the same panel
            const float* b_stage = ring + slot * B_FLOATS;
            const float* b_next = ring + next_slot * B_FLOATS;
            if (ks == 0) {
#pragma unroll
                for (int i = 0; i < MB; ++i)
#pragma unroll
                    for (int j = 0; j < NB; ++j)
#pragma unroll
                        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
            }
            const int klimit = ragged_k && last_step ? ra.k_tail : GEMM_BK;
            if (klimit < GEMM_BK) mask_tail(0, klimit);
            // chunk 0; behind its MFMAs the operand fetch of chunk 1
            mfma_chunk(0, [&](int n) {
#pragma unroll
                for (int q = 0; q < PER_MFMA; ++q)
                    if (n * PER_MFMA + q < PA + PB) fetch_part(a_step, b_stage, 1, n * PER_MFMA + q);
            });
            if (klimit > 8) {
                if (klimit < GEMM_BK) mask_tail(1, klimit);
                // chunk 1; behind its MFMAs the operand fetch of the next step's chunk 0 (harmless when there is no next
                // step: the registers are not used, the addresses lie inside the panel and the ring)
                mfma_chunk(1, [&](int n) {
#pragma unroll
                    for (int q = 0; q < PER_MFMA; ++q)
                        if (n * PER_MFMA + q < PA + PB) fetch_part(a_next, b_next, 0, n * PER_MFMA + q);
                });
            } else {
#pragma unroll
                for (int p = 0; p < PA + PB; ++p) fetch_part(a_next, b_next, 0, p);
            }
        },
        [&](uint32_t tile, int) {
            uint32_t b;
            int64_t m0, n0;
            tile_origin(tile, tiles_m, tiles_n, 1, BM, BN, b, m0, n0);
            char* tile_base = reinterpret_cast<char*>(g.C + m0 * g.N + n0);
            const int rows = (int)min((int64_t)BM, g.M - m0), cols = (int)min((int64_t)BN, g.N - n0);
            if (rows == BM && cols == BN) {
#pragma unroll
                for (int sl = 0; sl < NSLOT; ++sl) store_slot(std::true_type{}, tile_base, rows, cols, sl);
            } else { // a ragged tile (last tile row or column block): lane by lane under its bounds
#pragma unroll
                for (int sl = 0; sl < NSLOT; ++sl) store_slot(std::false_type{}, tile_base, rows, cols, sl);
            }
        });
}

namespace {

template <int AMODE, int BMODE, int BM, int BN, int NKMAX, int NP, int WPC>
bool launch_resident(const GemmArgs& g, unsigned cus, hipStream_t stream) {
    const unsigned tiles_m = (unsigned)g.tiles_m, tiles_n = (unsigned)g.tiles_n;
    // workgroups per XCD: a multiple of the tile rows, so that a workgroup's walk stays in one of them
    const unsigned per_xcd = cus * WPC / 8 / tiles_m * tiles_m;
    if (per_xcd == 0) return false;
    ResidentArgs ra{};
    ra.total_tiles = tiles_m * tiles_n;
    ra.xcds = 8; ra.chunk = tiles_m;
    ra.nk = (int32_t)((g.K + GEMM_BK - 1) / GEMM_BK);
    ra.k_tail = (int32_t)(g.K - (int64_t)(ra.nk - 1) * GEMM_BK);
    if (ra.nk > NKMAX) return false;
    hipLaunchKernelGGL((gemm_resident_kernel<AMODE, BMODE, BM, BN, NKMAX, NP, WPC>), dim3(8 * per_xcd), dim3(RESIDENT_THREADS), 0, stream, g, ra);
    return true;
}

// the panel sizes: up to 128 and up to 256 k; the rings take what LDS is left (two workgroups per CU with 64-row tiles)
template <int AMODE, int BMODE>
bool launch_resident_sizes(const GemmArgs& g, int bm, unsigned cus, hipStream_t stream) {
    const int nk = (int)((g.K + GEMM_BK - 1) / GEMM_BK);
    if (bm == 128) return nk <= 8 ? launch_resident<AMODE, BMODE, 128, 64, 8, 8, 1>(g, cus, stream) : launch_resident<AMODE, BMODE, 128, 64, 16, 7, 1>(g, cus, stream);
    return nk <= 8 ? launch_resident<AMODE, BMODE, 64, 64, 8, 8, 2>(g, cus, stream) : launch_resident<AMODE, BMODE, 64, 64, 16, 4, 2>(g, cus, stream);
}

} // namespace

bool launch_gemm_resident(const GemmArgs& g, int bm, int amode, int bmode, unsigned cus, hipStream_t stream) {
    if (g.K < 1 || g.K > 256 || g.accumulate || (bm != 64 && bm != 128) || bmode != MNMAJOR_VEC) return false;
    if (amode == KMAJOR_VEC) return launch_resident_sizes<KMAJOR_VEC, MNMAJOR_VEC>(g, bm, cus, stream);
    if (amode == MNMAJOR_VEC) return launch_resident_sizes<MNMAJOR_VEC, MNMAJOR_VEC>(g, bm, cus, stream);
    return false;
}

} // namespace tenmo
