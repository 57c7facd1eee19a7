// Index arithmetic of the GEMM kernels that decides which bytes a lane touches: LDS tile layouts, the per-lane
// source offsets of the direct global->LDS loads, the order in which persistent workgroups walk tiles, and which
// elements of C a lane stores.  Plain integer functions with no GPU builtins, usable from device code and from a
// host compiler alike: the kernels call them, and a CPU test replays them lane by lane over whole launches and
// checks every address against the operands' extents.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define TENMO_HD __host__ __device__ __forceinline__
#else
#define TENMO_HD inline
#endif

namespace tenmo {

constexpr int INDEX_BK = 16; // K step of every tiled kernel (GEMM_BK)

constexpr int MAX_BATCH_RANK = 6;

TENMO_HD int64_t imin64(int64_t a, int64_t b) { return a < b ? a : b; }

// Broadcast batch dimensions of a product, folded into the grid: the result's batch shape and, per operand, the stride
// of each batch dimension in elements (0 where that operand's dimension is 1 or missing).
struct BatchDesc {
    int32_t rank;
    int64_t shape[MAX_BATCH_RANK];
    int64_t a_str[MAX_BATCH_RANK];
    int64_t b_str[MAX_BATCH_RANK];
};

// Element offsets of batch number b in the two operands.  The batch index and every batch dimension are below 2^31
// (the host refuses larger grids), so the mixed-radix decode runs in 32-bit arithmetic: a 64-bit division costs a
// workgroup hundreds of instructions before its first load.
TENMO_HD void batch_offsets(const BatchDesc& bd, int64_t b, int64_t& a_off, int64_t& b_off) {
    a_off = 0; b_off = 0;
    uint32_t rest = (uint32_t)b;
    for (int d = bd.rank - 1; d >= 0; --d) {
        const uint32_t extent = (uint32_t)bd.shape[d];
        const uint32_t q = rest / extent;
        const int64_t c = rest - q * extent;
        rest = q;
        a_off += c * bd.a_str[d];
        b_off += c * bd.b_str[d];
    }
}

// float offset of 16-byte chunk q (0..3) of `row` in a K-major tile [row][16 k], chunks XOR-swizzled by (row>>2)&3
TENMO_HD int kmajor_off(int row, int q) { return 4 * (4 * row + (q ^ ((row >> 2) & 3))); }

// ---- direct loads of one ROWS x 16 operand tile -------------------------------------------------------------
// The tile is moved by ROWS/16 wave-loads ("parts") of 1 KiB; lane l of part p writes LDS bytes [1024p + 16l, +16).
// The source of part p is a wave-uniform origin plus a per-lane byte offset:
//   K-major  (element (row, k) at base[row*rs + k]):  origin = base + row0*rs + k_begin, and lane l moves chunk
//            q = (l&3) ^ ((l>>4)&3) of row 16p + (l>>2) (the swizzle of kmajor_off); rows at or beyond the extent R are
//            clamped onto row R-1 (their products are never stored)
//   MN-major (element (row, k) at base[k*ks + row]):  origin = base + k_begin*ks + row0, and lane l moves 4 rows starting
//            at (4l) % ROWS of k row p*(256/ROWS) + (4l)/ROWS; rows are clamped onto R-4 (needs R % 4 == 0, R >= 4)
// `k_valid` (1..16) is the number of k of this step that exist (16 except in the last step of a K that is no multiple
// of 16): a lane whose k lie at or beyond it reads the step's first chunk / first k row instead (always valid), and the
// consumer discards what it brought.  A K-major operand then needs K % 4 == 0, so that no chunk straddles K.
template <int ROWS>
TENMO_HD uint32_t direct_lane_off_kmajor(int64_t rs, int64_t row0, int64_t R, int lane, int part, int k_valid = INDEX_BK) {
    int q = (lane & 3) ^ ((lane >> 4) & 3);
    if (4 * q + 4 > k_valid) q = 0;
    const int64_t row = imin64(row0 + part * 16 + (lane >> 2), R - 1);
    return (uint32_t)(((row - row0) * rs + 4 * q) * 4);
}

template <int ROWS>
TENMO_HD uint32_t direct_lane_off_mnmajor(int64_t ks, int64_t row0, int64_t R, int lane, int part, int k_valid = INDEX_BK) {
    constexpr int KROWS = 256 / ROWS > 0 ? 256 / ROWS : 1; // k rows per part
    const int64_t row = imin64(row0 + (4 * lane) % ROWS, R - 4);
    int kk = part * KROWS + (4 * lane) / ROWS;
    if (kk >= k_valid) kk = 0;
    return (uint32_t)((kk * ks + (row - row0)) * 4);
}

// ---- LDS -> MFMA operand registers --------------------------------------------------------------------------
// v_mfma_f32_32x32x2 takes from lane l the operand element (index i = l & 31, k = l >> 5).  Within every 8-wide k chunk kc
// of a stage the kernels give MFMA step s (0..3) of lane half h = l >> 5 the index k = 8 kc + 4 h + s, so that
//   a K-major tile is fetched with one 16-byte read per 32x32 block b: the 4 consecutive k (steps 0..3) of row
//       wave_row0 + 32 b + i, at frag_off_kmajor (floats from the tile's start);
//   an MN-major tile with one read per step s: the nblk consecutive rows wave_row0 + nblk i + b (b = 0..nblk-1) of k row
//       8 kc + 4 h + s, at frag_off_mnmajor.
TENMO_HD int frag_off_kmajor(int wave_row0, int kc, int lane, int b) { return kmajor_off(wave_row0 + 32 * b + (lane & 31), 2 * kc + (lane >> 5)); }
TENMO_HD int frag_off_mnmajor(int rows, int nblk, int wave_row0, int kc, int lane, int s) {
    return (kc * 8 + 4 * (lane >> 5) + s) * rows + wave_row0 + nblk * (lane & 31);
}

// ---- the order in which a persistent grid walks tiles -------------------------------------------------------
// Workgroup ids are dealt round-robin to `xcds` groups (the 8 XCDs of the chip, or 1 for a plain round-robin over the
// grid); the workgroups of one group walk `chunk` consecutive tile numbers together (one batch, or one column block),
// then the chunk `xcds` further on, so that a group's L2 reads the operands of its own chunks only.
struct TileWalk {
    uint32_t total, xcds, chunk, per_xcd, xcd, q;
    TENMO_HD void start(uint32_t block, uint32_t grid, uint32_t total_tiles, uint32_t xcds_, uint32_t chunk_) {
        total = total_tiles; xcds = xcds_; chunk = chunk_;
        per_xcd = grid / xcds; xcd = block % xcds; q = block / xcds;
    }
    // tile number at this workgroup's current position; increasing along the walk; >= total: the walk is over
    TENMO_HD uint32_t tile() const {
        const uint32_t c = q / chunk;
        const uint64_t tl = ((uint64_t)c * xcds + xcd) * chunk + (q - c * chunk);
        return tl < total ? (uint32_t)tl : total;
    }
    TENMO_HD void advance() { q += per_xcd; }
};

// The grid of a persistent launch over `total_tiles` tiles (batches x tiles_m x tiles_n) and the walk its workgroups
// take.  With 8 or more batches the workgroups of an XCD take whole batches; else, with fewer than 8 tile-rows and many
// tile-columns, whole column blocks (tiles then numbered column block by column block): a panel of B is fetched by one
// L2.  Both need a grid divisible by the 8 XCDs; otherwise the tiles are dealt round-robin over the grid.
struct TileWalkPlan {
    uint32_t grid, xcds, chunk;
    int32_t col_major;
};
TENMO_HD TileWalkPlan plan_tile_walk(uint32_t total_tiles, uint32_t tiles_m, uint32_t tiles_n, uint32_t cus, uint32_t wgs_per_cu, bool group_by_xcd) {
    TileWalkPlan p;
    p.grid = total_tiles < cus * wgs_per_cu ? total_tiles : cus * wgs_per_cu;
    p.xcds = 1; p.chunk = 1; p.col_major = 0;
    const uint32_t per_batch = tiles_m * tiles_n;
    if (group_by_xcd && p.grid % 8 == 0 && per_batch > 0) {
        if (total_tiles / per_batch >= 8) { p.xcds = 8; p.chunk = per_batch; }
        else if (tiles_m < 8 && tiles_n >= 64) { p.xcds = 8; p.chunk = tiles_m; p.col_major = 1; }
    }
    return p;
}

// batch and first row / column of tile number `tl`: tiles are numbered batch by batch, inside a batch row by row
// (or column block by column block when `col_major`)
TENMO_HD void tile_origin(uint32_t tl, uint32_t tiles_m, uint32_t tiles_n, int col_major, int bm, int bn, uint32_t& batch, int64_t& m0, int64_t& n0) {
    const uint32_t per_batch = tiles_m * tiles_n;
    batch = tl / per_batch;
    const uint32_t r = tl - batch * per_batch;
    uint32_t tm, tn;
    if (col_major) { tn = r / tiles_m; tm = r - tn * tiles_m; }
    else { tm = r / tiles_n; tn = r - tm * tiles_n; }
    m0 = (int64_t)tm * bm;
    n0 = (int64_t)tn * bn;
}

// ---- the K-stream of a persistent workgroup (gemm_panel.hip) ------------------------------------------------
// The K steps of all the tiles of a workgroup's walk form one stream, step u of it living in ring stage u % np.
// Loading wavefronts run kstream_loader, multiplying wavefronts kstream_consumer; both meet at one workgroup barrier per
// step.  Barrier u: steps u and u+1 have landed (the loaders waited for them), and the consumers are done with step u-1,
// whose stage the loaders refill with step u+np-1 right behind the barrier.  Both sides execute exactly as many
// barriers as the stream has steps.
//   init_tile(tile)      a tile of the walk begins (loader side)
//   issue(slot, ks)      start the loads of K step `ks` of the current tile into ring stage `slot`
//   wait_barrier(ahead)  wait until at most `ahead` issued steps are still in flight, then the workgroup barrier
template <class InitTile, class Issue, class WaitBarrier>
TENMO_HD void kstream_loader(TileWalk walk, int nk, int np, InitTile&& init_tile, Issue&& issue, WaitBarrier&& wait_barrier) {
    int ks = 0, slot = 0, issued = 0;
    bool more = true;
    auto next = [&]() {
        issue(slot, ks);
        slot = slot + 1 == np ? 0 : slot + 1;
        ++issued;
        if (++ks == nk) {
            ks = 0;
            walk.advance();
            if (walk.tile() >= walk.total) more = false;
            else init_tile(walk.tile());
        }
    };
    init_tile(walk.tile());
    for (int i = 0; i < np - 1 && more; ++i) next();
    for (int u = 0; u < issued; ++u) {
        const int ahead = issued - (u + 2);
        wait_barrier(ahead > 0 ? ahead : 0);
        if (more) next();
    }
}
//   barrier()                              the workgroup barrier
//   step(slot, next_slot, ks, last_step, parity)   multiply K step `ks` of the current tile from stage `slot`; the first operands
//                                          of the following step may be fetched from `next_slot` (they have landed)
//   tile_end(tile, parity)                 the step just multiplied was the tile's last
// `parity` alternates 0, 1 from tile to tile of the walk (two sets of accumulators take turns).
template <class Barrier, class Step, class TileEnd>
TENMO_HD void kstream_consumer(TileWalk walk, int nk, int np, Barrier&& barrier, Step&& step, TileEnd&& tile_end) {
    int ks = 0, slot = 0, parity = 0;
    barrier();
    for (;;) {
        const int next_slot = slot + 1 == np ? 0 : slot + 1;
        const bool last_step = ks == nk - 1;
        bool have_next = true;
        if (last_step) {
            TileWalk peek = walk;
            peek.advance();
            have_next = peek.tile() < walk.total;
        }
        step(slot, next_slot, ks, last_step, parity);
        if (last_step) tile_end(walk.tile(), parity);
        if (!have_next) break;
        if (last_step) { walk.advance(); ks = 0; parity ^= 1; }
        else ++ks;
        slot = next_slot;
        barrier();
    }
}

// ---- which element of C an accumulator register holds -------------------------------------------------------
// v_mfma_f32_32x32x2 leaves, in lane l, element e (0..15) of a 32x32 block at block row 8(e>>2) + 4(l>>5) + (e&3) and
// block column l & 31.
TENMO_HD int mfma_row(int e, int lane) { return 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3); }
// position inside the wave tile of index x (0..31) of block b of nblk: an MN-major operand interleaves its blocks
// (block b owns positions nblk*x + b), a K-major one stacks them
TENMO_HD int wave_tile_pos(bool mn_major, int nblk, int b, int x) { return mn_major ? nblk * x + b : 32 * b + x; }

} // namespace tenmo
