// CPU replay of one launch of the persistent K-stream GEMM kernel (tenmo_amd/csrc/gemm_panel.hip): every workgroup,
// wavefront and lane, through the same index arithmetic and the same control-flow templates the kernel uses
// (tenmo_amd/csrc/gemm_index.hpp).  No arithmetic on data: it tracks WHICH element every load brings to which LDS word
// and which element of C every store writes, and checks
//   * every global load lies inside the operand's view (first to last element that belongs to it),
//   * every direct load writes its 16 bytes inside the ring, and one K step fills its stage exactly once,
//   * the loading and the multiplying wavefronts execute the same number of barriers,
//   * the ring protocol: every operand word a multiplying wavefront reads was certified as landed by a barrier it has
//     passed, belongs to the K step it is multiplying, and is not overwritten before the wavefront's next barrier
//     (loader code behind barrier e runs concurrently with consumer code behind barrier e, and only with it),
//   * every operand register holds the element (row, k) the MFMA expects, or is zeroed when k lies beyond K,
//   * every element of C is stored exactly once, in bounds.
// Built by tests/test_kstream_addresses.py with g++; test infrastructure only.
#include <climits>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "../tenmo_amd/csrc/gemm_index.hpp"

using namespace tenmo;

extern "C" {

struct EmuProblem {
    int64_t M, N, K;
    int32_t a_mn_major, b_mn_major; // operand forms: 0 K-major (unit stride along k), 1 MN-major (unit stride along the row index)
    int64_t a_rs, a_cs, b_rs, b_cs; // A(m,k) = A[m*a_rs + k*a_cs], B(k,n) = B[k*b_rs + n*b_cs]
    BatchDesc batch;
    int64_t batch_count;
    int32_t bm, bn, np;             // workgroup tile and ring depth
    uint32_t cus, wgs_per_cu;       // the launch: persistent workgroups per compute unit
    int32_t group_by_xcd;
};

struct EmuReport {
    int64_t loads, lds_reads, stores, steps, workgroups;
    char message[512];
};

int emulate_kstream(const EmuProblem* pp, EmuReport* rep);
}

namespace {

struct Fail {
    char msg[512];
};

#define CHECK(cond, ...)                                   \
    do {                                                   \
        if (!(cond)) {                                     \
            Fail f;                                        \
            snprintf(f.msg, sizeof f.msg, __VA_ARGS__);    \
            throw f;                                       \
        }                                                  \
    } while (0)

// first and last element offset (from the operand pointer) that belongs to a view [batch..., rows, k]
void view_extent(const BatchDesc& bd, bool is_a, int64_t rows, int64_t K, int64_t row_s, int64_t k_s, int64_t& lo, int64_t& hi) {
    lo = 0; hi = 0;
    auto span = [&](int64_t extent, int64_t stride) {
        if (extent <= 0) return;
        const int64_t d = (extent - 1) * stride;
        if (d < 0) lo += d; else hi += d;
    };
    span(rows, row_s);
    span(K, k_s);
    for (int d = 0; d < bd.rank; ++d) span(bd.shape[d], is_a ? bd.a_str[d] : bd.b_str[d]);
}

struct LdsWord {
    int64_t elem = -1;   // element offset loaded into this word
    int32_t unit = -1;   // K-stream step it belongs to
    int32_t epoch = -1;  // loader epoch (barriers passed) in which the load was issued
    int32_t certified = -1; // first barrier before which the loaders waited for it (-1: not yet)
};

template <int BM, int BN>
void run(const EmuProblem& P, EmuReport& R) {
    constexpr int STAGE = (BM + BN) * INDEX_BK, A_FLOATS = BM * INDEX_BK;
    constexpr int TM = BM / 2, TN = BN / 2, MB = TM / 32, NB = TN / 32;
    constexpr int NCH_A = BM / 64, NCH_B = BN / 64;
    const int NP = P.np;
    const int nk = (int)((P.K + INDEX_BK - 1) / INDEX_BK);
    const int k_tail = (int)(P.K - (int64_t)(nk - 1) * INDEX_BK);
    const bool ragged_k = k_tail < INDEX_BK;
    const uint32_t tiles_m = (uint32_t)((P.M + BM - 1) / BM), tiles_n = (uint32_t)((P.N + BN - 1) / BN);
    const uint32_t total_tiles = tiles_m * tiles_n * (uint32_t)P.batch_count;
    const TileWalkPlan plan = plan_tile_walk(total_tiles, tiles_m, tiles_n, P.cus, P.wgs_per_cu, P.group_by_xcd != 0);
    // operands in (row, k) form, as the kernel sees them
    const int64_t a_row_s = P.a_rs, a_k_s = P.a_cs, b_row_s = P.b_cs, b_k_s = P.b_rs;
    int64_t a_lo, a_hi, b_lo, b_hi;
    view_extent(P.batch, true, P.M, P.K, a_row_s, a_k_s, a_lo, a_hi);
    view_extent(P.batch, false, P.N, P.K, b_row_s, b_k_s, b_lo, b_hi);
    std::vector<uint8_t> written((size_t)(P.batch_count * P.M * P.N), 0);

    for (uint32_t wg = 0; wg < plan.grid; ++wg) {
        TileWalk walk;
        walk.start(wg, plan.grid, total_tiles, plan.xcds, plan.chunk);
        if (walk.tile() >= total_tiles) continue;
        ++R.workgroups;
        std::vector<LdsWord> lds((size_t)NP * STAGE);

        // ---- loader side: records, per step of the stream, the words it fills; epochs and certifications ----
        struct Issue { int slot, ks, epoch; uint32_t tile; };
        std::vector<Issue> issues;          // index = stream step
        std::vector<int> certified_by;      // stream step -> first barrier that certifies it
        int loader_barriers = 0;
        {
            uint32_t cur_tile = 0;
            kstream_loader(
                walk, nk, NP,
                [&](uint32_t tile) { cur_tile = tile; },
                [&](int slot, int ks) { issues.push_back({slot, ks, loader_barriers, cur_tile}); certified_by.push_back(-1); },
                [&](int ahead) {
                    // loads complete in issue order: everything but the last `ahead` steps has landed
                    const int done = (int)issues.size() - ahead;
                    for (int u = 0; u < done; ++u)
                        if (certified_by[u] < 0) certified_by[u] = loader_barriers;
                    ++loader_barriers;
                });
        }
        R.steps += (int64_t)issues.size();
        CHECK(loader_barriers == (int)issues.size(), "workgroup %u: %d loader barriers for %zu steps", wg, loader_barriers, issues.size());

        // the loads of stream step u, lane by lane: fills `lds` (called in consumer order below, see the protocol check)
        auto perform_issue = [&](int u) {
            const Issue& is = issues[u];
            uint32_t b;
            int64_t m0, n0, a_boff, b_boff;
            tile_origin(is.tile, tiles_m, tiles_n, plan.col_major, BM, BN, b, m0, n0);
            batch_offsets(P.batch, b, a_boff, b_boff);
            const bool tail = ragged_k && is.ks == nk - 1;
            std::vector<uint8_t> filled(STAGE, 0);
            for (int operand = 0; operand < 2; ++operand) {
                const bool mn = operand ? P.b_mn_major : P.a_mn_major;
                const int64_t rs = operand ? b_row_s : a_row_s, ks_ = operand ? b_k_s : a_k_s;
                const int64_t row0 = operand ? n0 : m0, Rext = operand ? P.N : P.M, boff = operand ? b_boff : a_boff;
                const int64_t lo = operand ? b_lo : a_lo, hi = operand ? b_hi : a_hi;
                const int nch = operand ? NCH_B : NCH_A;
                const int base_word = is.slot * STAGE + (operand ? A_FLOATS : 0);
                // origin as TileLoader::init_direct computes it, advanced by the K step
                const int64_t origin = mn ? boff + (int64_t)is.ks * INDEX_BK * ks_ + row0 : boff + row0 * rs + (int64_t)is.ks * INDEX_BK;
                for (int w = 0; w < 4; ++w)
                    for (int j = 0; j < nch; ++j) {
                        const int part = w * nch + j;
                        for (int lane = 0; lane < 64; ++lane) {
                            uint32_t off;
                            const int kv = tail ? k_tail : INDEX_BK;
                            if (operand == 0) off = mn ? direct_lane_off_mnmajor<BM>(ks_, row0, Rext, lane, part, kv) : direct_lane_off_kmajor<BM>(rs, row0, Rext, lane, part, kv);
                            else off = mn ? direct_lane_off_mnmajor<BN>(ks_, row0, Rext, lane, part, kv) : direct_lane_off_kmajor<BN>(rs, row0, Rext, lane, part, kv);
                            CHECK(off % 4 == 0, "lane offset not a multiple of 4 bytes");
                            const int64_t e0 = origin + off / 4;
                            CHECK(e0 >= lo && e0 + 3 <= hi, "workgroup %u step %d operand %c part %d lane %d: load of elements [%lld, %lld] outside the view [%lld, %lld]",
                                  wg, u, operand ? 'B' : 'A', part, lane, (long long)e0, (long long)(e0 + 3), (long long)lo, (long long)hi);
                            const int word = part * 256 + 4 * lane; // 1 KiB per part, 16 bytes per lane
                            CHECK(word + 3 < (operand ? BN : BM) * INDEX_BK, "LDS destination beyond the operand's stage");
                            for (int q = 0; q < 4; ++q) {
                                LdsWord& wd = lds[base_word + word + q];
                                wd.elem = e0 + q; wd.unit = u; wd.epoch = is.epoch; wd.certified = certified_by[u];
                                CHECK(!filled[(operand ? A_FLOATS : 0) + word + q], "stage word filled twice in one step");
                                filled[(operand ? A_FLOATS : 0) + word + q] = 1;
                            }
                            ++R.loads;
                        }
                    }
            }
            for (int i = 0; i < STAGE; ++i) CHECK(filled[i], "workgroup %u step %d: stage word %d not filled", wg, u, i);
        };
        // when (in loader epochs) is the stage of step u overwritten next?  by step u + NP
        auto overwritten_epoch = [&](int u) { return u + NP < (int)issues.size() ? issues[u + NP].epoch : INT32_MAX; };

        // ---- consumer side ----
        int consumer_barriers = 0, unit = 0;
        int next_issue = 0; // steps whose loads have been replayed into `lds`
        // replay loads so that the ring holds what a consumer in epoch `e` may see at the latest: every step issued in a
        // loader epoch <= e has been written (older contents of its stage are gone)
        auto advance_lds = [&](int epoch) {
            while (next_issue < (int)issues.size() && issues[next_issue].epoch <= epoch) perform_issue(next_issue++);
        };
        auto read_fragment = [&](int slot, int of_unit, int ks, uint32_t tile, int kc, bool zeroed_beyond_k) {
            // one operand fetch of chunk kc of stream step `of_unit` by all four multiplying wavefronts, in consumer epoch
            // `consumer_barriers` (barriers passed so far)
            const int epoch = consumer_barriers;
            uint32_t b;
            int64_t m0, n0, a_boff, b_boff;
            tile_origin(tile, tiles_m, tiles_n, plan.col_major, BM, BN, b, m0, n0);
            batch_offsets(P.batch, b, a_boff, b_boff);
            for (int wave = 0; wave < 4; ++wave) {
                const int wm = wave >> 1, wn = wave & 1;
                for (int lane = 0; lane < 64; ++lane)
                    for (int operand = 0; operand < 2; ++operand) {
                        const bool mn = operand ? P.b_mn_major : P.a_mn_major;
                        const int rows = operand ? BN : BM, nblk = operand ? NB : MB, wave_row0 = operand ? wn * TN : wm * TM;
                        const int base_word = slot * STAGE + (operand ? A_FLOATS : 0);
                        for (int blk = 0; blk < nblk; ++blk)
                            for (int s = 0; s < 4; ++s) {
                                const int word = mn ? frag_off_mnmajor(rows, nblk, wave_row0, kc, lane, s) + blk : frag_off_kmajor(wave_row0, kc, lane, blk) + s;
                                CHECK(word >= 0 && word < rows * INDEX_BK, "operand fetch outside the tile");
                                const LdsWord& wd = lds[base_word + word];
                                ++R.lds_reads;
                                CHECK(wd.unit == of_unit, "workgroup %u: fetch in epoch %d for step %d finds step %d in the stage", wg, epoch, of_unit, wd.unit);
                                CHECK(wd.certified >= 0 && wd.certified < epoch, "workgroup %u: step %d read in epoch %d but certified by barrier %d", wg, of_unit, epoch, wd.certified);
                                CHECK(overwritten_epoch(of_unit) > epoch, "workgroup %u: stage of step %d may be overwritten in epoch %d while it is read", wg, of_unit, epoch);
                                // the element the MFMA expects here
                                const int64_t row = (operand ? n0 : m0) + wave_row0 + wave_tile_pos(mn, nblk, blk, lane & 31);
                                const int64_t k = (int64_t)ks * INDEX_BK + 8 * kc + 4 * (lane >> 5) + s;
                                const int64_t Rext = operand ? P.N : P.M;
                                if (row >= Rext) continue;          // clamped rows: never stored
                                if (k >= P.K) { CHECK(zeroed_beyond_k, "operand beyond K is not zeroed"); continue; }
                                const int64_t want = (operand ? b_boff : a_boff) + row * (operand ? b_row_s : a_row_s) + k * (operand ? b_k_s : a_k_s);
                                CHECK(wd.elem == want, "workgroup %u step %d %c(row %lld, k %lld): register holds element %lld, expected %lld", wg, of_unit,
                                      operand ? 'B' : 'A', (long long)row, (long long)k, (long long)wd.elem, (long long)want);
                            }
                    }
            }
        };
        struct Pending { bool valid = false; uint32_t tile = 0; } pend;
        auto store_tile = [&](uint32_t tile) {
            uint32_t b;
            int64_t m0, n0;
            tile_origin(tile, tiles_m, tiles_n, plan.col_major, BM, BN, b, m0, n0);
            const int rows = (int)imin64(BM, P.M - m0), cols = (int)imin64(BN, P.N - n0);
            for (int wave = 0; wave < 4; ++wave) {
                const int wm = wave >> 1, wn = wave & 1;
                for (int lane = 0; lane < 64; ++lane) {
                    const int h = lane >> 5, x = lane & 31;
                    const int lane_row = wm * TM + (P.a_mn_major ? MB : 1) * 4 * h;
                    const int lane_col = wn * TN + (P.b_mn_major ? NB * x : x);
                    for (int sl = 0; sl < MB * 16; ++sl) {
                        const int i = sl / 16, e = sl % 16;
                        const int c = P.a_mn_major ? MB * (8 * (e >> 2) + (e & 3)) + i : 32 * i + 8 * (e >> 2) + (e & 3);
                        // the kernel's constants must agree with the accumulator layout
                        CHECK(lane_row + c == wm * TM + wave_tile_pos(P.a_mn_major, MB, i, mfma_row(e, lane)), "store row formula disagrees with the MFMA layout");
                        for (int j = 0; j < NB; ++j) {
                            const int dc = P.b_mn_major ? j : 32 * j;
                            CHECK(lane_col + dc == wn * TN + wave_tile_pos(P.b_mn_major, NB, j, x), "store column formula disagrees with the MFMA layout");
                            if (!(lane_row + c < rows && lane_col + dc < cols)) continue;
                            const int64_t row = m0 + lane_row + c, col = n0 + lane_col + dc;
                            CHECK(row < P.M && col < P.N, "store outside C");
                            const int64_t byte = ((int64_t)lane_row * P.N + lane_col) * 4 + (int64_t)c * P.N * 4 + dc * 4;
                            CHECK(byte >= 0 && byte <= 0xffffffffLL, "store offset exceeds 32 bits");
                            uint8_t& wflag = written[(size_t)(((int64_t)b * P.M + row) * P.N + col)];
                            CHECK(!wflag, "element (%u, %lld, %lld) of C stored twice", b, (long long)row, (long long)col);
                            wflag = 1;
                            ++R.stores;
                        }
                    }
                }
            }
        };
        // the fetches of one step, in the order and epochs the kernel performs them:
        //   chunk 0 of step u: behind barrier 0 for u = 0, else during step u-1 (before barrier u)
        //   chunk 1 of step u: during step u (behind barrier u)
        kstream_consumer(
            walk, nk, NP,
            [&]() {
                ++consumer_barriers;
                advance_lds(consumer_barriers);
            },
            [&](int slot, int next_slot, int ks, bool last_step, int) {
                const int epoch_here = consumer_barriers;
                (void)epoch_here;
                const Issue& is = issues[unit];
                CHECK(is.slot == slot && is.ks == ks, "workgroup %u: consumer step %d (stage %d, k step %d) but the loaders put it in stage %d as k step %d", wg, unit, slot, ks, is.slot, is.ks);
                const bool tail = ragged_k && last_step;
                if (unit == 0) read_fragment(slot, 0, ks, is.tile, 0, tail);
                const bool second = !(tail && k_tail <= 8);
                if (second) read_fragment(slot, unit, ks, is.tile, 1, tail);
                if (unit + 1 < (int)issues.size()) {
                    const Issue& nx = issues[unit + 1];
                    CHECK(nx.slot == next_slot, "next stage mismatch");
                    read_fragment(next_slot, unit + 1, nx.ks, nx.tile, 0, ragged_k && nx.ks == nk - 1);
                }
                if (pend.valid) { store_tile(pend.tile); pend.valid = false; }
                ++unit;
            },
            [&](uint32_t tile, int) { pend.valid = true; pend.tile = tile; });
        if (pend.valid) store_tile(pend.tile);
        CHECK(unit == (int)issues.size(), "workgroup %u multiplied %d steps, the loaders issued %zu", wg, unit, issues.size());
        CHECK(consumer_barriers == loader_barriers, "workgroup %u: %d consumer barriers, %d loader barriers", wg, consumer_barriers, loader_barriers);
    }
    for (size_t i = 0; i < written.size(); ++i) CHECK(written[i], "element %zu of C never stored", i);
}

} // namespace

extern "C" int emulate_kstream(const EmuProblem* pp, EmuReport* rep) {
    memset(rep, 0, sizeof *rep);
    try {
        if (pp->bm == 128 && pp->bn == 128) run<128, 128>(*pp, *rep);
        else if (pp->bm == 128 && pp->bn == 64) run<128, 64>(*pp, *rep);
        else if (pp->bm == 64 && pp->bn == 128) run<64, 128>(*pp, *rep);
        else if (pp->bm == 64 && pp->bn == 64) run<64, 64>(*pp, *rep);
        else { snprintf(rep->message, sizeof rep->message, "no such tile %dx%d", pp->bm, pp->bn); return 2; }
    } catch (const Fail& f) {
        memcpy(rep->message, f.msg, sizeof rep->message);
        return 1;
    }
    return 0;
}
