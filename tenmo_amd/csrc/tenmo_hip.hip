// libtenmo_hip.so — host side of the C ABI declared in include/tenmo_hip.h.
//
// Shape validation, broadcast-batch resolution and kernel selection happen here; the arithmetic is
// in gemm_mfma.hpp (matrix cores), gemv.hpp (HBM-bound products) and elementwise.hpp.
// This file is what the bodies of the reference's launch functions become:
//   MatmulNdGpu.launch          tenmo/kernels/matmul_kernel.mojo:128-283
//   MatrixVectorNdGpu.launch    tenmo/kernels/matrixvector_kernel.mojo:80-171
//   VectorMatmulNdGpu.launch    tenmo/kernels/vectormatrix_kernel.mojo:80-170
// plus the backward entries that the reference runs through the same launches
// (tenmo/matmul.mojo:22-54, :99-137) and the CBLAS prototype it already binds
// (tenmo/blashandle.mojo:136-151).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <numeric>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/tenmo_hip.h"
#include "cross_entropy.hpp"
#include "gemm_launch.hpp"
#include "elementwise.hpp"
#include "gemv.hpp"

using namespace tenmo;

// Device memory of the allocation-free entry point (tenmo_hip_vm_f32_noalloc): the partial sums of its K slices.
// One copy per GPU, at its own address there, held until the process ends.  Host code never uses this name as an
// address: tenmo_hip_init asks each device for the array's address once and keeps it in `g_scratch_ptr`.
constexpr size_t TENMO_STATIC_SCRATCH_BYTES = TENMO_VM_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) float scratch[TENMO_STATIC_SCRATCH_BYTES / sizeof(float)];

namespace {

constexpr int kMaxDevices = 64;
float* g_scratch_ptr[kMaxDevices] = {nullptr}; // device id -> address of `scratch` on that device (survives shutdown / re-init)

thread_local std::string t_err;

int fail(int code, const char* fmt, ...) {
    char buf[1024];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    t_err = buf;
    return code;
}

#define HIP_TRY(expr)                                                                              \
    do {                                                                                           \
        hipError_t e_ = (expr);                                                                    \
        if (e_ != hipSuccess) return fail(TENMO_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

struct State {
    bool ready = false;
    int device = -1;
    int cus = 0;
    std::string name;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    // grow-only device scratch: split-K / column-split partials, batched gradients before reduction
    float* ws = nullptr;
    size_t ws_bytes = 0;
    // second scratch, for results that must outlive a kernel which itself uses `ws`
    float* ws2 = nullptr;
    uint32_t* arrivals = nullptr; // zeroed counters of the in-launch K-slice reduction of the column kernels
    size_t ws2_bytes = 0;
    // staging buffers of the host-pointer CBLAS entry point
    float* stage[3] = {nullptr, nullptr, nullptr};
    size_t stage_bytes[3] = {0, 0, 0};
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    bool capturing = false;  // a stream capture is open: the scratch cannot grow (no allocation inside a capture)
    size_t ws_wanted = 0;    // what a kernel selection inside a capture asked of the first scratch buffer
    float* one = nullptr; // device constant 1.0f: a stride-0 vector of ones for column sums
    int32_t* conv_tables = nullptr;  // offset tables [C_in*KH*KW | H_out*W_out] of the last convolution geometry
    size_t conv_tables_len = 0;      // capacity in entries
    ConvGeometry conv_geometry{};    // the geometry the tables hold (c_in == 0: none)
    // tuning overrides (environment, read once): -1 = automatic
    int force_tile = -1;
    int force_splitk = -1;
    int force_conv_phases = -1; // strided image gradient phase by phase: -1 automatic (large layers), 0 never, 1 always
    int force_streamk = -1;    // -1 automatic, 0 never, n > 0: stream-K with n workgroups per CU
    int force_smallk = -1;     // -1 automatic, 0 never, 1: the short-reduction kernel wherever it can run (2: without XCD grouping, 3: also for K <= 16)
    int force_resident = 0;    // the resident-A kernel for a few tile rows against a very wide B: 1 with 128x64 tiles, 2 with 64x64, 0 never
    int force_panel = -1;      // -1 automatic, 0 never, 1: the persistent K-stream kernel wherever it can run (2: without XCD grouping, 3: 64x64 tiles)
    int mlp_fused_tail = 0;    // MLP step: 1 the last two layers, loss, their backward and update in one launch when the shapes fit; 2 also the first layer's weight gradient and update in one; 3 also the first layer's forward in one; 0 neither
    int fold_reduce = -1;      // the gradient of a broadcast parent summed inside the GEMM launch: -1 automatic, 0 never, 1 wherever it can
    int verbose = 0;
    int cols_join = 0;         // column kernels: 1 the K slices are added by the last workgroup of the streaming launch, 0 by a second launch
    int cols_waves_per_cu = 2; // target workgroups per CU of the column-streaming kernels (long K slices stream best)
};
State S;
std::mutex S_mu;

int env_int(const char* name, int dflt) {
    const char* v = getenv(name);
    return v && *v ? atoi(v) : dflt;
}

int ensure_ready() {
    if (!S.ready) return fail(TENMO_ERR_NOT_INITIALIZED, "tenmo_hip: not initialised, call tenmo_hip_init(device_id) first");
    return 0;
}

int workspace(size_t bytes, float** out) {
    if (bytes > S.ws_bytes && S.capturing) { // the caller ends the capture, grows the buffer and captures again
        S.ws_wanted = std::max(S.ws_wanted, bytes);
        return fail(TENMO_ERR_HIP, "library scratch of %zu bytes wanted inside a stream capture (have %zu)", bytes, S.ws_bytes);
    }
    if (bytes > S.ws_bytes) {
        if (S.ws) {
            HIP_TRY(hipStreamSynchronize(S.stream));
            HIP_TRY(hipFree(S.ws));
            S.ws = nullptr; S.ws_bytes = 0;
        }
        size_t want = std::max(bytes, (size_t)64 << 20);
        HIP_TRY(hipMalloc(&S.ws, want));
        S.ws_bytes = want;
    }
    *out = S.ws;
    return 0;
}

int workspace2(size_t bytes, float** out) {
    if (bytes > S.ws2_bytes) {
        if (S.ws2) {
            HIP_TRY(hipStreamSynchronize(S.stream));
            HIP_TRY(hipFree(S.ws2));
            S.ws2 = nullptr; S.ws2_bytes = 0;
        }
        HIP_TRY(hipMalloc(&S.ws2, bytes));
        S.ws2_bytes = bytes;
    }
    *out = S.ws2;
    return 0;
}

int finish(int32_t sync) {
    HIP_TRY(hipGetLastError());
    if (sync) HIP_TRY(hipStreamSynchronize(S.stream));
    return 0;
}

std::string shape_str(const int64_t* s, int r) {
    std::string o = "(";
    for (int i = 0; i < r; ++i) o += (i ? ", " : "") + std::to_string(s[i]);
    return o + ")";
}

int64_t product(const int64_t* s, int r) {
    int64_t p = 1;
    for (int i = 0; i < r; ++i) p *= s[i];
    return p;
}

int fill_batch(BatchDesc& bd, int32_t rank, const int64_t* shape, const int64_t* a_str, const int64_t* b_str, int64_t* count) {
    if (rank < 0 || rank > MAX_BATCH_RANK) return fail(TENMO_ERR_INVALID_ARGUMENT, "batch rank %d outside 0..%d", rank, MAX_BATCH_RANK);
    if (rank > 0 && (!shape || !a_str || !b_str)) return fail(TENMO_ERR_INVALID_ARGUMENT, "batch_rank > 0 needs batch_shape and both batch stride arrays");
    bd.rank = rank;
    int64_t n = 1;
    for (int d = 0; d < MAX_BATCH_RANK; ++d) {
        bd.shape[d] = d < rank ? shape[d] : 1;
        bd.a_str[d] = d < rank ? a_str[d] : 0;
        bd.b_str[d] = d < rank ? b_str[d] : 0;
        if (d < rank) {
            if (shape[d] < 0) return fail(TENMO_ERR_INVALID_SHAPE, "negative batch dim");
            n *= shape[d];
        }
    }
    *count = n;
    return 0;
}

// ------------------------------------------------------------------------------------------------
// GEMM dispatch
// ------------------------------------------------------------------------------------------------

int operand_mode(int64_t row_stride, int64_t k_stride, int64_t rows, int64_t K) {
    if (k_stride == 1) return KMAJOR_VEC;
    if (row_stride == 1) return MNMAJOR_VEC;
    if (K == 1) return KMAJOR_VEC;     // the k stride is never used
    if (rows == 1) return MNMAJOR_VEC; // the row stride is never used
    return KMAJOR_GEN;
}

struct TileShape { int bm, bn; };
constexpr int kNumTiles = 5;
const TileShape kTiles[kNumTiles] = {{256, 128}, {128, 128}, {64, 64}, {128, 64}, {64, 128}};

const double kOccupancy[kNumTiles] = {2, 3, 6, 4, 4}; // resident workgroups per CU of each tile's kernel (LDS / VGPR limits)
const int kStreamKOccupancy[kNumTiles] = {2, 2, 4, 4, 0}; // the same for the stream-K kernels (more registers; none for 64x128)

// what the GEMM store does besides writing the sums (all optional)
struct Epilogue {
    const float* bias = nullptr; // + bias[col]
    const float* mask = nullptr; // dense like C: zero the result where mask <= 0
    int relu = 0;                // max(., 0) after the bias
    int bias_rows = 0;           // bias[row] instead of bias[col]
    const int32_t* gather_row = nullptr; // B gathered through offset tables (implicit im2col), see GemmArgs
    const int32_t* gather_k = nullptr;
    bool gather_kmajor = false;          // the gathered B is contiguous along k (16-byte loads along k) rather than along n
    float* colsum = nullptr;             // [batch][N]: also write the column sums of the result (needs M <= 128, see GemmArgs)
    float* bsum = nullptr;               // [N]: += the column sums of B over K (GemmArgs::bsum; see bsum_fits); goes with accumulate
    bool any() const { return bias || mask || relu || colsum; }
};

// Stream-K launch of `tiles` tiles of `nks` K steps on `wgs` persistent workgroups: `whole_rounds` rounds of
// whole tiles (one per workgroup and round), then `shared` tiles whose K steps are spread evenly.  The shared
// part gives every workgroup at least eight K steps where the tile count allows: a shorter piece is all
// prologue and epilogue, so one round of whole tiles goes into the shared part instead.
void streamk_partition(int64_t tiles, int64_t nks, int64_t wgs, int64_t* whole_rounds, int64_t* shared) {
    int64_t full = tiles / wgs, rest = tiles - full * wgs;
    if (rest > 0 && rest * nks < 8 * wgs && full > 0) { --full; rest += wgs; }
    *whole_rounds = full;
    *shared = rest;
}

// What a launch with Epilogue::bsum needs: one matrix, the operand forms of a Linear layer's weight gradient X^T(view) . dY
// (the only instantiations that add up their B fragments), nothing else fused.
bool bsum_fits(int64_t a_rs, int64_t a_cs, int64_t b_rs, int64_t b_cs, int64_t M, int64_t N, int64_t K, int64_t batch_count, const Epilogue& ep) {
    return batch_count == 1 && M > 0 && N > 0 && K > 0 && !ep.any() && !ep.gather_row &&
           operand_mode(a_rs, a_cs, M, K) == MNMAJOR_VEC && operand_mode(b_cs, b_rs, N, K) == MNMAJOR_VEC;
}

int gemm_dispatch(const float* A, int64_t a_rs, int64_t a_cs, const float* B, int64_t b_rs, int64_t b_cs, float* C,
                  int64_t M, int64_t N, int64_t K, const BatchDesc& bd, int64_t batch_count, int accumulate, const Epilogue& ep = Epilogue()) {
    if (M == 0 || N == 0 || batch_count == 0) return 0;
    if (ep.any() && accumulate) return fail(TENMO_ERR_INVALID_ARGUMENT, "a fused epilogue cannot be combined with accumulate");
    if (K == 0) { // empty reduction: the reference's zero-initialised result
        if (ep.any()) return fail(TENMO_ERR_UNSUPPORTED, "fused epilogue with K = 0");
        if (!accumulate) {
            const int64_t n = batch_count * M * N;
            hipLaunchKernelGGL(fill_kernel, dim3((unsigned)std::min<int64_t>((n + 255) / 256, 65535)), dim3(256), 0, S.stream, C, n, 0.f);
        }
        return 0;
    }
    GemmArgs g{};
    g.A = A; g.B = B; g.C = C;
    g.a_rs = a_rs; g.a_cs = a_cs; g.b_rs = b_rs; g.b_cs = b_cs;
    g.M = M; g.N = N; g.K = K;
    g.accumulate = accumulate;
    g.bias = ep.bias; g.mask = ep.mask; g.relu = ep.relu; g.bias_rows = ep.bias_rows;
    g.b_gather_row = ep.gather_row; g.b_gather_k = ep.gather_k;
    g.colsum = ep.colsum;
    BsumArgs bsum_args{};
    bsum_args.out = ep.bsum;
    const BsumArgs* const bsum = ep.bsum ? &bsum_args : nullptr;
    if (ep.bsum && !bsum_fits(a_rs, a_cs, b_rs, b_cs, M, N, K, batch_count, ep))
        return fail(TENMO_ERR_UNSUPPORTED, "column sums of B beside the product: one matrix, both operands with unit stride along M / N, no other epilogue");
    if (ep.colsum && (M > 128 || accumulate)) return fail(TENMO_ERR_UNSUPPORTED, "column sums in the GEMM store need M <= 128 and no accumulate");
    g.batch = bd;
    g.batch_count = batch_count;
    const int am = operand_mode(a_rs, a_cs, M, K);
    const int bm = ep.gather_row ? (ep.gather_kmajor ? KMAJOR_VEC : MNMAJOR_VEC) : operand_mode(b_cs, b_rs, N, K);

    // Pick the workgroup tile and the number of K slices with a small cost model of this chip
    // (constants fitted to measured launches on MI355X): per CU the matrix-pipe time is the sum over
    // its workgroups (the K loop runs at full rate from one wavefront per SIMD up), every workgroup
    // pays a fixed prologue/epilogue, and the launch can never beat its HBM and L2 traffic.
    int tile = 0, splits = 1;
    int sk_tile = 0, sk_wpc = 0;
    double best_sk = 1e300;
    {
        const double* kOcc = kOccupancy;
        static const double kEff[kNumTiles] = {0.96, 0.93, 0.84, 0.90, 0.90}; // matrix-pipe efficiency of the K loop
        static const int kSplits[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32};
        const double cus = (double)S.cus;
        double best = 1e300;
        for (int t = 0; t < kNumTiles; ++t) {
            // a gathered operand is loaded through registers: measured on convolution layers (forward and both
            // gradients), the 128x64 tile wins there by 10-40 % over the larger ones, whose staging registers crowd the
            // accumulators, and 64x64 when there are at most 64 rows
            if (ep.gather_row && t != (M > 64 ? 3 : 2)) continue;
            if (ep.colsum && (t < 2 || kTiles[t].bm < M)) continue; // one tile must hold every row, and only the small tiles sum columns
            const double tm = (double)((M + kTiles[t].bm - 1) / kTiles[t].bm), tn = (double)((N + kTiles[t].bn - 1) / kTiles[t].bn);
            const double tiles = tm * tn * (double)batch_count;
            const double m_us = (kTiles[t].bm / 64) * (kTiles[t].bn / 64) * 8 * 64 / 2400.0; // MFMA time of one K step of one wavefront
            for (int sp : kSplits) {
                if (sp > 1 && (K / sp < 64 || (double)sp * batch_count * M * N * 4.0 > 1.0e9 || ep.bias_rows || ep.colsum)) break;
                const double wgs = tiles * sp, slots = cus * kOcc[t];
                // one round = every CU runs `conc` workgroups side by side.  After the full rounds the rest
                // runs with fewer workgroups per CU, each of them faster for it; the rounds do not end in
                // step, which costs a quarter of a round where a partial one follows full ones.
                const double iters = std::ceil((double)K / sp / GEMM_BK);
                // a gathered operand is loaded through a table lookup and registers, one K step ahead only: a workgroup
                // cannot finish a step in less than about 1.4 us however few share the CU (measured: 256 workgroups of
                // 128 steps 200 us), so a launch with few tiles is better cut into K slices
                const double step_floor = ep.gather_row ? 1.4 : 0.0;
                auto round_us = [&](double conc) { return iters * std::max(conc * m_us / kEff[t], step_floor) + 1.5; };
                const double full = std::floor(wgs / slots), rest = wgs - full * slots;
                double t_rounds = full * round_us(kOcc[t]);
                if (rest > 0) t_rounds += round_us(std::ceil(rest / cus)) + (full > 0 ? 0.25 * round_us(kOcc[t]) : 0.0);
                const double bytes = 4.0 * batch_count * ((double)M * K + (double)K * N + (double)M * N * (sp > 1 ? sp + 1.0 : 1.0));
                const double l2_bytes = 4.0 * batch_count * (double)K * ((double)M * tn + (double)N * tm);
                double est = std::max({t_rounds, bytes / 5.0e6, l2_bytes / 8.0e6}) + 3.0;
                if (sp > 1) est += 5.0 + 4.0 * batch_count * (double)M * N * (sp + 1.0) / 6.0e6;
                if (est < best) { best = est; tile = t; splits = sp; }
            }
        }
        // stream-K (persistent workgroups: rounds of whole tiles, then the K steps of the remaining tiles
        // spread evenly, see gemm_mfma.hpp): no partial last round, at the price of the fix-up traffic
        if (S.force_streamk < 0 && am != KMAJOR_GEN && bm != KMAJOR_GEN && !ep.colsum) {
            // Measured: 128x128 wins, with one workgroup per CU while there are at most two tiles per CU and with two
            // beyond (three do not fit its registers); 256x128 with two per CU comes within 1-2 % at large sizes.
            // A gathered operand keeps its tile (see above) at that tile's resident workgroups per CU.
            const int gather_tile = M > 64 ? 3 : 2;
            for (int t = ep.gather_row ? gather_tile : 1; t >= 0; --t) {
                if (ep.bsum && t != 1) continue; // (the column sums of B beside the product: the 128x128 stream-K kernel has the registers for them)
                const int64_t tiles = ((M + kTiles[t].bm - 1) / kTiles[t].bm) * ((N + kTiles[t].bn - 1) / kTiles[t].bn) * batch_count;
                const int wpc = ep.gather_row ? kStreamKOccupancy[t] : (t == 0 || tiles >= 2 * (int64_t)S.cus) ? 2 : 1;
                const int64_t nks = (K + GEMM_BK - 1) / GEMM_BK, wgs = (int64_t)S.cus * wpc;
                int64_t whole_rounds, shared;
                streamk_partition(tiles, nks, wgs, &whole_rounds, &shared);
                const bool last = ep.gather_row != nullptr; // one candidate only
                if (shared == 0 || shared * nks < wgs * 8) { if (last) break; continue; } // nothing to share / pieces of under eight K steps are all overhead
                // with fewer tiles than workgroups only 128x128 at one workgroup per CU wins; with rounds of whole tiles and a
                // short K the shared part must be small (measured at K = 768: -10 % with a third of the tiles shared, +5 %
                // with 2 %; from K = 2560 up +5 to +18 % whatever the share)
                if (!ep.gather_row && (whole_rounds == 0 ? (t != 1 || wpc != 1) : (nks < 64 && shared * 10 > tiles))) continue;
                // gathered: measured on convolution layers, 128x64 gains 5-8 % from K = 1024 up while the tiles make at most
                // two rounds, and loses 9 % at three (its stream-K kernel spills a few registers) and with a short K; 64x64 loses
                if (ep.gather_row && (t != 3 || nks < 64 || whole_rounds > 1)) break;
                // 16-byte loads from rows that are not 16-byte aligned are slow enough to be the bound, and one workgroup
                // per CU hides them badly (measured [2048,50257].[50257,768]: 118 against 126 TFLOP/s with K slices)
                const int64_t a_pitch = am == KMAJOR_VEC ? a_rs : a_cs, b_pitch = bm == KMAJOR_VEC ? b_cs : b_rs;
                if (wpc == 1 && ((M > 1 && K > 1 && a_pitch % 4 != 0) || (N > 1 && K > 1 && b_pitch % 4 != 0))) continue;
                const double m_us = (kTiles[t].bm / 64) * (kTiles[t].bn / 64) * 8 * 64 / 2400.0;
                // one K step of every workgroup of a CU.  The 256x128 stream-K kernel spills a few registers: up to about a
                // thousand of its tiles the 128x128 one at two per CU is 2-4 % ahead (3072^3 .. 5120^3), beyond that 256x128
                // is level or ahead (6144^3 .. 10240^3: the smaller tile's operand traffic starts to count)
                const double step_us = wpc * m_us / (t == 0 && tiles <= 1024 ? kEff[1] : kEff[t]);
                const double pieces = (double)std::min(2 * wgs, 2 * shared);
                const double fix = 2.0 * pieces * kTiles[t].bm * kTiles[t].bn * 4.0 / 5.0e6;
                const double est = whole_rounds * (nks * step_us + 1.5) + (double)shared * nks / wgs * step_us + fix + 10.0;
                if (est < 0.98 * best && est < best_sk) { best_sk = est; sk_tile = t; sk_wpc = wpc; }
                if (last) break;
            }
        }
        // A product with K <= 128 and a large result is bound by its stores, which the model does not rank: all tiles
        // sit on the same byte floor.  Measured there (K = 32 .. 128, results of 64 MB and more, one matrix and batches),
        // the small tiles win — more workgroups per CU overlap one's stores with another's loads: 64x64 for a K-major B
        // (8192x8192x64: 112 us against 135 with 256x128; attention Q.K^T 179 against 202), 64x128 for an MN-major B
        // (110 against 116).
        if (K <= 128 && splits == 1 && sk_wpc == 0 && !ep.gather_row && !ep.colsum && am != KMAJOR_GEN && bm != KMAJOR_GEN &&
            ((M + 63) / 64) * ((N + 63) / 64) * batch_count >= 2048)
            tile = bm == KMAJOR_VEC ? 2 : 4;
        // A short reduction (K <= 512) into a large result whose 256x128 or 128x128 tiles do not even fill one round: the
        // model underrates what the few large workgroups lose to their prologue and to storing 64-128 KB each with
        // nothing beside them.  Measured ([256,192..512].[.,50000], [512,256].[256,16384], [1024,256].[256,8192], both
        // layouts of B): 128x64 is 11-16 % faster there and within 3 % of the best tile.
        else if (K <= 512 && tile <= 1 && splits == 1 && sk_wpc == 0 && !ep.gather_row && !ep.colsum && am != KMAJOR_GEN && bm != KMAJOR_GEN &&
                 (double)batch_count * M * N * 4.0 >= 16.0e6 &&
                 ((M + kTiles[tile].bm - 1) / kTiles[tile].bm) * ((N + kTiles[tile].bn - 1) / kTiles[tile].bn) * batch_count < (int64_t)(S.cus * kOccupancy[tile]))
            tile = 3;
        if (S.verbose) fprintf(stderr, "tenmo_hip gemm M=%lld N=%lld K=%lld batch=%lld -> tile %dx%d, %d K slice(s), est %.1f us%s\n",
                               (long long)M, (long long)N, (long long)K, (long long)batch_count, kTiles[tile].bm, kTiles[tile].bn, splits, best,
                               sk_wpc ? " (stream-K chosen instead)" : "");
    }
    // A few tile rows against a very wide B (gemm_resident.hip): the tile row of A stays in LDS, B alone is streamed.
    // Only on request (gemm_resident knob: 1 tiles of 128x64, 2 of 64x64) until it has been measured.
    if (S.force_resident > 0) {
        const int rbm = S.force_resident == 2 ? 64 : 128;
        const int64_t tm = (M + rbm - 1) / rbm, tn = (N + 63) / 64;
        const bool a_ok = am == KMAJOR_VEC ? (a_cs == 1 && a_rs >= 0 && a_rs <= (int64_t(1) << 21) && K % 4 == 0)
                                           : (am == MNMAJOR_VEC && a_rs == 1 && a_cs >= 0 && a_cs <= (int64_t(1) << 25) && M % 4 == 0 && M >= 4);
        const bool b_ok = bm == MNMAJOR_VEC && b_cs == 1 && b_rs >= 0 && b_rs <= (int64_t(1) << 25) && N % 4 == 0 && N >= 4;
        const bool can = batch_count == 1 && !accumulate && K > GEMM_BK && K <= 256 && a_ok && b_ok && !ep.any() && !ep.gather_row && !ep.colsum && !ep.bsum &&
                         N <= (int64_t(1) << 22) && tm <= (int64_t)S.cus * (rbm == 64 ? 2 : 1) / 8; // (worth it with several column blocks per workgroup: for the policy that will choose it once it has been measured)
        if (can) {
            g.tiles_m = (int32_t)tm; g.tiles_n = (int32_t)tn;
            g.k_splits = 1; g.k_per_split = K; g.partial = nullptr;
            if (S.verbose) fprintf(stderr, "tenmo_hip gemm: resident-A kernel, %lld x %lld tiles of %dx64\n", (long long)tm, (long long)tn, rbm);
            if (launch_gemm_resident(g, rbm, am, bm, (unsigned)S.cus, S.stream)) return 0;
        }
    }
    // The persistent K-stream kernel (gemm_panel.hip): vector operand forms, plain or accumulating store.  Automatic for
    // a reduction of 65 .. 512 into a result of at least three 128x128 tiles per CU (measured against the tile the model
    // picks: 96 x [1024,128].[128,1024] 293 -> 229 us, [4096,256].[256,4096] 75 -> 70 us, [4096,512].[512,4096] 129 -> 127 us,
    // the CBOW logits [256,100].[100,50000] 42 -> 39 us; level at K = 1024, and 8-25 % slower with fewer tiles than that,
    // where its two workgroups per CU are not filled).  Reductions of one K step (K <= 16) never take it: see below.
    {
        auto operand_ok = [&](int mode, int64_t row_s, int64_t k_s, int64_t extent) {
            if (mode == KMAJOR_VEC) return k_s == 1 && row_s >= 0 && row_s <= (int64_t(1) << 21) && (K % GEMM_BK == 0 || K % 4 == 0);
            if (mode == MNMAJOR_VEC) return row_s == 1 && k_s >= 0 && k_s <= (int64_t(1) << 25) && extent % 4 == 0 && extent >= 4;
            return false;
        };
        // (3: its 64x64-tile variant, a ring of eight stages, forced: for long reductions over few tiles)
        const int pt = S.force_panel == 3 ? 64 : 128;
        const int64_t tm = (M + pt - 1) / pt, tn = (N + pt - 1) / pt, tiles = tm * tn * batch_count;
        const bool can = K > GEMM_BK && operand_ok(am, a_rs, a_cs, M) && operand_ok(bm, b_cs, b_rs, N) && !ep.any() && !ep.gather_row && !ep.colsum && !ep.bsum &&
                         N <= (int64_t(1) << 22) && tiles <= 0x7fffffffLL;
        const bool want = S.force_panel > 0 || (S.force_panel < 0 && S.force_tile < 0 && S.force_splitk <= 0 && S.force_streamk <= 0 && S.force_smallk <= 0 &&
                                                 splits == 1 && sk_wpc == 0 && K > 64 && K <= 512 && tiles >= 3 * (int64_t)S.cus);
        if (can && want) {
            g.tiles_m = (int32_t)tm; g.tiles_n = (int32_t)tn;
            g.k_splits = 1; g.k_per_split = K; g.partial = nullptr;
            if (S.verbose) fprintf(stderr, "tenmo_hip gemm: K-stream kernel, %lld tiles of %dx%d\n", (long long)tiles, pt, pt);
            const int which = pt == 64 ? PANEL_TILE_64x64 : PANEL_TILE_128x128;
            if (launch_gemm_panel(g, which, am, bm, (unsigned)S.cus, (unsigned)tiles, S.force_panel != 2, S.stream)) return 0;
        }
    }
    // Short reduction, vector operand forms and a plain (or accumulating) store: the persistent whole-K-in-LDS kernel
    // (gemm_smallk.hip).  Automatic for K <= 64 where the launch is store-bound as above and every workgroup gets several
    // tiles (measured: 8192x8192xK, K = 32 / 64, every operand layout 76-115 -> 60-93 us; [256,64].[64,50000] 27 -> 21 us;
    // K = 96 .. 112, one workgroup per CU, measured level with the ordinary kernel: not built).
    {
        const int64_t tm = (M + 63) / 64, tn = (N + 63) / 64, tiles64 = tm * tn * batch_count;
        // what the direct loads need: a K-major operand a row pitch below 2^21 and, when K is no multiple of 16, K % 4 == 0
        // (it moves 4 consecutive k at a time); an MN-major one a k pitch below 2^25 and an extent divisible by 4
        auto operand_ok = [&](int mode, int64_t row_s, int64_t k_s, int64_t extent) {
            if (mode == KMAJOR_VEC) return k_s == 1 && row_s >= 0 && row_s <= (int64_t(1) << 21) && (K % GEMM_BK == 0 || K % 4 == 0);
            if (mode == MNMAJOR_VEC) return row_s == 1 && k_s >= 0 && k_s <= (int64_t(1) << 25) && extent % 4 == 0 && extent >= 4;
            return false;
        };
        // (Reductions of a single K step, K <= 16, stay with the ordinary kernel for now: a timing run of [8192,16].[16,8192]
        // through this kernel faulted — an undeclared SCC clobber of the masked direct load, since fixed (gfx950_asm.hpp) — and
        // the one-step instantiations come back once the fix has been confirmed on a GPU.  Until then the automatic choice
        // is also limited to K % 16 == 0, which never takes the masked load; a ragged K reaches it only through the knob.)
        // (gemm_smallk = 3 forces the kernel onto one-step reductions too: for the checks of exactly that path)
        const bool can = (K > GEMM_BK || S.force_smallk == 3) && K <= 64 && operand_ok(am, a_rs, a_cs, M) && operand_ok(bm, b_cs, b_rs, N) && !ep.any() && !ep.gather_row && !ep.colsum && !ep.bsum &&
                         N < (int64_t(1) << 29) && tiles64 <= 0x7fffffffLL;
        const bool want = S.force_smallk > 0 || (S.force_smallk < 0 && S.force_tile < 0 && S.force_splitk <= 0 && S.force_streamk <= 0 &&
                                                  splits == 1 && sk_wpc == 0 && tiles64 >= 2048 && K <= 64 && K % GEMM_BK == 0);
        if (can && want) {
            g.tiles_m = (int32_t)tm; g.tiles_n = (int32_t)tn;
            g.k_splits = 1; g.k_per_split = K; g.partial = nullptr;
            if (S.verbose) fprintf(stderr, "tenmo_hip gemm: short-reduction kernel, %lld tiles of 64x64\n", (long long)tiles64);
            if (launch_gemm_smallk_64x64(g, am, bm, (unsigned)S.cus, (unsigned)tiles64, S.force_smallk != 2, S.stream)) return 0;
        }
    }
    if (S.force_tile >= 0 && S.force_tile < kNumTiles && !(ep.colsum && (S.force_tile < 2 || kTiles[S.force_tile].bm < M))) tile = S.force_tile;
    if (S.force_splitk > 0 && !ep.bias_rows && !ep.colsum) splits = S.force_splitk; // the slice reduction applies the bias by column only
    int streamk = S.force_streamk > 0 && !ep.colsum ? S.force_streamk : 0;
    if (S.force_streamk < 0 && sk_wpc > 0 && S.force_tile < 0 && S.force_splitk <= 0) { streamk = sk_wpc; tile = sk_tile; }
    if (streamk > 0 && ep.bsum) tile = 1; // the one stream-K kernel that also adds up the column sums of B
    if (streamk > 0 && tile <= 3 && am != KMAJOR_GEN && bm != KMAJOR_GEN && (!ep.gather_row || tile >= 2)) {
        const int bmt = kTiles[tile].bm, bnt = kTiles[tile].bn;
        g.tiles_m = (int32_t)((M + bmt - 1) / bmt);
        g.tiles_n = (int32_t)((N + bnt - 1) / bnt);
        g.k_splits = 1; g.k_per_split = K; g.partial = nullptr;
        const int64_t tiles_total = (int64_t)g.tiles_m * g.tiles_n * batch_count;
        StreamKArgs sk{};
        sk.nks = (K + GEMM_BK - 1) / GEMM_BK;
        const int64_t want = (int64_t)S.cus * std::min(streamk, kStreamKOccupancy[tile]); // every workgroup of the grid must be resident
        int64_t whole_rounds, shared;
        streamk_partition(tiles_total, sk.nks, want, &whole_rounds, &shared);
        sk.dp_tiles = whole_rounds * want;
        sk.total = shared * sk.nks;
        int64_t per = std::max<int64_t>((sk.total + want - 1) / want, 1);
        per = (per + 3) / 4 * 4; // no piece shorter than four K steps except at the end of K
        sk.per_wg = per;
        // every workgroup of the grid takes whole tiles; with none of those, only the workgroups that get a run
        const int64_t wgs = whole_rounds > 0 ? want : (sk.total + per - 1) / per;
        if (tiles_total <= 0x7fffffffLL && wgs >= 1) {
            float* ws;
            if (int rc = workspace((size_t)(2 * wgs) * (bmt + (ep.bsum ? 1 : 0)) * bnt * sizeof(float), &ws)) return rc;
            sk.partial = ws;
            bsum_args.partial = ep.bsum ? ws + (size_t)(2 * wgs) * bmt * bnt : nullptr;
            const bool need_fixup = shared > 0 && per % sk.nks != 0;
            if (S.verbose) fprintf(stderr, "tenmo_hip gemm stream-K: %lld workgroups, %lld whole tiles each, then %lld K steps each of %lld shared tiles of %dx%d\n",
                                   (long long)wgs, (long long)whole_rounds, (long long)per, (long long)shared, bmt, bnt);
            // parts per shared tile in the fix-up: a power of two that brings it to a few workgroups per CU
            unsigned parts = 0;
            if (need_fixup) for (parts = 1; parts < 32 && shared * parts < (int64_t)S.cus * 4; parts *= 2) {}
            const bool ok = tile == 0   ? launch_streamk_256x128(g, sk, (unsigned)wgs, (unsigned)shared, parts, am, bm, S.stream, bsum)
                            : tile == 1 ? launch_streamk_128x128(g, sk, (unsigned)wgs, (unsigned)shared, parts, am, bm, S.stream, bsum)
                            : tile == 2 ? launch_streamk_64x64(g, sk, (unsigned)wgs, (unsigned)shared, parts, am, bm, S.stream, bsum)
                                        : launch_streamk_128x64(g, sk, (unsigned)wgs, (unsigned)shared, parts, am, bm, S.stream, bsum);
            return ok ? 0 : fail(TENMO_ERR_UNSUPPORTED, "no stream-K variant for operand modes %d/%d", am, bm);
        }
    }
    const int64_t nb = ((M + kTiles[tile].bm - 1) / kTiles[tile].bm) * ((N + kTiles[tile].bn - 1) / kTiles[tile].bn) * batch_count;
    g.k_splits = splits;
    g.k_per_split = K;
    if (splits > 1) {
        int64_t per = (K + splits - 1) / splits;
        per = (per + GEMM_BK - 1) / GEMM_BK * GEMM_BK;
        g.k_per_split = per;
        splits = (int)((K + per - 1) / per);
        g.k_splits = splits;
    }
    if (splits > 1) {
        float* ws;
        if (int rc = workspace((size_t)splits * (batch_count * M + (ep.bsum ? 1 : 0)) * N * sizeof(float), &ws)) return rc;
        g.partial = ws;
        bsum_args.partial = ep.bsum ? ws + (size_t)splits * batch_count * M * N : nullptr;
    }
    g.tiles_m = (int32_t)((M + kTiles[tile].bm - 1) / kTiles[tile].bm);
    g.tiles_n = (int32_t)((N + kTiles[tile].bn - 1) / kTiles[tile].bn);
    if (nb > 0x7fffffffLL) return fail(TENMO_ERR_UNSUPPORTED, "grid too large");
    dim3 grid((unsigned)nb, (unsigned)splits, 1);
    bool ok = false;
    switch (tile) {
        case 0: ok = launch_gemm_256x128(g, grid, am, bm, S.stream, bsum); break;
        case 1: ok = launch_gemm_128x128(g, grid, am, bm, S.stream, bsum); break;
        case 3: ok = launch_gemm_128x64(g, grid, am, bm, S.stream, bsum); break;
        case 4: ok = launch_gemm_64x128(g, grid, am, bm, S.stream, bsum); break;
        default: ok = launch_gemm_64x64(g, grid, am, bm, S.stream, bsum); break;
    }
    if (!ok) return fail(TENMO_ERR_UNSUPPORTED, "no GEMM variant for operand modes %d/%d", am, bm);
    if (splits > 1) {
        const int64_t n = batch_count * M * N;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)std::min<int64_t>((n + 255) / 256, 8192)), dim3(256), 0, S.stream,
                           g.partial, C, n, splits, accumulate, ep.bias, ep.mask, ep.relu, N, (const float*)bsum_args.partial, ep.bsum, ep.bsum ? N : (int64_t)0);
    }
    return 0;
}

// ------------------------------------------------------------------------------------------------
// mv / vm dispatch.  Both reduce to two streaming kernels chosen by which matrix dim has unit stride:
//   rows kernel : unit stride along the reduction  -> one wavefront per few outputs
//   cols kernel : unit stride along the outputs    -> one lane per four outputs, k split over blocks
// ------------------------------------------------------------------------------------------------

// every row of every batch of the streamed matrix starts on a 16-byte boundary
bool cols_aligned(const ColsArgs& c) {
    if ((uintptr_t)c.Mx % 16 != 0 || c.m_rs % 4 != 0) return false;
    for (int d = 0; d < c.batch.rank; ++d) if (c.batch.b_str[d] % 4 != 0) return false;
    return true;
}

// the first row of every batch is 16-byte aligned but the row pitch is not a multiple of 4 floats:
// cols_shift_kernel keeps every load aligned (up to 4 left-operand rows)
bool cols_shiftable(const ColsArgs& c) {
    if ((uintptr_t)c.Mx % 16 != 0 || c.m_rs % 4 == 0 || c.m_rs < c.n || c.n < 4 || c.rows > 4) return false;
    for (int d = 0; d < c.batch.rank; ++d) if (c.batch.b_str[d] % 4 != 0) return false;
    return true;
}

template <int R>
void launch_cols(const ColsArgs& c, dim3 grid, int variant, bool join) {
    if (join) { // the K slices are added by the last workgroup of each column block
        if (variant == 0) hipLaunchKernelGGL((cols_kernel<R, true, true>), grid, dim3(COLS_THREADS), 0, S.stream, c);
        else if (variant == 2) hipLaunchKernelGGL((cols_kernel<R, false, true>), grid, dim3(COLS_THREADS), 0, S.stream, c);
        else if constexpr (R <= 4) hipLaunchKernelGGL((cols_shift_kernel<R, true>), grid, dim3(COLS_THREADS), 0, S.stream, c);
        return;
    }
    if (variant == 0) hipLaunchKernelGGL((cols_kernel<R, true>), grid, dim3(COLS_THREADS), 0, S.stream, c);
    else if (variant == 2) hipLaunchKernelGGL((cols_kernel<R, false>), grid, dim3(COLS_THREADS), 0, S.stream, c);
    else if constexpr (R <= 4) hipLaunchKernelGGL((cols_shift_kernel<R>), grid, dim3(COLS_THREADS), 0, S.stream, c);
}

// largest batch count of one launch (a grid's y and z dimensions hold 65535)
constexpr int64_t kMaxGridBatches = 65535;
// arrival counters of the in-launch K-slice reduction (one per column block and batch of a launch)
constexpr int64_t kArrivalCounters = 1 << 16;

// Scratch for the K-slice partial sums of a column-streaming product: the library's grow-only buffer, or a
// fixed buffer the caller brings (the allocation-free entry point), which is never grown.
struct ScratchSource {
    float* fixed = nullptr;
    size_t fixed_bytes = 0;
};

// Runs the column-streaming product described by `c` (c.out is set here): picks the kernel variant,
// cuts K into slices when the column blocks alone would not fill the chip, and adds the slices.
int cols_run(ColsArgs c, int64_t batch_count, float* out, int accumulate, const ScratchSource& scratch_src = ScratchSource()) {
    const int variant = cols_aligned(c) ? 0 : cols_shiftable(c) ? 1 : 2; // 16-byte loads / shifted sets / dword loads
    const int64_t width = variant == 1 ? COLS_SHIFT_WIDTH : COLS_THREADS * 4;
    const int64_t col_blocks = (c.n + width - 1) / width;
    const int64_t K = c.k, R = c.rows;
    int64_t splits = 1;
    const int64_t want = (int64_t)S.cus * S.cols_waves_per_cu;
    if (col_blocks * batch_count < want) splits = std::min<int64_t>((want + col_blocks * batch_count - 1) / (col_blocks * batch_count), (K + COLS_KSLICE_MIN - 1) / COLS_KSLICE_MIN);
    splits = std::max<int64_t>(1, std::min<int64_t>(splits, 65535));
    int64_t per = (K + splits - 1) / splits;
    per = (per + COLS_KSLICE_MIN - 1) / COLS_KSLICE_MIN * COLS_KSLICE_MIN;
    splits = (K + per - 1) / per;
    c.k_splits = (int32_t)splits; c.k_per_split = per;
    c.accumulate = accumulate;
    c.batch_total = batch_count;
    float* target = out;
    if (splits > 1) {
        const size_t bytes = (size_t)splits * batch_count * R * c.n * sizeof(float);
        float* ws;
        if (scratch_src.fixed) {
            if (bytes > scratch_src.fixed_bytes)
                return fail(TENMO_ERR_UNSUPPORTED, "the partial sums of %lld K slices x %lld batches x %lld rows x %lld columns need %zu bytes of scratch; "
                            "the static buffer of the allocation-free entry point holds %zu", (long long)splits, (long long)batch_count, (long long)R,
                            (long long)c.n, bytes, scratch_src.fixed_bytes);
            ws = scratch_src.fixed;
        } else if (int rc = workspace(bytes, &ws)) return rc;
        target = ws;
    }
    c.out = target;
    // One launch instead of two: the last workgroup of a column block adds the block's K slices (cols_join knob).  The
    // arrival counters are the library's, zero between launches; products with more column blocks x batches than there
    // are counters keep the separate reduction.
    const bool join = splits > 1 && S.cols_join > 0 && S.arrivals && col_blocks * std::min(kMaxGridBatches, batch_count) <= kArrivalCounters;
    c.joined = out;
    c.arrivals = S.arrivals;
    for (int64_t b0 = 0; b0 < batch_count; b0 += kMaxGridBatches) {
        c.batch0 = b0;
        const dim3 grid((unsigned)col_blocks, (unsigned)splits, (unsigned)std::min(kMaxGridBatches, batch_count - b0));
        if (R <= 1) launch_cols<1>(c, grid, variant, join);
        else if (R <= 2) launch_cols<2>(c, grid, variant, join);
        else if (R <= 4) launch_cols<4>(c, grid, variant, join);
        else launch_cols<8>(c, grid, variant, join);
    }
    if (splits > 1 && !join) {
        const int64_t n = batch_count * R * c.n;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)std::min<int64_t>((n + 255) / 256, 8192)), dim3(256), 0, S.stream,
                           target, out, n, (int)splits, accumulate, (const float*)nullptr, (const float*)nullptr, 0, (int64_t)1);
    }
    return 0;
}

template <int WPR, int RPW, int UNROLL>
void launch_rows(GemvArgs g, int64_t batch_count) {
    const int64_t units = (g.rows + RPW - 1) / RPW;
    for (int64_t b0 = 0; b0 < batch_count; b0 += kMaxGridBatches) {
        g.batch0 = b0;
        const dim3 grid((unsigned)(WPR == 1 ? (units + MV_WAVES - 1) / MV_WAVES : units), (unsigned)std::min(kMaxGridBatches, batch_count - b0));
        if (g.v_s == 1) hipLaunchKernelGGL((mv_rows_kernel<WPR, RPW, UNROLL, true>), grid, dim3(64 * MV_WAVES), 0, S.stream, g);
        else hipLaunchKernelGGL((mv_rows_kernel<WPR, RPW, UNROLL, false>), grid, dim3(64 * MV_WAVES), 0, S.stream, g);
    }
}

// one thread per output, any strides; grid.x blocks of 256 outputs per batch
void launch_generic(GemvArgs g, int64_t batch_count) {
    for (int64_t b0 = 0; b0 < batch_count; b0 += kMaxGridBatches) {
        g.batch0 = b0;
        hipLaunchKernelGGL(mv_generic_kernel, dim3((unsigned)((g.rows + 255) / 256), (unsigned)std::min(kMaxGridBatches, batch_count - b0)), dim3(256), 0, S.stream, g);
    }
}

// out[b][i] = sum_j Mat[b](i, j) * vec[b](j), i < n_out, j < n_red;  Mat(i,j) = Mx[i*out_s + j*red_s]
int matvec_dispatch(const float* Mx, int64_t out_s, int64_t red_s, const float* vec, int64_t v_s, float* out,
                    int64_t n_out, int64_t n_red, const BatchDesc& bd_mat_vec, int64_t batch_count, int accumulate,
                    const ScratchSource& scratch_src = ScratchSource()) {
    if (n_out == 0 || batch_count == 0) return 0;
    if (batch_count > 0x7fffffffLL) return fail(TENMO_ERR_UNSUPPORTED, "more than 2^31 batches in mv/vm");
    if (n_red == 0) {
        if (!accumulate) {
            const int64_t n = batch_count * n_out;
            hipLaunchKernelGGL(fill_kernel, dim3((unsigned)std::min<int64_t>((n + 255) / 256, 65535)), dim3(256), 0, S.stream, out, n, 0.f);
        }
        return 0;
    }
    if (red_s == 1 || n_red == 1) {
        GemvArgs g{};
        g.Mx = Mx; g.v = vec; g.out = out;
        g.m_rs = out_s; g.m_cs = 1; g.v_s = v_s; g.rows = n_out; g.k = n_red; g.accumulate = accumulate; g.batch = bd_mat_vec;
        if (n_red == 1 && red_s != 1) { // degenerate: a single product per output
            g.m_cs = red_s;
            launch_generic(g, batch_count);
            return 0;
        }
        // long rows: the whole workgroup walks 4 rows (bursts of 32 KiB per row); shorter rows get shorter
        // bursts and fewer rows per unit; rows under 2048 elements go one wavefront per unit
        if (n_red >= 8192) {
            if (n_out * batch_count >= 2 * (int64_t)S.cus) launch_rows<4, 4, 8>(g, batch_count);
            else launch_rows<4, 1, 8>(g, batch_count);
        } else if (n_red >= 2048) launch_rows<4, 2, 4>(g, batch_count);
        else if (n_red >= 1024) launch_rows<1, 1, 8>(g, batch_count);
        else launch_rows<1, 4, 4>(g, batch_count);
        return 0;
    }
    if (out_s == 1 || n_out == 1) {
        if (n_out == 1 && out_s != 1) {
            GemvArgs g{};
            g.Mx = Mx; g.v = vec; g.out = out;
            g.m_rs = out_s; g.m_cs = red_s; g.v_s = v_s; g.rows = n_out; g.k = n_red; g.accumulate = accumulate; g.batch = bd_mat_vec;
            launch_generic(g, batch_count);
            return 0;
        }
        ColsArgs c{};
        c.X = vec; c.Mx = Mx; c.out = out;
        c.x_rs = 0; c.x_ks = v_s; c.m_rs = red_s; c.k = n_red; c.n = n_out; c.rows = 1; c.accumulate = accumulate;
        // in ColsArgs the X operand uses a_str and the matrix b_str: swap relative to (matrix, vector)
        c.batch = bd_mat_vec;
        for (int d = 0; d < MAX_BATCH_RANK; ++d) std::swap(c.batch.a_str[d], c.batch.b_str[d]);
        if (int rc = cols_run(c, batch_count, out, accumulate, scratch_src)) return rc;
        return 0;
    }
    GemvArgs g{};
    g.Mx = Mx; g.v = vec; g.out = out;
    g.m_rs = out_s; g.m_cs = red_s; g.v_s = v_s; g.rows = n_out; g.k = n_red; g.accumulate = accumulate; g.batch = bd_mat_vec;
    launch_generic(g, batch_count);
    return 0;
}

// Two small products in ONE launch of the 64x64 tile (no batches, one K slice each); `ep1` belongs to the second.
// Returns 1 when the pair form does not apply (sizes, operand forms): the caller then launches them one by one.
int gemm_pair_dispatch(const float* A0, int64_t a0_rs, int64_t a0_cs, const float* B0, int64_t b0_rs, int64_t b0_cs, float* C0, int64_t M0, int64_t N0, int64_t K0,
                       const float* A1, int64_t a1_rs, int64_t a1_cs, const float* B1, int64_t b1_rs, int64_t b1_cs, float* C1, int64_t M1, int64_t N1, int64_t K1,
                       const Epilogue& ep1) {
    if (S.force_tile >= 0 || S.force_splitk > 0 || S.force_streamk > 0) return 1; // overrides apply to single launches
    if (M0 < 1 || N0 < 1 || K0 < 1 || M1 < 1 || N1 < 1 || K1 < 1 || ep1.gather_row || ep1.bias_rows) return 1;
    if (ep1.colsum && M1 > 64) return 1;
    auto fill = [](GemmArgs& g, const float* A, int64_t a_rs, int64_t a_cs, const float* B, int64_t b_rs, int64_t b_cs, float* C, int64_t M, int64_t N, int64_t K) {
        g.A = A; g.B = B; g.C = C;
        g.a_rs = a_rs; g.a_cs = a_cs; g.b_rs = b_rs; g.b_cs = b_cs;
        g.M = M; g.N = N; g.K = K;
        g.tiles_m = (int32_t)((M + 63) / 64); g.tiles_n = (int32_t)((N + 63) / 64);
        g.k_splits = 1; g.k_per_split = K; g.batch_count = 1;
        g.batch.rank = 0;
        for (int d = 0; d < MAX_BATCH_RANK; ++d) g.batch.shape[d] = 1;
    };
    GemmArgs g0{}, g1{};
    fill(g0, A0, a0_rs, a0_cs, B0, b0_rs, b0_cs, C0, M0, N0, K0);
    fill(g1, A1, a1_rs, a1_cs, B1, b1_rs, b1_cs, C1, M1, N1, K1);
    g1.bias = ep1.bias; g1.mask = ep1.mask; g1.relu = ep1.relu; g1.colsum = ep1.colsum;
    const int64_t c0 = (int64_t)g0.tiles_m * g0.tiles_n, c1 = (int64_t)g1.tiles_m * g1.tiles_n;
    // small products only: beyond a few workgroups per CU each product fills the chip by itself and wants its own tile choice
    if (c0 + c1 > (int64_t)S.cus * 2 || K0 > 4096 || K1 > 4096) return 1;
    const bool ok = launch_gemm_pair_64x64(g0, g1, (unsigned)c0, (unsigned)c1, operand_mode(a0_rs, a0_cs, M0, K0), operand_mode(b0_cs, b0_rs, N0, K0),
                                           operand_mode(a1_rs, a1_cs, M1, K1), operand_mode(b1_cs, b1_rs, N1, K1), S.stream);
    return ok ? 0 : 1;
}

// skinny GEMM: M <= 8 rows against a row-major B — the matrix is streamed once, like vm
int skinny_dispatch(const float* A, int64_t a_rs, int64_t a_cs, const float* B, int64_t b_rs, float* C,
                    int64_t M, int64_t N, int64_t K, const BatchDesc& bd, int64_t batch_count, int accumulate) {
    ColsArgs c{};
    c.X = A; c.Mx = B; c.x_rs = a_rs; c.x_ks = a_cs; c.m_rs = b_rs; c.k = K; c.n = N; c.rows = (int32_t)M; c.accumulate = accumulate;
    c.batch = bd;
    if (int rc = cols_run(c, batch_count, C, accumulate)) return rc;
    return 0;
}

// C (+)= A . B: a few rows against a wide row-major B is HBM-bound and streams B once through the column kernel;
// everything else goes to the matrix cores
int product_dispatch(const float* A, int64_t a_rs, int64_t a_cs, const float* B, int64_t b_rs, int64_t b_cs, float* C,
                     int64_t M, int64_t N, int64_t K, const BatchDesc& bd, int64_t batch_count, int accumulate, const Epilogue& ep = Epilogue()) {
    if (M >= 1 && M <= 8 && (b_cs == 1 || N == 1) && N >= 2048 && K > 0 && batch_count > 0 && !ep.any() && !ep.gather_row)
        return skinny_dispatch(A, a_rs, a_cs, B, b_rs, C, M, N, K, bd, batch_count, accumulate);
    return gemm_dispatch(A, a_rs, a_cs, B, b_rs, b_cs, C, M, N, K, bd, batch_count, accumulate, ep);
}

// ------------------------------------------------------------------------------------------------
// view helpers
// ------------------------------------------------------------------------------------------------

int check_view(const tenmo_view* v, const char* who, bool need_data) {
    if (!v) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: null view", who);
    if (v->rank < 0 || v->rank > TENMO_MAX_RANK) return fail(TENMO_ERR_INVALID_SHAPE, "%s: rank %d exceeds max_rank %d", who, v->rank, TENMO_MAX_RANK);
    for (int d = 0; d < v->rank; ++d)
        if (v->shape[d] < 0) return fail(TENMO_ERR_INVALID_SHAPE, "%s: negative dimension", who);
    if (need_data && !v->data && product(v->shape, v->rank) > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: view without data", who);
    return 0;
}

// a result / gradient pointer that will be written must not be null
int need(const void* p, bool written, const char* who, const char* what) {
    if (!p && written) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: null %s", who, what);
    return 0;
}

// right-aligned broadcast (tenmo/broadcasthelper.mojo:33-62)
bool broadcast_batch(const int64_t* sa, int ra, const int64_t* sb, int rb, int64_t* out, int* rout) {
    const int r = std::max(ra, rb);
    for (int d = 0; d < r; ++d) {
        const int ia = d - (r - ra), ib = d - (r - rb);
        const int64_t da = ia >= 0 ? sa[ia] : 1, db = ib >= 0 ? sb[ib] : 1;
        if (da == db) out[d] = da;
        else if (da == 1) out[d] = db;
        else if (db == 1) out[d] = da;
        else return false;
    }
    *rout = r;
    return true;
}

// strides an operand contributes to the result batch dims: 0 where its dim is 1 or missing
void batch_strides_of(const tenmo_view* v, int own_batch_rank, int result_batch_rank, int64_t* out) {
    for (int d = 0; d < result_batch_rank; ++d) {
        const int od = d - (result_batch_rank - own_batch_rank);
        out[d] = (od >= 0 && v->shape[od] > 1) ? v->strides[od] : 0;
    }
}

struct Geometry {
    int64_t oshape[TENMO_MAX_RANK + 2];
    int32_t orank;
    int batch_rank;
    int64_t batch_count;
};

// trailing dims: MM (2,2), MV (2,1), VM (1,2)
// need_data = false for pure shape queries, which never touch the operands
int resolve(int op, const tenmo_view* A, const tenmo_view* B, Geometry* g, const char* who, bool need_data = true) {
    if (int rc = check_view(A, who, need_data)) return rc;
    if (int rc = check_view(B, who, need_data)) return rc;
    const int ta = op == TENMO_OP_VM ? 1 : 2, tb = op == TENMO_OP_MV ? 1 : 2;
    if (op == TENMO_OP_MM) {
        if (A->rank < 2) return fail(TENMO_ERR_INVALID_SHAPE, "MatmulNdGpu: A must have rank >= 2");
        if (B->rank < 2) return fail(TENMO_ERR_INVALID_SHAPE, "MatmulNdGpu: B must have rank >= 2");
    } else if (op == TENMO_OP_MV) {
        if (A->rank < 2) return fail(TENMO_ERR_INVALID_SHAPE, "MatrixVectorMulNd: matrix must have at least 2 dimensions");
        if (B->rank < 1) return fail(TENMO_ERR_INVALID_SHAPE, "MatrixVectorMulNd: vector must have at least 1 dimension");
    } else if (op == TENMO_OP_VM) {
        if (A->rank < 1) return fail(TENMO_ERR_INVALID_SHAPE, "VectorMatmulNd: vector must have rank >= 1");
        if (B->rank < 2) return fail(TENMO_ERR_INVALID_SHAPE, "VectorMatmulNd: matrix must have rank >= 2");
    } else {
        return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: unknown op %d", who, op);
    }
    const int64_t ka = A->shape[A->rank - 1], kb = B->shape[B->rank - tb];
    if (ka != kb) {
        if (op == TENMO_OP_MM) return fail(TENMO_ERR_INVALID_SHAPE, "MatmulNdGpu: inner dims must match, got %lld and %lld", (long long)ka, (long long)kb);
        if (op == TENMO_OP_MV) return fail(TENMO_ERR_INVALID_SHAPE, "MatrixVectorMulNd: inner dimensions must match");
        return fail(TENMO_ERR_INVALID_SHAPE, "VectorMatmulNd: inner dimensions must match");
    }
    int br = 0;
    if (!broadcast_batch(A->shape, A->rank - ta, B->shape, B->rank - tb, g->oshape, &br))
        return fail(TENMO_ERR_INVALID_SHAPE, "ShapeBroadcaster -> broadcast_shape - cannot broadcast shapes: %s, %s",
                    shape_str(A->shape, A->rank - ta).c_str(), shape_str(B->shape, B->rank - tb).c_str());
    if (br > MAX_BATCH_RANK) return fail(TENMO_ERR_INVALID_SHAPE, "%s: result rank exceeds max_rank %d", who, TENMO_MAX_RANK);
    g->batch_rank = br;
    g->batch_count = product(g->oshape, br);
    if (op != TENMO_OP_VM) g->oshape[br++] = A->shape[A->rank - 2];
    if (op != TENMO_OP_MV) g->oshape[br++] = B->shape[B->rank - 1];
    g->orank = br;
    return 0;
}

BatchDesc make_batch(const Geometry& g, const tenmo_view* A, int ta, const tenmo_view* B, int tb) {
    BatchDesc bd{};
    bd.rank = g.batch_rank;
    int64_t as[MAX_BATCH_RANK] = {0}, bs[MAX_BATCH_RANK] = {0};
    batch_strides_of(A, A->rank - ta, g.batch_rank, as);
    batch_strides_of(B, B->rank - tb, g.batch_rank, bs);
    for (int d = 0; d < MAX_BATCH_RANK; ++d) {
        bd.shape[d] = d < g.batch_rank ? g.oshape[d] : 1;
        bd.a_str[d] = d < g.batch_rank ? as[d] : 0;
        bd.b_str[d] = d < g.batch_rank ? bs[d] : 0;
    }
    return bd;
}

tenmo_view transposed_last2(const tenmo_view* v) {
    tenmo_view t = *v;
    std::swap(t.shape[t.rank - 1], t.shape[t.rank - 2]);
    std::swap(t.strides[t.rank - 1], t.strides[t.rank - 2]);
    return t;
}

tenmo_view dense_view(const float* p, const int64_t* shape, int rank) {
    tenmo_view v{};
    v.data = p; v.offset = 0; v.rank = rank;
    int64_t acc = 1;
    for (int d = rank - 1; d >= 0; --d) { v.shape[d] = shape[d]; v.strides[d] = acc; acc *= shape[d]; }
    return v;
}

int matmul_views(const tenmo_view* A, const tenmo_view* B, float* C, int accumulate, const char* who, const Epilogue& ep = Epilogue()) {
    Geometry g;
    if (int rc = resolve(TENMO_OP_MM, A, B, &g, who)) return rc;
    int64_t batch_count = g.batch_count;
    if (batch_count == 0) return 0; // no output elements (the reference only widens the loop count, matmul_cpu.mojo:666-667)
    if (int rc = need(C, product(g.oshape, g.orank) > 0, who, "result pointer")) return rc;
    const BatchDesc bd = make_batch(g, A, 2, B, 2);
    const int64_t M = A->shape[A->rank - 2], K = A->shape[A->rank - 1], N = B->shape[B->rank - 1];
    const float* Ap = A->data + A->offset;
    const float* Bp = B->data + B->offset;
    const int64_t a_rs = A->strides[A->rank - 2], a_cs = A->strides[A->rank - 1];
    const int64_t b_rs = B->strides[B->rank - 2], b_cs = B->strides[B->rank - 1];
    return product_dispatch(Ap, a_rs, a_cs, Bp, b_rs, b_cs, C, M, N, K, bd, batch_count, accumulate, ep);
}

// dst (dense, parent's shape) += sum over the batch dims of `full` that the parent broadcast
int reduce_to_parent(const float* full, const Geometry& g, const tenmo_view* parent, int trailing, float* dst) {
    BroadcastReduceArgs r{};
    r.src = full; r.dst = dst;
    r.inner = 1;
    for (int d = g.batch_rank; d < g.orank; ++d) r.inner *= g.oshape[d];
    r.rank = g.batch_rank;
    const int own = parent->rank - trailing;
    int64_t acc = 1, kept_total = 1, red_total = 1;
    for (int d = g.batch_rank - 1; d >= 0; --d) {
        r.shape[d] = g.oshape[d];
        r.src_str[d] = acc;
        acc *= g.oshape[d];
        const int od = d - (g.batch_rank - own);
        r.kept[d] = (od >= 0 && parent->shape[od] > 1) ? 1 : 0;
        if (r.kept[d]) kept_total *= g.oshape[d]; else red_total *= g.oshape[d];
    }
    r.dst_batch = kept_total;
    r.reduced_total = red_total;
    const int64_t total = kept_total * r.inner;
    if (total == 0) return 0;
    if (r.inner % 4 == 0 && (uintptr_t)r.src % 16 == 0 && (uintptr_t)r.dst % 16 == 0)
        hipLaunchKernelGGL(broadcast_reduce_add_vec_kernel, dim3((unsigned)std::min<int64_t>((total / 4 + 255) / 256, 65535)), dim3(256), 0, S.stream, r);
    else
        hipLaunchKernelGGL(broadcast_reduce_add_kernel, dim3((unsigned)std::min<int64_t>((total + 255) / 256, 65535)), dim3(256), 0, S.stream, r);
    return 0;
}

// every batch dim of the parent has extent 1 (or the parent has none)
bool all_broadcast(const tenmo_view* parent, int trailing) {
    for (int d = 0; d < parent->rank - trailing; ++d) if (parent->shape[d] != 1) return false;
    return true;
}

// the batch dims of A stack its [M, K] matrices at a constant row pitch, i.e. A is one
// [batch*M, K] matrix with row stride A.strides[-2]
bool rows_fold(const tenmo_view* A, const Geometry& g) {
    const int own = A->rank - 2;
    if (own != g.batch_rank) return false;
    int64_t expect = A->shape[A->rank - 2] * A->strides[A->rank - 2];
    for (int d = own - 1; d >= 0; --d) {
        if (A->shape[d] != g.oshape[d]) return false;
        if (A->shape[d] > 1 && A->strides[d] != expect) return false;
        expect *= A->shape[d];
    }
    return true;
}

bool same_batch(const Geometry& g, const tenmo_view* parent, int trailing) {
    const int own = parent->rank - trailing;
    if (own != g.batch_rank) {
        // missing leading dims are fine only if the result's are all 1
        for (int d = 0; d < g.batch_rank - own; ++d) if (g.oshape[d] != 1) return false;
    }
    for (int d = std::max(0, g.batch_rank - own); d < g.batch_rank; ++d)
        if (parent->shape[d - (g.batch_rank - own)] != g.oshape[d]) return false;
    return true;
}

// grad (dense, at `parent`'s shape) += the product X . Y summed over the batch dims of the result that `parent` broadcast:
// the sum runs inside the GEMM launch (gemm_reduce_kernel), so no batched gradient is written and no reduction pass
// follows.  X, Y: the two factors as views whose batch dims broadcast to g's.  Returns 1 when it ran, 0 when the shape is
// not one the reducing launch takes (generic strides, or a result of so few tiles that spreading the batches over the
// chip and adding them afterwards is the better plan), a negative status on error.
int folded_gradient(const tenmo_view* X, const tenmo_view* Y, const Geometry& g, const tenmo_view* parent, float* grad) {
    if (S.fold_reduce == 0) return 0;
    const int64_t M = X->shape[X->rank - 2], K = X->shape[X->rank - 1], N = Y->shape[Y->rank - 1];
    const int64_t x_rs = X->strides[X->rank - 2], x_cs = X->strides[X->rank - 1], y_rs = Y->strides[Y->rank - 2], y_cs = Y->strides[Y->rank - 1];
    const int am = operand_mode(x_rs, x_cs, M, K), bm = operand_mode(y_cs, y_rs, N, K);
    if (M == 0 || N == 0) return 0;
    const bool generic = am == KMAJOR_GEN || bm == KMAJOR_GEN; // an operand without a unit stride: the 64x64 tile's element-wise loader
    int64_t xs[MAX_BATCH_RANK] = {0}, ys[MAX_BATCH_RANK] = {0};
    batch_strides_of(X, X->rank - 2, g.batch_rank, xs);
    batch_strides_of(Y, Y->rank - 2, g.batch_rank, ys);
    GemmArgs a{};
    BatchReduce red{};
    for (int d = 0; d < MAX_BATCH_RANK; ++d) { a.batch.shape[d] = 1; red.dims.shape[d] = 1; }
    const int own = parent->rank - 2;
    int64_t kept_count = 1;
    red.count = 1;
    for (int d = 0; d < g.batch_rank; ++d) {
        const int od = d - (g.batch_rank - own);
        const bool kept = od >= 0 && parent->shape[od] > 1;
        BatchDesc& bd = kept ? a.batch : red.dims;
        bd.shape[bd.rank] = g.oshape[d];
        bd.a_str[bd.rank] = xs[d];
        bd.b_str[bd.rank] = ys[d];
        ++bd.rank;
        (kept ? kept_count : red.count) *= g.oshape[d];
    }
    if (red.count <= 1) return 0;
    const int64_t tiles128 = ((M + 127) / 128) * ((N + 127) / 128) * kept_count, tiles64 = ((M + 63) / 64) * ((N + 63) / 64) * kept_count;
    const bool big = tiles128 >= (int64_t)S.cus && !generic;
    if (S.fold_reduce < 0 && !big && tiles64 < (int64_t)S.cus / 2) return 0;
    if (tiles64 > 0x7fffffffLL) return 0;
    a.A = X->data + X->offset; a.B = Y->data + Y->offset; a.C = grad;
    a.a_rs = x_rs; a.a_cs = x_cs; a.b_rs = y_rs; a.b_cs = y_cs;
    a.M = M; a.N = N; a.K = K;
    a.accumulate = 1;
    a.batch_count = kept_count;
    a.k_splits = 1; a.k_per_split = K;
    const int t = big ? 128 : 64;
    a.tiles_m = (int32_t)((M + t - 1) / t);
    a.tiles_n = (int32_t)((N + t - 1) / t);
    if (S.verbose) fprintf(stderr, "tenmo_hip gradient of a broadcast parent: %lld batches summed inside %lld tiles of %dx%d\n", (long long)red.count,
                           (long long)(big ? tiles128 : tiles64), t, t);
    const bool ok = big ? launch_gemm_reduce_128x128(a, red, (unsigned)tiles128, am, bm, S.stream) : launch_gemm_reduce_64x64(a, red, (unsigned)tiles64, am, bm, S.stream);
    return ok ? 1 : 0;
}

// ---- cross-entropy forward: pick the kernel that reads a row once --------------------------------
template <typename IdxT, bool VEC>
void launch_ce_forward_t(const CeForwardArgs& a) {
    const int64_t C = a.C, M = a.M;
    // the row lives in registers: THREADS * EPT >= C, the smallest EPT that fits
#define TENMO_CE_REGS(THREADS, EPT)                                                                                      \
    if (C + 3 <= (int64_t)(THREADS) * (EPT)) {                                                                           \
        const dim3 grid((unsigned)std::min<int64_t>(M, (int64_t)S.cus * (2048 / (THREADS)))), block(THREADS);             \
        hipLaunchKernelGGL((ce_forward_regs_kernel<IdxT, THREADS, EPT, VEC>), grid, block, 0, S.stream, a);               \
        return;                                                                                                          \
    }
    TENMO_CE_REGS(256, 4) TENMO_CE_REGS(256, 8) TENMO_CE_REGS(256, 16) TENMO_CE_REGS(256, 32)
    TENMO_CE_REGS(1024, 16) TENMO_CE_REGS(1024, 32) TENMO_CE_REGS(1024, 64)
#undef TENMO_CE_REGS
    // longer rows: three passes over the row (16-byte accesses only when every row is aligned)
    const dim3 grid((unsigned)std::min<int64_t>(M, (int64_t)S.cus * 8)), block(CE_THREADS);
    if (VEC && C % 4 == 0 && (uintptr_t)a.logits % 16 == 0) hipLaunchKernelGGL((ce_forward_block_kernel<IdxT, true>), grid, block, 0, S.stream, a);
    else hipLaunchKernelGGL((ce_forward_block_kernel<IdxT, false>), grid, block, 0, S.stream, a);
}

void launch_ce_forward(const CeForwardArgs& a, bool int64_target, bool vec) {
    if (int64_target) { if (vec) launch_ce_forward_t<int64_t, true>(a); else launch_ce_forward_t<int64_t, false>(a); }
    else { if (vec) launch_ce_forward_t<int32_t, true>(a); else launch_ce_forward_t<int32_t, false>(a); }
}

} // namespace

// ================================================================================================
// C ABI
// ================================================================================================
extern "C" {

const char* tenmo_hip_last_error(void) { return t_err.c_str(); }

int tenmo_hip_init(int device_id) {
    std::lock_guard<std::mutex> lock(S_mu);
    if (S.ready) {
        if (S.device == device_id) return 0;
        return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_init: already initialised on device %d", S.device);
    }
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count));
    if (device_id < 0 || device_id >= count) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_init: device %d not present (%d visible)", device_id, count);
    HIP_TRY(hipSetDevice(device_id));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device_id));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail(TENMO_ERR_UNSUPPORTED, "tenmo_hip_init: device %d is %s; this library is built for gfx950 only", device_id, prop.gcnArchName);
    S.device = device_id;
    S.cus = prop.multiProcessorCount;
    S.name = prop.name;
    HIP_TRY(hipStreamCreate(&S.own_stream));
    S.stream = S.own_stream;
    HIP_TRY(hipEventCreate(&S.ev0));
    HIP_TRY(hipEventCreate(&S.ev1));
    // address of the static scratch array on THIS device (each GPU holds its own copy); asked for once per device
    if (device_id < kMaxDevices && !g_scratch_ptr[device_id]) {
        float* p = nullptr;
        HIP_TRY(hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch)));
        g_scratch_ptr[device_id] = p;
    }
    HIP_TRY(hipMalloc(&S.one, sizeof(float)));
    const float one = 1.0f;
    HIP_TRY(hipMemcpy(S.one, &one, sizeof one, hipMemcpyHostToDevice));
    HIP_TRY(hipMalloc(&S.arrivals, kArrivalCounters * sizeof(uint32_t)));
    HIP_TRY(hipMemset(S.arrivals, 0, kArrivalCounters * sizeof(uint32_t)));
    S.force_tile = env_int("TENMO_HIP_GEMM_TILE", -1);
    S.force_splitk = env_int("TENMO_HIP_GEMM_SPLITK", -1);
    S.force_streamk = env_int("TENMO_HIP_GEMM_STREAMK", -1);
    S.force_smallk = env_int("TENMO_HIP_GEMM_SMALLK", -1);
    S.force_panel = env_int("TENMO_HIP_GEMM_PANEL", -1);
    S.verbose = env_int("TENMO_HIP_VERBOSE", 0);
    S.ready = true;
    return 0;
}

int tenmo_hip_shutdown(void) {
    std::lock_guard<std::mutex> lock(S_mu);
    if (!S.ready) return 0;
    // teardown: nothing useful can be done with a failure here
    (void)hipStreamSynchronize(S.stream);
    if (S.ws) (void)hipFree(S.ws);
    if (S.ws2) (void)hipFree(S.ws2);
    if (S.one) (void)hipFree(S.one);
    if (S.arrivals) (void)hipFree(S.arrivals);
    if (S.conv_tables) (void)hipFree(S.conv_tables);
    for (int i = 0; i < 3; ++i) if (S.stage[i]) (void)hipFree(S.stage[i]);
    (void)hipEventDestroy(S.ev0);
    (void)hipEventDestroy(S.ev1);
    (void)hipStreamDestroy(S.own_stream);
    S = State();
    return 0;
}

int tenmo_hip_sync(void) {
    if (int rc = ensure_ready()) return rc;
    HIP_TRY(hipStreamSynchronize(S.stream));
    return 0;
}

void* tenmo_hip_get_stream(void) { return S.ready ? (void*)S.stream : nullptr; }

int tenmo_hip_set_stream(void* s) {
    if (int rc = ensure_ready()) return rc;
    HIP_TRY(hipStreamSynchronize(S.stream));
    S.stream = s ? (hipStream_t)s : S.own_stream;
    return 0;
}

int tenmo_hip_device_info(int* cus, char* name, int name_len) {
    if (int rc = ensure_ready()) return rc;
    if (cus) *cus = S.cus;
    if (name && name_len > 0) { strncpy(name, S.name.c_str(), name_len - 1); name[name_len - 1] = 0; }
    return 0;
}

int tenmo_hip_set_tuning(const char* name, int value) {
    if (!name) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_set_tuning: null name");
    if (!strcmp(name, "gemm_tile")) { S.force_tile = value; return 0; }
    if (!strcmp(name, "gemm_splitk")) { S.force_splitk = value; return 0; }
    if (!strcmp(name, "gemm_streamk")) { S.force_streamk = value; return 0; }
    if (!strcmp(name, "gemm_smallk")) { S.force_smallk = value; return 0; }
    if (!strcmp(name, "gemm_panel")) { S.force_panel = value; return 0; }
    if (!strcmp(name, "gemm_resident")) { S.force_resident = value > 0 ? value : 0; return 0; }
    if (!strcmp(name, "fold_reduce")) { S.fold_reduce = value; return 0; }
    if (!strcmp(name, "mlp_fused_tail")) { S.mlp_fused_tail = value; return 0; }
    if (!strcmp(name, "conv_phases")) { S.force_conv_phases = value; return 0; }
    if (!strcmp(name, "cols_join")) { S.cols_join = value > 0 ? 1 : 0; return 0; }
    if (!strcmp(name, "cols_wg_per_cu")) { S.cols_waves_per_cu = value > 0 ? value : 2; return 0; }
    return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_set_tuning: unknown knob '%s'", name);
}

int tenmo_hip_timer_begin(void) {
    if (int rc = ensure_ready()) return rc;
    HIP_TRY(hipEventRecord(S.ev0, S.stream));
    return 0;
}

int tenmo_hip_timer_end(float* ms) {
    if (int rc = ensure_ready()) return rc;
    HIP_TRY(hipEventRecord(S.ev1, S.stream));
    HIP_TRY(hipEventSynchronize(S.ev1));
    HIP_TRY(hipEventElapsedTime(ms, S.ev0, S.ev1));
    return 0;
}

int tenmo_hip_clock_probe(int32_t rounds, float* effective_mhz) {
    if (int rc = ensure_ready()) return rc;
    if (rounds < 1 || !effective_mhz) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_clock_probe: needs rounds >= 1 and a result pointer");
    hipLaunchKernelGGL(clock_probe_kernel, dim3((unsigned)S.cus), dim3(256), 0, S.stream, 1000, 1.0f); // brings the clocks up
    HIP_TRY(hipEventRecord(S.ev0, S.stream));
    hipLaunchKernelGGL(clock_probe_kernel, dim3((unsigned)S.cus), dim3(256), 0, S.stream, (int)rounds, 1.0f);
    HIP_TRY(hipEventRecord(S.ev1, S.stream));
    HIP_TRY(hipEventSynchronize(S.ev1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, S.ev0, S.ev1));
    HIP_TRY(hipGetLastError());
    if (!(ms > 0.f)) return fail(TENMO_ERR_HIP, "tenmo_hip_clock_probe: no elapsed time");
    *effective_mhz = (float)(4.0 * rounds * 64.0 / (ms * 1e-3) / 1e6);
    return 0;
}

int tenmo_hip_gemm_f32(const float* A, int64_t a_off, int64_t a_rs, int64_t a_cs,
                       const float* B, int64_t b_off, int64_t b_rs, int64_t b_cs,
                       float* C, int64_t M, int64_t N, int64_t K,
                       int32_t batch_rank, const int64_t* batch_shape,
                       const int64_t* a_batch_strides, const int64_t* b_batch_strides,
                       int32_t accumulate, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (M < 0 || N < 0 || K < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_gemm_f32: negative dimension");
    if (int rc = need(C, M * N > 0, "tenmo_hip_gemm_f32", "result pointer")) return rc;
    if ((!A || !B) && M * N * K > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_gemm_f32: null pointer");
    BatchDesc bd{};
    int64_t count = 1;
    if (int rc = fill_batch(bd, batch_rank, batch_shape, a_batch_strides, b_batch_strides, &count)) return rc;
    if (int rc = product_dispatch(A + a_off, a_rs, a_cs, B + b_off, b_rs, b_cs, C, M, N, K, bd, count, accumulate)) return rc;
    return finish(sync);
}

int tenmo_hip_gemm_epilogue_f32(const float* A, int64_t a_off, int64_t a_rs, int64_t a_cs,
                                const float* B, int64_t b_off, int64_t b_rs, int64_t b_cs,
                                float* C, int64_t M, int64_t N, int64_t K,
                                int32_t batch_rank, const int64_t* batch_shape,
                                const int64_t* a_batch_strides, const int64_t* b_batch_strides,
                                const float* bias, int32_t relu, const float* mask, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (M < 0 || N < 0 || K < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_gemm_epilogue_f32: negative dimension");
    if (int rc = need(C, M * N > 0, "tenmo_hip_gemm_epilogue_f32", "result pointer")) return rc;
    if ((!A || !B) && M * N * K > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_gemm_epilogue_f32: null pointer");
    if (K == 0 && M * N > 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_gemm_epilogue_f32: K = 0");
    BatchDesc bd{};
    int64_t count = 1;
    if (int rc = fill_batch(bd, batch_rank, batch_shape, a_batch_strides, b_batch_strides, &count)) return rc;
    Epilogue ep;
    ep.bias = bias; ep.relu = relu ? 1 : 0; ep.mask = mask;
    if (int rc = gemm_dispatch(A + a_off, a_rs, a_cs, B + b_off, b_rs, b_cs, C, M, N, K, bd, count, 0, ep)) return rc;
    return finish(sync);
}

int tenmo_hip_mv_f32(const float* Mx, int64_t m_off, int64_t m_rs, int64_t m_cs,
                     const float* v, int64_t v_off, int64_t v_s,
                     float* out, int64_t m, int64_t k,
                     int32_t batch_rank, const int64_t* batch_shape,
                     const int64_t* m_batch_strides, const int64_t* v_batch_strides,
                     int32_t accumulate, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (m < 0 || k < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_mv_f32: negative dimension");
    BatchDesc bd{};
    int64_t count = 1;
    if (int rc = fill_batch(bd, batch_rank, batch_shape, m_batch_strides, v_batch_strides, &count)) return rc;
    if (int rc = need(out, m * count > 0, "tenmo_hip_mv_f32", "result pointer")) return rc;
    if ((!Mx || !v) && m * k * count > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mv_f32: null operand");
    if (int rc = matvec_dispatch(Mx + m_off, m_rs, m_cs, v + v_off, v_s, out, m, k, bd, count, accumulate)) return rc;
    return finish(sync);
}

int tenmo_hip_vm_f32(const float* v, int64_t v_off, int64_t v_s,
                     const float* Mx, int64_t m_off, int64_t m_rs, int64_t m_cs,
                     float* out, int64_t k, int64_t n,
                     int32_t batch_rank, const int64_t* batch_shape,
                     const int64_t* v_batch_strides, const int64_t* m_batch_strides,
                     int32_t accumulate, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (n < 0 || k < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_vm_f32: negative dimension");
    BatchDesc bd{};
    int64_t count = 1;
    // matvec_dispatch wants (matrix, vector) order in the batch descriptor
    if (int rc = fill_batch(bd, batch_rank, batch_shape, m_batch_strides, v_batch_strides, &count)) return rc;
    if (int rc = need(out, n * count > 0, "tenmo_hip_vm_f32", "result pointer")) return rc;
    if ((!Mx || !v) && n * k * count > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_vm_f32: null operand");
    // out[j] = sum_i Mx(i, j) v(i): outputs walk the matrix columns, the reduction walks its rows
    if (int rc = matvec_dispatch(Mx + m_off, m_cs, m_rs, v + v_off, v_s, out, n, k, bd, count, accumulate)) return rc;
    return finish(sync);
}

// tenmo_hip_vm_f32 for callers that cannot allocate: the K-slice partial sums go to the static device array
// `scratch` (through the address this device reported at init) instead of the grow-only library buffer.  No
// hipMalloc / hipFree on this path; every partial sum the slice reduction reads is written by the launch before it,
// so nothing has to be cleared between calls.
int tenmo_hip_vm_f32_noalloc(const float* v, int64_t v_off, int64_t v_s,
                             const float* Mx, int64_t m_off, int64_t m_rs, int64_t m_cs,
                             float* out, int64_t k, int64_t n,
                             int32_t batch_rank, const int64_t* batch_shape,
                             const int64_t* v_batch_strides, const int64_t* m_batch_strides,
                             int32_t accumulate, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (n < 0 || k < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_vm_f32_noalloc: negative dimension");
    if (S.device < 0 || S.device >= kMaxDevices || !g_scratch_ptr[S.device])
        return fail(TENMO_ERR_NOT_INITIALIZED, "tenmo_hip_vm_f32_noalloc: no static scratch address for device %d", S.device);
    BatchDesc bd{};
    int64_t count = 1;
    if (int rc = fill_batch(bd, batch_rank, batch_shape, m_batch_strides, v_batch_strides, &count)) return rc;
    if (int rc = need(out, n * count > 0, "tenmo_hip_vm_f32_noalloc", "result pointer")) return rc;
    if ((!Mx || !v) && n * k * count > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_vm_f32_noalloc: null operand");
    ScratchSource src;
    src.fixed = g_scratch_ptr[S.device];
    src.fixed_bytes = TENMO_STATIC_SCRATCH_BYTES;
    if (int rc = matvec_dispatch(Mx + m_off, m_cs, m_rs, v + v_off, v_s, out, n, k, bd, count, accumulate, src)) return rc;
    return finish(sync);
}

int tenmo_hip_column_sum_f32(const float* G, int64_t g_off, int64_t g_rs, int64_t rows, int64_t cols,
                             float* out, int32_t accumulate, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (rows < 0 || cols < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_column_sum_f32: negative dimension");
    if (int rc = need(out, cols > 0, "tenmo_hip_column_sum_f32", "result pointer")) return rc;
    if (!G && rows * cols > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_column_sum_f32: null operand");
    // ones[rows] . G[rows, cols] with the ones read through stride 0: the matrix is streamed once
    BatchDesc bd{};
    for (int d = 0; d < MAX_BATCH_RANK; ++d) bd.shape[d] = 1;
    if (int rc = matvec_dispatch(G + g_off, 1, g_rs, S.one, 0, out, cols, rows, bd, 1, accumulate)) return rc;
    return finish(sync);
}

int tenmo_hip_cross_entropy_forward_f32(const float* logits, const void* target, int32_t target_is_int64, int64_t M, int64_t C,
                                        int64_t ignore_index, float label_smoothing,
                                        float* softmax_out, float* per_sample_loss, float* loss_sum, int32_t* valid_count, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    const char* who = "tenmo_hip_cross_entropy_forward_f32";
    if (M < 0 || C < 1) return fail(TENMO_ERR_INVALID_SHAPE, "%s: needs M >= 0 rows and C >= 1 classes", who);
    if (!(label_smoothing >= 0.f && label_smoothing <= 1.f))
        return fail(TENMO_ERR_INVALID_ARGUMENT, "CrossEntropyLoss: label_smoothing must be in [0, 1], got %g", (double)label_smoothing);
    if (int rc = need(loss_sum, true, who, "loss_sum")) return rc;
    if (int rc = need(valid_count, true, who, "valid_count")) return rc;
    if (M > 0 && (!logits || !target || !per_sample_loss)) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    if (M > 0) {
        CeForwardArgs a{};
        a.logits = logits; a.target = target; a.softmax_out = softmax_out; a.row_loss = per_sample_loss;
        a.M = M; a.C = C; a.ignore_index = ignore_index; a.label_smoothing = label_smoothing;
        if (C <= 32) { // short rows: a thread each
            const dim3 grid((unsigned)((M + 127) / 128)), block(128);
            if (target_is_int64) hipLaunchKernelGGL(ce_forward_rows_kernel<int64_t>, grid, block, 0, S.stream, a);
            else hipLaunchKernelGGL(ce_forward_rows_kernel<int32_t>, grid, block, 0, S.stream, a);
        } else if ((uintptr_t)logits % 4 == 0 &&
                   (softmax_out ? (C >= 40000 && (uintptr_t)softmax_out % 16 == 0 && (uintptr_t)logits % 16 == 0) : C >= 256)) {
            // streaming form: row statistics (max, 1/sum, loss) in one read-only pass, then the softmax as a flat
            // sweep.  Always when only the loss is wanted (2x faster than holding the row in registers); with the
            // softmax for the longest rows, where the two passes together beat the register-resident single pass
            CeRowStats* stats = nullptr;
            if (softmax_out) {
                float* ws;
                if (int rc = workspace((size_t)M * sizeof(CeRowStats), &ws)) return rc;
                stats = reinterpret_cast<CeRowStats*>(ws);
            }
            if (M > 0x7fffffffLL) return fail(TENMO_ERR_UNSUPPORTED, "%s: grid too large", who);
            const bool i64 = target_is_int64 != 0;
            if (C >= 8192) { // the whole workgroup on one row
                const dim3 grid((unsigned)M), block(CE_THREADS);
                if (i64) hipLaunchKernelGGL((ce_stats_kernel<int64_t, CE_THREADS / 64, 8>), grid, block, 0, S.stream, a, stats);
                else hipLaunchKernelGGL((ce_stats_kernel<int32_t, CE_THREADS / 64, 8>), grid, block, 0, S.stream, a, stats);
            } else { // a wavefront per row
                const dim3 grid((unsigned)((M + CE_THREADS / 64 - 1) / (CE_THREADS / 64))), block(CE_THREADS);
                if (i64) hipLaunchKernelGGL((ce_stats_kernel<int64_t, 1, 4>), grid, block, 0, S.stream, a, stats);
                else hipLaunchKernelGGL((ce_stats_kernel<int32_t, 1, 4>), grid, block, 0, S.stream, a, stats);
            }
            if (softmax_out) {
                constexpr int64_t per_block = CE_THREADS * 4 * 4; // elements per workgroup and pass
                const int64_t blocks = std::max<int64_t>(1, std::min<int64_t>((M * C + per_block - 1) / per_block, (int64_t)S.cus * 16));
                CeFlatSteps st{};
                st.pass_rows = blocks * per_block / C; st.pass_cols = blocks * per_block % C;
                st.unit_rows = CE_THREADS * 4 / C; st.unit_cols = CE_THREADS * 4 % C;
                hipLaunchKernelGGL(ce_softmax_flat_kernel, dim3((unsigned)blocks), dim3(CE_THREADS), 0, S.stream, logits, softmax_out, stats, M, C, st);
            }
        } else {
            // 16-byte accesses need the two arrays congruent modulo 16 bytes (then their rows are too)
            const bool vec = (uintptr_t)logits % 4 == 0 && (!softmax_out || (uintptr_t)softmax_out % 16 == (uintptr_t)logits % 16);
            launch_ce_forward(a, target_is_int64 != 0, vec);
        }
    }
    if (target_is_int64) hipLaunchKernelGGL(ce_finish_kernel<int64_t>, dim3(1), dim3(1024), 0, S.stream, per_sample_loss, (const int64_t*)target, M, ignore_index, loss_sum, valid_count);
    else hipLaunchKernelGGL(ce_finish_kernel<int32_t>, dim3(1), dim3(1024), 0, S.stream, per_sample_loss, (const int32_t*)target, M, ignore_index, loss_sum, valid_count);
    return finish(sync);
}

int tenmo_hip_cross_entropy_backward_f32(const float* softmax, const void* target, int32_t target_is_int64, const float* upstream,
                                         int64_t M, int64_t C, int64_t ignore_index, float label_smoothing,
                                         int32_t reduction, int32_t valid_count, float* grad_logits, int32_t accumulate, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    const char* who = "tenmo_hip_cross_entropy_backward_f32";
    if (M < 0 || C < 1) return fail(TENMO_ERR_INVALID_SHAPE, "%s: needs M >= 0 rows and C >= 1 classes", who);
    if (reduction < 0 || reduction > 2) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: reduction must be 0 (none), 1 (sum) or 2 (mean)", who);
    if (M == 0) return 0;
    if (!softmax || !target || !upstream || !grad_logits) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    CeBackwardArgs a{};
    a.softmax = softmax; a.target = target; a.upstream = upstream; a.grad = grad_logits;
    a.M = M; a.C = C; a.ignore_index = ignore_index; a.label_smoothing = label_smoothing;
    a.reduction = reduction; a.valid_count = valid_count; a.accumulate = accumulate ? 1 : 0;
    if (C >= 4 && (uintptr_t)softmax % 16 == 0 && (uintptr_t)grad_logits % 16 == 0) {
        // flat sweep: every group of four consecutive elements of the [M*C] array is one 16-byte access
        constexpr int64_t per_block = CE_THREADS * 4 * 4; // elements per workgroup and pass
        const int64_t blocks = std::max<int64_t>(1, std::min<int64_t>((M * C + per_block - 1) / per_block, (int64_t)S.cus * 16));
        CeFlatSteps st{};
        st.pass_rows = blocks * per_block / C; st.pass_cols = blocks * per_block % C;
        st.unit_rows = CE_THREADS * 4 / C; st.unit_cols = CE_THREADS * 4 % C;
        const dim3 grid((unsigned)blocks), block(CE_THREADS);
        if (target_is_int64) hipLaunchKernelGGL(ce_backward_flat_kernel<int64_t>, grid, block, 0, S.stream, a, st);
        else hipLaunchKernelGGL(ce_backward_flat_kernel<int32_t>, grid, block, 0, S.stream, a, st);
        return finish(sync);
    }
    // enough workgroups per row to fill the chip when there are few long rows
    int64_t chunks = std::max<int64_t>(1, std::min<int64_t>((C + CE_THREADS * 16 - 1) / (CE_THREADS * 16), ((int64_t)S.cus * 8 + M - 1) / M));
    if (M * chunks > 0x7fffffffLL) return fail(TENMO_ERR_UNSUPPORTED, "%s: grid too large", who);
    a.chunks = (int32_t)chunks;
    const dim3 grid((unsigned)(M * chunks)), block(CE_THREADS);
    const bool vec = (uintptr_t)softmax % 4 == 0 && (uintptr_t)softmax % 16 == (uintptr_t)grad_logits % 16;
    if (target_is_int64) {
        if (vec) hipLaunchKernelGGL((ce_backward_kernel<int64_t, true>), grid, block, 0, S.stream, a);
        else hipLaunchKernelGGL((ce_backward_kernel<int64_t, false>), grid, block, 0, S.stream, a);
    } else {
        if (vec) hipLaunchKernelGGL((ce_backward_kernel<int32_t, true>), grid, block, 0, S.stream, a);
        else hipLaunchKernelGGL((ce_backward_kernel<int32_t, false>), grid, block, 0, S.stream, a);
    }
    return finish(sync);
}

// out[n, c_out, h_out, w_out] (+)= conv(padded_image, kernel) + bias as an implicit GEMM per image:
// out[C_out, H_out*W_out] = kernel[C_out, C_in*KH*KW] . patches[C_in*KH*KW, H_out*W_out] + bias[row].
// Sizes are validated by the callers.  The offset tables are rebuilt only when the geometry changes.
static int conv_tables(const ConvGeometry& geo, int32_t** by_k, int32_t** by_pos) {
    const int64_t nk = (int64_t)geo.c_in * geo.kh * geo.kw, np = (int64_t)geo.h_out * geo.w_out;
    const size_t need_len = (size_t)(nk + np);
    if (need_len > S.conv_tables_len) {
        if (S.conv_tables) {
            HIP_TRY(hipStreamSynchronize(S.stream));
            HIP_TRY(hipFree(S.conv_tables));
            S.conv_tables = nullptr; S.conv_tables_len = 0;
        }
        HIP_TRY(hipMalloc(&S.conv_tables, need_len * sizeof(int32_t)));
        S.conv_tables_len = need_len;
        S.conv_geometry = ConvGeometry{};
    }
    *by_k = S.conv_tables;
    *by_pos = S.conv_tables + nk;
    if (memcmp(&geo, &S.conv_geometry, sizeof geo) != 0) {
        const int64_t n = std::max(nk, np);
        hipLaunchKernelGGL(conv_tables_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, S.stream, geo, *by_k, *by_pos);
        S.conv_geometry = geo;
    }
    return 0;
}

static int conv_forward_impl(const float* padded_image, int64_t n_images, const ConvGeometry& geo, const float* kernel, int64_t c_out,
                             const float* bias, float* out, int accumulate) {
    int32_t *by_k, *by_pos;
    if (int rc = conv_tables(geo, &by_k, &by_pos)) return rc;
    const int64_t nk = (int64_t)geo.c_in * geo.kh * geo.kw, np = (int64_t)geo.h_out * geo.w_out;
    BatchDesc bd{};
    bd.rank = 1; bd.shape[0] = n_images; bd.a_str[0] = 0; bd.b_str[0] = (int64_t)geo.c_in * geo.h_pad * geo.w_pad;
    Epilogue ep;
    ep.bias = bias; ep.bias_rows = 1; ep.gather_row = by_pos; ep.gather_k = by_k;
    return gemm_dispatch(kernel, nk, 1, padded_image, 0, 0, out, c_out, np, nk, bd, n_images, accumulate, ep);
}

// shared argument checks of the two convolution entries; fills `geo`
static int conv_check(const char* who, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad, int64_t c_out, int64_t kh, int64_t kw,
                      int64_t stride, int64_t dilation, ConvGeometry* geo) {
    if (n_images < 0 || c_in < 1 || c_out < 1 || kh < 1 || kw < 1 || h_pad < 1 || w_pad < 1)
        return fail(TENMO_ERR_INVALID_SHAPE, "%s: image (N=%lld, C_in=%lld, %lldx%lld), kernel (C_out=%lld, %lldx%lld): sizes must be positive",
                    who, (long long)n_images, (long long)c_in, (long long)h_pad, (long long)w_pad, (long long)c_out, (long long)kh, (long long)kw);
    if (stride < 1 || dilation < 1) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: stride and dilation must be >= 1", who);
    const int64_t dkh = kh + (kh - 1) * (dilation - 1), dkw = kw + (kw - 1) * (dilation - 1);
    if (h_pad < dkh || w_pad < dkw) return fail(TENMO_ERR_INVALID_SHAPE, "%s: Invalid output dimensions (the dilated kernel %lldx%lld exceeds the padded image %lldx%lld)",
                                                who, (long long)dkh, (long long)dkw, (long long)h_pad, (long long)w_pad);
    const int64_t h_out = (h_pad - dkh) / stride + 1, w_out = (w_pad - dkw) / stride + 1;
    // the input-gradient pass convolves an array of (h_pad + dkh - 1) x (w_pad + dkw - 1) per channel: bound that one too
    if (std::max(c_in, c_out) * (h_pad + dkh) * (w_pad + dkw) > 0x7fffffffLL || c_in * kh * kw > 0x7fffffffLL || c_out * kh * kw > 0x7fffffffLL)
        return fail(TENMO_ERR_UNSUPPORTED, "%s: one image or one patch matrix dimension exceeds 2^31 elements", who);
    *geo = ConvGeometry{(int32_t)c_in, (int32_t)h_pad, (int32_t)w_pad, (int32_t)kh, (int32_t)kw, (int32_t)h_out, (int32_t)w_out, (int32_t)stride, (int32_t)dilation};
    return 0;
}

int tenmo_hip_conv2d_forward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                                 const float* kernel, int64_t c_out, int64_t kh, int64_t kw, const float* bias,
                                 int64_t stride, int64_t dilation, float* out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    const char* who = "tenmo_hip_conv2d_forward_f32";
    ConvGeometry geo;
    if (int rc = conv_check(who, n_images, c_in, h_pad, w_pad, c_out, kh, kw, stride, dilation, &geo)) return rc;
    if (n_images == 0) return 0;
    if (!padded_image || !kernel || !out) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    if (int rc = conv_forward_impl(padded_image, n_images, geo, kernel, c_out, bias, out, 0)) return rc;
    return finish(sync);
}

int tenmo_hip_conv2d_backward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                                  const float* kernel, int64_t c_out, int64_t kh, int64_t kw, int64_t stride, int64_t dilation,
                                  const float* grad_out, float* grad_padded_image, float* grad_kernel, float* grad_bias,
                                  int32_t accumulate, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    const char* who = "tenmo_hip_conv2d_backward_f32";
    ConvGeometry geo;
    if (int rc = conv_check(who, n_images, c_in, h_pad, w_pad, c_out, kh, kw, stride, dilation, &geo)) return rc;
    if (n_images == 0) return 0;
    if (!grad_out) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: null upstream gradient", who);
    if (grad_kernel && !padded_image) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: the kernel gradient needs the padded image", who);
    if (grad_padded_image && !kernel) return fail(TENMO_ERR_INVALID_ARGUMENT, "%s: the image gradient needs the kernel", who);
    const int64_t np = (int64_t)geo.h_out * geo.w_out, nk = c_in * kh * kw;
    const int acc = accumulate ? 1 : 0;
    BatchDesc one_batch{};
    for (int d = 0; d < MAX_BATCH_RANK; ++d) one_batch.shape[d] = 1;

    if (grad_bias) { // sums over (n, y, x) per output channel: row sums of [N*C_out, H_out*W_out], then column sums over N
        if (n_images == 1) {
            if (int rc = matvec_dispatch(grad_out, np, 1, S.one, 0, grad_bias, c_out, np, one_batch, 1, acc)) return rc;
        } else {
            float* rows;
            if (int rc = workspace2((size_t)(n_images * c_out) * sizeof(float), &rows)) return rc;
            if (int rc = matvec_dispatch(grad_out, np, 1, S.one, 0, rows, n_images * c_out, np, one_batch, 1, 0)) return rc;
            if (int rc = matvec_dispatch(rows, 1, c_out, S.one, 0, grad_bias, c_out, n_images, one_batch, 1, acc)) return rc;
        }
    }
    if (grad_kernel) { // per image grad_out[C_out, P] . patches^T[P, C_in*KH*KW] (the patches gathered), summed over the images
        int32_t *by_k, *by_pos;
        if (int rc = conv_tables(geo, &by_k, &by_pos)) return rc;
        BatchDesc bd{};
        bd.rank = 1; bd.shape[0] = n_images; bd.a_str[0] = c_out * np; bd.b_str[0] = c_in * h_pad * w_pad;
        Epilogue ep;
        ep.gather_row = by_k; ep.gather_k = by_pos; // B(n = patch element, k = position)
        ep.gather_kmajor = stride == 1;             // neighbouring positions of an output row are neighbours in the image
        if (n_images == 1) {
            if (int rc = gemm_dispatch(grad_out, np, 1, padded_image, 0, 0, grad_kernel, c_out, nk, np, bd, 1, acc, ep)) return rc;
        } else {
            float* per_image;
            if (int rc = workspace2((size_t)(n_images * c_out * nk) * sizeof(float), &per_image)) return rc;
            if (int rc = gemm_dispatch(grad_out, np, 1, padded_image, 0, 0, per_image, c_out, nk, np, bd, n_images, 0, ep)) return rc;
            if (int rc = matvec_dispatch(per_image, 1, c_out * nk, S.one, 0, grad_kernel, c_out * nk, n_images, one_batch, 1, acc)) return rc;
        }
    }
    const bool by_phase = stride > 1 && (S.force_conv_phases >= 0 ? S.force_conv_phases != 0
                                                                     : (double)n_images * c_in * c_out * kh * kw * h_pad * w_pad >= 5.0e8);
    if (grad_padded_image && by_phase) {
        // Strided layer: the image gradient phase by phase.  The input positions (y, x) with y % stride = py and
        // x % stride = px are reached only by the kernel taps with ky*dilation = py and kx*dilation = px modulo the stride,
        // each from the upstream element ((y - ky*dilation) / stride, ...): a stride-1 convolution of the upstream gradient
        // (zero-padded, not spread out) with those taps reversed, whose result goes to every stride-th position.  All
        // phases together do the multiply-adds of the forward pass; the single convolution below does stride^2 times as
        // many, most of them with the zeros between the spread-out elements.  (Small layers keep it: fewer launches.)
        const int64_t g = std::gcd(stride, dilation), tap_step = stride / g, tap_dil = dilation / g;
        struct Axis { int64_t first, count, last, amax, size; }; // taps ky = first + i*tap_step; amax = upstream offset of the last tap
        auto axis = [&](int64_t phase, int64_t ksize, int64_t extent, int64_t out_extent) {
            Axis a{-1, 0, -1, 0, 0};
            for (int64_t k = 0; k < ksize; ++k)
                if ((k * dilation - phase) % stride == 0) { if (a.first < 0) a.first = k; a.last = k; ++a.count; }
            a.size = phase < extent ? (extent - phase + stride - 1) / stride : 0;
            if (a.count) a.amax = (a.last * dilation - phase) / stride;
            (void)out_extent;
            return a;
        };
        int64_t max_src = 0, max_out = 0;
        for (int64_t py = 0; py < stride; ++py)
            for (int64_t px = 0; px < stride; ++px) {
                const Axis ay = axis(py, kh, h_pad, geo.h_out), ax = axis(px, kw, w_pad, geo.w_out);
                if (!ay.count || !ax.count || !ay.size || !ax.size) continue;
                max_src = std::max(max_src, n_images * c_out * (ay.size + (ay.count - 1) * tap_dil) * (ax.size + (ax.count - 1) * tap_dil));
                max_out = std::max(max_out, n_images * c_in * ay.size * ax.size);
            }
        const int64_t flip_len = c_out * c_in * kh * kw;
        float* buf = nullptr;
        if (max_src > 0)
            if (int rc = workspace2((size_t)(max_src + max_out + flip_len) * sizeof(float), &buf)) return rc;
        float *padded = buf, *phase_out = buf + max_src, *taps = buf + max_src + max_out;
        for (int64_t py = 0; py < stride; ++py)
            for (int64_t px = 0; px < stride; ++px) {
                const Axis ay = axis(py, kh, h_pad, geo.h_out), ax = axis(px, kw, w_pad, geo.w_out);
                if (!ay.size || !ax.size) continue;
                const int64_t planes = n_images * c_in;
                const dim3 sgrid((unsigned)std::min<int64_t>(planes, (int64_t)S.cus * 32)); // a workgroup per plane
                if (!ay.count || !ax.count) { // no tap reaches this phase: its gradient is zero
                    if (!acc) hipLaunchKernelGGL(conv_scatter_phase_kernel, sgrid, dim3(256), 0, S.stream, (const float*)nullptr, grad_padded_image, planes,
                                                 (int)h_pad, (int)w_pad, (int)ay.size, (int)ax.size, (int)py, (int)px, (int)stride, 0);
                    continue;
                }
                const int64_t h_src = ay.size + (ay.count - 1) * tap_dil, w_src = ax.size + (ax.count - 1) * tap_dil;
                const int64_t taps_len = c_out * c_in * ay.count * ax.count;
                hipLaunchKernelGGL(conv_dilate_pad_kernel, dim3((unsigned)std::min<int64_t>(n_images * c_out, (int64_t)S.cus * 32)), dim3(256), 0, S.stream,
                                   grad_out, padded, n_images * c_out, (int)geo.h_out, (int)geo.w_out, (int)h_src, (int)w_src, 1, (int)ay.amax, (int)ax.amax);
                hipLaunchKernelGGL(conv_flip_taps_kernel, dim3((unsigned)((taps_len + 255) / 256)), dim3(256), 0, S.stream, kernel, taps, (int)c_out, (int)c_in,
                                   (int)kh, (int)kw, (int)ay.count, (int)ax.count, (int)ay.last, (int)ax.last, (int)tap_step);
                const ConvGeometry back{(int32_t)c_out, (int32_t)h_src, (int32_t)w_src, (int32_t)ay.count, (int32_t)ax.count,
                                        (int32_t)ay.size, (int32_t)ax.size, 1, (int32_t)tap_dil};
                if (int rc = conv_forward_impl(padded, n_images, back, taps, c_in, nullptr, phase_out, 0)) return rc;
                hipLaunchKernelGGL(conv_scatter_phase_kernel, sgrid, dim3(256), 0, S.stream, (const float*)phase_out, grad_padded_image, planes,
                                   (int)h_pad, (int)w_pad, (int)ay.size, (int)ax.size, (int)py, (int)px, (int)stride, acc);
            }
    } else if (grad_padded_image) {
        // The scatter of the reference's loop (cnn.mojo:818-948) as a gather: a stride-1 convolution, same dilation, of the
        // upstream gradient spread out by `stride` and zero-padded by the dilated kernel size - 1, with the kernel's
        // channel axes swapped and its spatial axes reversed.
        const int64_t dkh = kh + (kh - 1) * (dilation - 1), dkw = kw + (kw - 1) * (dilation - 1);
        const int64_t h_dst = h_pad + dkh - 1, w_dst = w_pad + dkw - 1;
        const int64_t spread_len = n_images * c_out * h_dst * w_dst, flip_len = c_out * nk;
        float* buf;
        if (int rc = workspace2((size_t)(spread_len + flip_len) * sizeof(float), &buf)) return rc;
        float* spread = buf;
        float* flipped = buf + spread_len;
        hipLaunchKernelGGL(conv_dilate_pad_kernel, dim3((unsigned)std::min<int64_t>(n_images * c_out, (int64_t)S.cus * 32)), dim3(256), 0, S.stream,
                           grad_out, spread, n_images * c_out, (int)geo.h_out, (int)geo.w_out, (int)h_dst, (int)w_dst, (int)stride, (int)(dkh - 1), (int)(dkw - 1));
        hipLaunchKernelGGL(conv_flip_taps_kernel, dim3((unsigned)((flip_len + 255) / 256)), dim3(256), 0, S.stream, kernel, flipped, (int)c_out, (int)c_in,
                           (int)kh, (int)kw, (int)kh, (int)kw, (int)(kh - 1), (int)(kw - 1), 1);
        const ConvGeometry back{(int32_t)c_out, (int32_t)h_dst, (int32_t)w_dst, (int32_t)kh, (int32_t)kw, (int32_t)h_pad, (int32_t)w_pad, 1, (int32_t)dilation};
        if (int rc = conv_forward_impl(spread, n_images, back, flipped, c_in, nullptr, grad_padded_image, acc)) return rc;
    }
    return finish(sync);
}

int tenmo_hip_sgd_step_f32(float* param, const float* grad, float* velocity, int64_t n, float lr, float momentum, float weight_decay, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (n < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_sgd_step_f32: negative length");
    if (n == 0) return 0;
    if (!param || !grad) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_sgd_step_f32: null pointer");
    const bool vec = (uintptr_t)param % 16 == 0 && (uintptr_t)grad % 16 == 0 && (uintptr_t)velocity % 16 == 0;
    const int64_t work = vec ? (n + 15) / 16 : n; // the vector path moves four groups of four per thread and pass
    const dim3 grid((unsigned)std::max<int64_t>(1, std::min<int64_t>((work + 255) / 256, (int64_t)S.cus * 16))), block(256);
    if (vec) hipLaunchKernelGGL(sgd_step_kernel<true>, grid, block, 0, S.stream, param, grad, velocity, n, lr, momentum, weight_decay);
    else hipLaunchKernelGGL(sgd_step_kernel<false>, grid, block, 0, S.stream, param, grad, velocity, n, lr, momentum, weight_decay);
    return finish(sync);
}

int tenmo_hip_dot_f32(const float* a, int64_t a_off, int64_t a_s, const float* b, int64_t b_off, int64_t b_s,
                      int64_t n, float* out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (n < 0) return fail(TENMO_ERR_INVALID_SHAPE, "tenmo_hip_dot_f32: negative length");
    if (int rc = need(out, true, "tenmo_hip_dot_f32", "result pointer")) return rc;
    if ((!a || !b) && n > 0) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_dot_f32: null operand");
    const bool vec = a_s == 1 && b_s == 1 && n >= 4096; // 16-byte loads (alignment of 4 bytes is enough for them)
    const int parts = (int)std::max<int64_t>(1, std::min<int64_t>((n + DOT_THREADS * 8 - 1) / (DOT_THREADS * 8), vec ? (int64_t)S.cus * 8 : 1024));
    float* ws;
    if (int rc = workspace(parts * sizeof(float), &ws)) return rc;
    if (vec) hipLaunchKernelGGL(dot_partial_vec_kernel<4>, dim3(parts), dim3(DOT_THREADS), 0, S.stream, a + a_off, b + b_off, n, ws);
    else hipLaunchKernelGGL(dot_partial_kernel, dim3(parts), dim3(DOT_THREADS), 0, S.stream, a + a_off, a_s, b + b_off, b_s, n, ws);
    hipLaunchKernelGGL(dot_final_kernel, dim3(1), dim3(DOT_THREADS), 0, S.stream, ws, parts, out);
    return finish(sync);
}

int tenmo_hip_classify_matmul(int32_t ra, const int64_t* a, int32_t rb, const int64_t* b) {
    if (ra <= 1 && rb <= 1) return TENMO_OP_DOT;
    if (ra == 1 && rb >= 2) return TENMO_OP_VM;
    if (ra >= 2 && rb == 1) return TENMO_OP_MV;
    if (ra >= 2 && rb >= 2) return a[ra - 1] == b[rb - 2] ? TENMO_OP_MM : TENMO_OP_INVALID;
    return TENMO_OP_INVALID;
}

int64_t tenmo_hip_result_shape(int32_t op, const tenmo_view* A, const tenmo_view* B, int64_t* out_shape, int32_t* out_rank) {
    Geometry g;
    if (int rc = resolve(op, A, B, &g, "tenmo_hip_result_shape", false)) return rc;
    if (out_shape) std::copy(g.oshape, g.oshape + g.orank, out_shape);
    if (out_rank) *out_rank = g.orank;
    return product(g.oshape, g.orank);
}

int tenmo_hip_matmul_nd(const tenmo_view* A, const tenmo_view* B, float* C, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (int rc = matmul_views(A, B, C, 0, "tenmo_hip_matmul_nd")) return rc;
    return finish(sync);
}

int tenmo_hip_linear_nd(const tenmo_view* X, const tenmo_view* W, const float* bias, int32_t relu, float* out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    Epilogue ep;
    ep.bias = bias; ep.relu = relu ? 1 : 0;
    if (int rc = matmul_views(X, W, out, 0, "tenmo_hip_linear_nd", ep)) return rc;
    return finish(sync);
}

int tenmo_hip_matrix_vector_nd(const tenmo_view* Mx, const tenmo_view* v, float* out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    Geometry g;
    if (int rc = resolve(TENMO_OP_MV, Mx, v, &g, "tenmo_hip_matrix_vector_nd")) return rc;
    if (int rc = need(out, product(g.oshape, g.orank) > 0, "tenmo_hip_matrix_vector_nd", "result pointer")) return rc;
    const BatchDesc bd = make_batch(g, Mx, 2, v, 1);
    const int64_t m = Mx->shape[Mx->rank - 2], k = Mx->shape[Mx->rank - 1];
    if (int rc = matvec_dispatch(Mx->data + Mx->offset, Mx->strides[Mx->rank - 2], Mx->strides[Mx->rank - 1],
                                 v->data + v->offset, v->strides[v->rank - 1], out, m, k, bd, g.batch_count, 0)) return rc;
    return finish(sync);
}

int tenmo_hip_vector_matmul_nd(const tenmo_view* v, const tenmo_view* Mx, float* out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    Geometry g;
    if (int rc = resolve(TENMO_OP_VM, v, Mx, &g, "tenmo_hip_vector_matmul_nd")) return rc;
    if (int rc = need(out, product(g.oshape, g.orank) > 0, "tenmo_hip_vector_matmul_nd", "result pointer")) return rc;
    const BatchDesc bd = make_batch(g, Mx, 2, v, 1); // (matrix, vector) order
    const int64_t k = Mx->shape[Mx->rank - 2], n = Mx->shape[Mx->rank - 1];
    if (int rc = matvec_dispatch(Mx->data + Mx->offset, Mx->strides[Mx->rank - 1], Mx->strides[Mx->rank - 2],
                                 v->data + v->offset, v->strides[v->rank - 1], out, n, k, bd, g.batch_count, 0)) return rc;
    return finish(sync);
}

// The two gradient products of Matmul backward (the body of tenmo_hip_matmul_backward; `g` = resolve(A, B)).
// grad_b: when not null, the gradient of a bias [N] added to the product (Linear: Matmul, then Adder) is wanted as well —
// the upstream gradient summed over everything but its last axis.  Where dB runs as ONE product with dC as its right
// operand (a shared B: always for a Linear weight), the sums come out of that launch (Epilogue::bsum) and *bias_done
// is set; otherwise the caller streams dC once more.
static int matmul_backward_impl(const tenmo_view* A, const tenmo_view* B, const float* dC, float* grad_A, float* grad_B, const Geometry& g,
                                float* grad_b = nullptr, bool* bias_done = nullptr) {
    const tenmo_view dCv = dense_view(dC, g.oshape, g.orank);
    if (grad_A) { // dA = dC . B^T(view)   (tenmo/matmul.mojo:36-38, :116-121)
        const tenmo_view Bt = transposed_last2(B);
        if (same_batch(g, A, 2)) {
            if (int rc = matmul_views(&dCv, &Bt, grad_A, 1, "tenmo_hip_matmul_backward")) return rc;
        } else if (const int folded = folded_gradient(&dCv, &Bt, g, A, grad_A)) {
            if (folded < 0) return folded;
        } else {
            Geometry gg;
            if (int rc = resolve(TENMO_OP_MM, &dCv, &Bt, &gg, "tenmo_hip_matmul_backward")) return rc;
            // the GEMM may itself use the first scratch for split-K: the batched gradient lives in the second
            float* full = nullptr;
            if (int rc = workspace2((size_t)product(gg.oshape, gg.orank) * sizeof(float), &full)) return rc;
            if (int rc = matmul_views(&dCv, &Bt, full, 0, "tenmo_hip_matmul_backward")) return rc;
            if (int rc = reduce_to_parent(full, gg, A, 2, grad_A)) return rc;
        }
    }
    if (grad_B) { // dB = A^T(view) . dC   (tenmo/matmul.mojo:46-48, :127-132)
        const tenmo_view At = transposed_last2(A);
        if (!same_batch(g, B, 2) && all_broadcast(B, 2) && rows_fold(A, g)) {
            // B is shared by every batch (a Linear weight under a batched input): the sum over batches
            // of A_b^T . dC_b is ONE product with the batch folded into the reduction,
            // [K, batch*M] . [batch*M, N], accumulated straight into the gradbox — no batched
            // gradient is materialised and no reduction pass runs.
            const int64_t M = A->shape[A->rank - 2], K = A->shape[A->rank - 1], N = B->shape[B->rank - 1];
            BatchDesc none{};
            for (int d = 0; d < MAX_BATCH_RANK; ++d) none.shape[d] = 1;
            Epilogue ep;
            if (grad_b && K > 8 && bsum_fits(A->strides[A->rank - 1], A->strides[A->rank - 2], N, 1, K, N, g.batch_count * M, 1, ep)) { ep.bsum = grad_b; *bias_done = true; }
            if (int rc = gemm_dispatch(A->data + A->offset, A->strides[A->rank - 1], A->strides[A->rank - 2], dC, N, 1, grad_B,
                                       K, N, g.batch_count * M, none, 1, 1, ep)) return rc;
        } else if (same_batch(g, B, 2)) {
            // (one matrix: the weight gradient of a Linear layer under a 2-D input is this product, with dC as its right operand)
            const int64_t M = A->shape[A->rank - 2], K = A->shape[A->rank - 1], N = B->shape[B->rank - 1];
            Epilogue ep;
            if (grad_b && K > 8 && g.batch_count == 1 && bsum_fits(At.strides[At.rank - 2], At.strides[At.rank - 1], N, 1, K, N, M, 1, ep)) {
                ep.bsum = grad_b; *bias_done = true;
                BatchDesc none{};
                for (int d = 0; d < MAX_BATCH_RANK; ++d) none.shape[d] = 1;
                if (int rc = gemm_dispatch(At.data + At.offset, At.strides[At.rank - 2], At.strides[At.rank - 1], dC, N, 1, grad_B, K, N, M, none, 1, 1, ep)) return rc;
            } else if (int rc = matmul_views(&At, &dCv, grad_B, 1, "tenmo_hip_matmul_backward")) return rc;
        } else if (const int folded = folded_gradient(&At, &dCv, g, B, grad_B)) {
            if (folded < 0) return folded;
        } else {
            Geometry gg;
            if (int rc = resolve(TENMO_OP_MM, &At, &dCv, &gg, "tenmo_hip_matmul_backward")) return rc;
            float* full = nullptr;
            if (int rc = workspace2((size_t)product(gg.oshape, gg.orank) * sizeof(float), &full)) return rc;
            if (int rc = matmul_views(&At, &dCv, full, 0, "tenmo_hip_matmul_backward")) return rc;
            if (int rc = reduce_to_parent(full, gg, B, 2, grad_B)) return rc;
        }
    }
    return 0;
}

int tenmo_hip_matmul_backward(const tenmo_view* A, const tenmo_view* B, const float* dC,
                              float* grad_A, float* grad_B, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    Geometry g;
    if (int rc = resolve(TENMO_OP_MM, A, B, &g, "tenmo_hip_matmul_backward")) return rc;
    if (g.batch_count == 0) return 0;
    if (int rc = need(dC, product(g.oshape, g.orank) > 0 && (grad_A || grad_B), "tenmo_hip_matmul_backward", "upstream gradient")) return rc;
    if (int rc = matmul_backward_impl(A, B, dC, grad_A, grad_B, g)) return rc;
    return finish(sync);
}

int tenmo_hip_linear_backward(const tenmo_view* X, const tenmo_view* W, const float* dY,
                              float* grad_X, float* grad_W, float* grad_bias, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    const char* who = "tenmo_hip_linear_backward";
    Geometry g;
    if (int rc = resolve(TENMO_OP_MM, X, W, &g, who)) return rc;
    if (g.batch_count == 0) return 0;
    const int64_t total = product(g.oshape, g.orank);
    if (int rc = need(dY, total > 0 && (grad_X || grad_W || grad_bias), who, "upstream gradient")) return rc;
    bool bias_done = false;
    if (int rc = matmul_backward_impl(X, W, dY, grad_X, grad_W, g, grad_W ? grad_bias : nullptr, &bias_done)) return rc;
    if (grad_bias && !bias_done) {
        // sum_over_broadcasted_axes for the bias operand of Adder (tenmo/broadcast.mojo:66-88): dY [rows, N] summed over its rows, one streaming pass
        const int64_t N = g.oshape[g.orank - 1], rows = N > 0 ? total / N : 0;
        BatchDesc bd{};
        for (int d = 0; d < MAX_BATCH_RANK; ++d) bd.shape[d] = 1;
        if (int rc = matvec_dispatch(dY, 1, N, S.one, 0, grad_bias, N, rows, bd, 1, 1)) return rc;
    }
    return finish(sync);
}

static int outer_grad(const float* p, int64_t p_s, const int64_t* p_bstr, const float* q, int64_t q_s, const int64_t* q_bstr,
                      float* grad, int64_t I, int64_t J, const Geometry& g, const tenmo_view* parent) {
    OuterArgs o{};
    o.p = p; o.p_s = p_s; o.q = q; o.q_s = q_s; o.grad = grad; o.I = I; o.J = J;
    o.rank = g.batch_rank;
    const int own = parent->rank - 2;
    int64_t kept_total = 1, red_total = 1;
    for (int d = 0; d < g.batch_rank; ++d) {
        o.shape[d] = g.oshape[d];
        o.p_str[d] = p_bstr[d];
        o.q_str[d] = q_bstr[d];
        const int od = d - (g.batch_rank - own);
        o.kept[d] = (od >= 0 && parent->shape[od] > 1) ? 1 : 0;
        if (o.kept[d]) kept_total *= g.oshape[d]; else red_total *= g.oshape[d];
    }
    o.parent_batch = kept_total;
    o.reduced_total = red_total;
    const int64_t total = kept_total * I * J;
    if (total == 0) return 0;
    if (q_s == 1 && J % 4 == 0 && (uintptr_t)grad % 16 == 0) {
        const int64_t blocks = std::max<int64_t>(1, std::min<int64_t>((total / 4 + 1023) / 1024, (int64_t)S.cus * 16));
        hipLaunchKernelGGL(outer_add_vec_kernel, dim3((unsigned)blocks), dim3(256), 0, S.stream, o);
    } else {
        hipLaunchKernelGGL(outer_add_kernel, dim3((unsigned)std::min<int64_t>((total + 255) / 256, 65535)), dim3(256), 0, S.stream, o);
    }
    return 0;
}

int tenmo_hip_mv_backward(const tenmo_view* Mx, const tenmo_view* v, const float* dy,
                          float* grad_M, float* grad_v, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    Geometry g;
    if (int rc = resolve(TENMO_OP_MV, Mx, v, &g, "tenmo_hip_mv_backward")) return rc;
    if (g.batch_count == 0) return 0;
    if (int rc = need(dy, product(g.oshape, g.orank) > 0 && (grad_M || grad_v), "tenmo_hip_mv_backward", "upstream gradient")) return rc;
    const int64_t m = Mx->shape[Mx->rank - 2], k = Mx->shape[Mx->rank - 1];
    int64_t dy_bstr[MAX_BATCH_RANK] = {0}, v_bstr[MAX_BATCH_RANK] = {0}, m_bstr[MAX_BATCH_RANK] = {0};
    { int64_t acc = m; for (int d = g.batch_rank - 1; d >= 0; --d) { dy_bstr[d] = acc; acc *= g.oshape[d]; } }
    batch_strides_of(v, v->rank - 1, g.batch_rank, v_bstr);
    batch_strides_of(Mx, Mx->rank - 2, g.batch_rank, m_bstr);
    if (grad_M) // dM[i][j] += dy[i] * v[j]   (tenmo/matrixvector.mojo:87-139)
        if (int rc = outer_grad(dy, 1, dy_bstr, v->data + v->offset, v->strides[v->rank - 1], v_bstr, grad_M, m, k, g, Mx)) return rc;
    if (grad_v) { // dv = M^T . dy  (:162-196), reduced over the batches v broadcast
        // as a batched vector x matrix: dy[.., m] . M[.., m, k] -> [.., k]
        BatchDesc bd{};
        bd.rank = g.batch_rank;
        for (int d = 0; d < MAX_BATCH_RANK; ++d) {
            bd.shape[d] = d < g.batch_rank ? g.oshape[d] : 1;
            bd.a_str[d] = d < g.batch_rank ? m_bstr[d] : 0;  // matrix
            bd.b_str[d] = d < g.batch_rank ? dy_bstr[d] : 0; // vector
        }
        Geometry gg = g;
        gg.oshape[g.batch_rank] = k; gg.orank = g.batch_rank + 1;
        const bool direct = same_batch(g, v, 1);
        if (!direct && S.fold_reduce != 0 && all_broadcast(v, 1) && rows_fold(Mx, g)) {
            // v is shared by every batch and the matrices stack at a constant row pitch: the sum over batches of
            // M_b^T . dy_b is ONE product dy[batch*m] . M[batch*m, k], added straight into the gradbox
            BatchDesc none{};
            for (int d = 0; d < MAX_BATCH_RANK; ++d) none.shape[d] = 1;
            if (int rc = matvec_dispatch(Mx->data + Mx->offset, Mx->strides[Mx->rank - 1], Mx->strides[Mx->rank - 2], dy, 1, grad_v, k, g.batch_count * m, none, 1, 1)) return rc;
            return finish(sync);
        }
        float* target = grad_v;
        float* full = nullptr;
        if (!direct) {
            if (int rc = workspace2((size_t)g.batch_count * k * sizeof(float), &full)) return rc;
            target = full;
        }
        if (int rc = matvec_dispatch(Mx->data + Mx->offset, Mx->strides[Mx->rank - 1], Mx->strides[Mx->rank - 2], dy, 1, target, k, m, bd, g.batch_count, direct ? 1 : 0)) return rc;
        if (!direct) if (int rc = reduce_to_parent(full, gg, v, 1, grad_v)) return rc;
    }
    return finish(sync);
}

int tenmo_hip_vm_backward(const tenmo_view* v, const tenmo_view* Mx, const float* dy,
                          float* grad_v, float* grad_M, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    Geometry g;
    if (int rc = resolve(TENMO_OP_VM, v, Mx, &g, "tenmo_hip_vm_backward")) return rc;
    if (g.batch_count == 0) return 0;
    if (int rc = need(dy, product(g.oshape, g.orank) > 0 && (grad_v || grad_M), "tenmo_hip_vm_backward", "upstream gradient")) return rc;
    const int64_t k = Mx->shape[Mx->rank - 2], n = Mx->shape[Mx->rank - 1];
    int64_t dy_bstr[MAX_BATCH_RANK] = {0}, v_bstr[MAX_BATCH_RANK] = {0}, m_bstr[MAX_BATCH_RANK] = {0};
    { int64_t acc = n; for (int d = g.batch_rank - 1; d >= 0; --d) { dy_bstr[d] = acc; acc *= g.oshape[d]; } }
    batch_strides_of(v, v->rank - 1, g.batch_rank, v_bstr);
    batch_strides_of(Mx, Mx->rank - 2, g.batch_rank, m_bstr);
    if (grad_M) // dM[i][j] += v[i] * dy[j]   (tenmo/vectormatrix.mojo:145-201)
        if (int rc = outer_grad(v->data + v->offset, v->strides[v->rank - 1], v_bstr, dy, 1, dy_bstr, grad_M, k, n, g, Mx)) return rc;
    if (grad_v) { // dv[i] = sum_j dy[j] M[i][j]  (:65-100): a matrix x vector with M as is
        BatchDesc bd{};
        bd.rank = g.batch_rank;
        for (int d = 0; d < MAX_BATCH_RANK; ++d) {
            bd.shape[d] = d < g.batch_rank ? g.oshape[d] : 1;
            bd.a_str[d] = d < g.batch_rank ? m_bstr[d] : 0;
            bd.b_str[d] = d < g.batch_rank ? dy_bstr[d] : 0;
        }
        Geometry gg = g;
        gg.oshape[g.batch_rank] = k; gg.orank = g.batch_rank + 1;
        const bool direct = same_batch(g, v, 1);
        float* target = grad_v;
        float* full = nullptr;
        if (!direct) {
            if (int rc = workspace2((size_t)g.batch_count * k * sizeof(float), &full)) return rc;
            target = full;
        }
        if (int rc = matvec_dispatch(Mx->data + Mx->offset, Mx->strides[Mx->rank - 2], Mx->strides[Mx->rank - 1], dy, 1, target, k, n, bd, g.batch_count, direct ? 1 : 0)) return rc;
        if (!direct) if (int rc = reduce_to_parent(full, gg, v, 1, grad_v)) return rc;
    }
    return finish(sync);
}

// ---- CBLAS-compatible host-pointer entry point --------------------------------------------------

static int stage_buffer(int i, size_t bytes, float** out) {
    if (bytes > S.stage_bytes[i]) {
        if (S.stage[i]) { HIP_TRY(hipStreamSynchronize(S.stream)); HIP_TRY(hipFree(S.stage[i])); S.stage[i] = nullptr; S.stage_bytes[i] = 0; }
        HIP_TRY(hipMalloc(&S.stage[i], bytes));
        S.stage_bytes[i] = bytes;
    }
    *out = S.stage[i];
    return 0;
}

static int sgemm_impl(int order, int ta, int tb, int M, int N, int K, float alpha, const float* A, int lda,
                      const float* B, int ldb, float beta, float* C, int ldc) {
    if (!S.ready) { if (int rc = tenmo_hip_init(0)) return rc; }
    const bool row = (order == 101);
    if (!row && order != 102) return fail(TENMO_ERR_INVALID_ARGUMENT, "cblas_sgemm: order must be 101 (RowMajor) or 102 (ColMajor)");
    auto is_t = [](int t) { return t == 112 || t == 113; };
    if ((ta != 111 && !is_t(ta)) || (tb != 111 && !is_t(tb))) return fail(TENMO_ERR_INVALID_ARGUMENT, "cblas_sgemm: bad transpose flag");
    if (M < 0 || N < 0 || K < 0) return fail(TENMO_ERR_INVALID_SHAPE, "cblas_sgemm: negative dimension");
    if (M == 0 || N == 0) return 0;
    // stored extents of A and B in their own storage order
    const int a_r = row ? (is_t(ta) ? K : M) : (is_t(ta) ? M : K); // number of ld-strided lines of A
    const int a_c = row ? (is_t(ta) ? M : K) : (is_t(ta) ? K : M); // contiguous extent
    const int b_r = row ? (is_t(tb) ? N : K) : (is_t(tb) ? K : N);
    const int b_c = row ? (is_t(tb) ? K : N) : (is_t(tb) ? N : K);
    const int c_r = row ? M : N, c_c = row ? N : M;
    if (lda < std::max(1, a_c) || ldb < std::max(1, b_c) || ldc < std::max(1, c_c)) return fail(TENMO_ERR_INVALID_ARGUMENT, "cblas_sgemm: leading dimension too small");
    float *dA, *dB, *dC;
    if (int rc = stage_buffer(0, std::max<size_t>(1, (size_t)a_r * a_c) * sizeof(float), &dA)) return rc;
    if (int rc = stage_buffer(1, std::max<size_t>(1, (size_t)b_r * b_c) * sizeof(float), &dB)) return rc;
    if (int rc = stage_buffer(2, (size_t)M * N * sizeof(float), &dC)) return rc;
    if (K > 0) {
        HIP_TRY(hipMemcpy2DAsync(dA, (size_t)a_c * 4, A, (size_t)lda * 4, (size_t)a_c * 4, a_r, hipMemcpyHostToDevice, S.stream));
        HIP_TRY(hipMemcpy2DAsync(dB, (size_t)b_c * 4, B, (size_t)ldb * 4, (size_t)b_c * 4, b_r, hipMemcpyHostToDevice, S.stream));
    }
    // logical (M x K) and (K x N) operands as strided views of the staged dense copies
    int64_t a_rs, a_cs, b_rs, b_cs;
    if (row) {
        a_rs = is_t(ta) ? 1 : a_c; a_cs = is_t(ta) ? a_c : 1;
        b_rs = is_t(tb) ? 1 : b_c; b_cs = is_t(tb) ? b_c : 1;
    } else { // column-major storage: element (i,j) of the stored matrix at i + j*ld
        a_rs = is_t(ta) ? a_c : 1; a_cs = is_t(ta) ? 1 : a_c;
        b_rs = is_t(tb) ? b_c : 1; b_cs = is_t(tb) ? 1 : b_c;
    }
    BatchDesc bd{};
    for (int d = 0; d < MAX_BATCH_RANK; ++d) bd.shape[d] = 1;
    int rc;
    if (row) rc = gemm_dispatch(dA, a_rs, a_cs, dB, b_rs, b_cs, dC, M, N, K, bd, 1, 0);
    else     rc = gemm_dispatch(dB, b_cs, b_rs, dA, a_cs, a_rs, dC, N, M, K, bd, 1, 0); // C^T = B^T . A^T, dense [N][M] == column-major C
    if (rc) return rc;
    HIP_TRY(hipGetLastError());
    std::vector<float> host((size_t)M * N);
    HIP_TRY(hipMemcpyAsync(host.data(), dC, (size_t)M * N * sizeof(float), hipMemcpyDeviceToHost, S.stream));
    HIP_TRY(hipStreamSynchronize(S.stream));
    for (int r = 0; r < c_r; ++r) {
        float* crow = C + (size_t)r * ldc;
        const float* hrow = host.data() + (size_t)r * c_c;
        if (beta == 0.f) for (int c = 0; c < c_c; ++c) crow[c] = alpha * hrow[c];
        else for (int c = 0; c < c_c; ++c) crow[c] = alpha * hrow[c] + beta * crow[c];
    }
    return 0;
}

void cblas_sgemm(int order, int ta, int tb, int M, int N, int K, float alpha, const float* A, int lda,
                 const float* B, int ldb, float beta, float* C, int ldc) {
    // the CBLAS prototype has no error channel; failures are left in tenmo_hip_last_error() and
    // reported on stderr, as a BLAS would do through xerbla
    if (int rc = sgemm_impl(order, ta, tb, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc))
        fprintf(stderr, "libtenmo_hip cblas_sgemm: error %d: %s\n", rc, t_err.c_str());
}

// ---- MLP training-step harness --------------------------------------------------------------------

struct tenmo_mlp {
    int L = 0;
    std::vector<int64_t> dims;
    int64_t max_batch = 0;
    std::vector<float*> W, b, dW, db, act, grad; // act[l]: output of layer l ([B, dims[l+1]]); grad[l]: its gradient
    float* row_loss = nullptr;
    // captured training step (tenmo_hip_mlp_step_graph): fixed input staging + the executable graph
    float* x_stage = nullptr;
    int32_t* y_stage = nullptr;
    hipGraphExec_t exec = nullptr;
    int64_t g_batch = -1;
    float g_lr = 0.f;
    float* g_loss = nullptr;
    float* g_ws = nullptr;      // library scratch pointer the captured kernels hold
    int g_fused = 0;            // mlp_fused_tail level the capture was made at
};

static unsigned grid_for(int64_t n) { return (unsigned)std::max<int64_t>(1, std::min<int64_t>((n + 255) / 256, 4096)); }

tenmo_mlp* tenmo_hip_mlp_create(int32_t L, const int64_t* dims, const float* const* Wh, const float* const* bh, int64_t max_batch) {
    if (ensure_ready()) return nullptr;
    if (L < 1 || !dims || !Wh || !bh || max_batch < 1) { fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mlp_create: bad arguments"); return nullptr; }
    auto* m = new tenmo_mlp();
    m->L = L; m->dims.assign(dims, dims + L + 1); m->max_batch = max_batch;
    m->W.assign(L, nullptr); m->b.assign(L, nullptr); m->dW.assign(L, nullptr); m->db.assign(L, nullptr);
    m->act.assign(L, nullptr); m->grad.assign(L, nullptr);
    bool ok = true;
    for (int l = 0; l < L && ok; ++l) {
        const size_t wn = (size_t)dims[l] * dims[l + 1], bn = (size_t)dims[l + 1], an = (size_t)max_batch * dims[l + 1];
        ok = ok && hipMalloc(&m->W[l], wn * 4) == hipSuccess && hipMalloc(&m->dW[l], wn * 4) == hipSuccess;
        ok = ok && hipMalloc(&m->b[l], bn * 4) == hipSuccess && hipMalloc(&m->db[l], bn * 4) == hipSuccess;
        ok = ok && hipMalloc(&m->act[l], an * 4) == hipSuccess && hipMalloc(&m->grad[l], an * 4) == hipSuccess;
        ok = ok && hipMemcpy(m->W[l], Wh[l], wn * 4, hipMemcpyHostToDevice) == hipSuccess;
        ok = ok && hipMemcpy(m->b[l], bh[l], bn * 4, hipMemcpyHostToDevice) == hipSuccess;
    }
    ok = ok && hipMalloc(&m->row_loss, (size_t)max_batch * 4) == hipSuccess;
    ok = ok && hipMalloc(&m->x_stage, (size_t)max_batch * dims[0] * 4) == hipSuccess;
    ok = ok && hipMalloc(&m->y_stage, (size_t)max_batch * 4) == hipSuccess;
    if (!ok) { fail(TENMO_ERR_HIP, "tenmo_hip_mlp_create: device allocation or upload failed"); tenmo_hip_mlp_destroy(m); return nullptr; }
    return m;
}

void tenmo_hip_mlp_destroy(tenmo_mlp* m) {
    if (!m) return;
    if (S.ready) (void)hipStreamSynchronize(S.stream);
    for (auto* v : {&m->W, &m->b, &m->dW, &m->db, &m->act, &m->grad})
        for (float* p : *v) if (p) (void)hipFree(p);
    if (m->row_loss) (void)hipFree(m->row_loss);
    if (m->x_stage) (void)hipFree(m->x_stage);
    if (m->y_stage) (void)hipFree(m->y_stage);
    if (m->exec) (void)hipGraphExecDestroy(m->exec);
    delete m;
}

// the first `layers` layers (all of them by default)
static int mlp_forward(tenmo_mlp* m, const float* x, int64_t B, int layers = -1) {
    if (layers < 0) layers = m->L;
    BatchDesc bd{};
    for (int d = 0; d < MAX_BATCH_RANK; ++d) bd.shape[d] = 1;
    const float* in = x;
    for (int l = 0; l < layers; ++l) {
        const int64_t I = m->dims[l], O = m->dims[l + 1];
        Epilogue ep; // bias add and ReLU happen in the GEMM store
        ep.bias = m->b[l]; ep.relu = l + 1 < m->L ? 1 : 0;
        // a small batch against a long input: one launch whose workgroups cut K among their own wavefronts, instead of K
        // slices over many workgroups and a launch that adds them (mlp_fused_tail knob, level 3)
        if (S.mlp_fused_tail >= 3 && l == 0 && B <= 128 && O <= 256 && I >= 256 && I <= (1 << 20)) {
            MlpFwdArgs f{};
            f.x = in; f.W = m->W[0]; f.b = m->b[0]; f.h = m->act[0];
            f.B = (int32_t)B; f.I = (int32_t)I; f.O = (int32_t)O; f.relu = ep.relu;
            hipLaunchKernelGGL(mlp_first_forward_kernel, dim3((unsigned)((O + 31) / 32), (unsigned)((B + 31) / 32)), dim3(MLP_FWD_THREADS), 0, S.stream, f);
            in = m->act[l];
            continue;
        }
        if (int rc = gemm_dispatch(in, I, 1, m->W[l], O, 1, m->act[l], B, O, I, bd, 1, 0, ep)) return rc;
        in = m->act[l];
    }
    return 0;
}

int tenmo_hip_mlp_forward(tenmo_mlp* m, const float* x, int64_t B, float* logits_out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (!m || B < 1 || B > m->max_batch) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mlp_forward: batch outside 1..max_batch");
    if (!x || !logits_out) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mlp_forward: null pointer");
    if (int rc = mlp_forward(m, x, B)) return rc;
    HIP_TRY(hipMemcpyAsync(logits_out, m->act[m->L - 1], (size_t)B * m->dims[m->L] * 4, hipMemcpyDeviceToDevice, S.stream));
    return finish(sync);
}

// enqueues every kernel of one training step on the library stream
static int mlp_step_enqueue(tenmo_mlp* m, const float* x, const int32_t* y, int64_t B, float lr, float* loss_out) {
    const int L = m->L;
    const int64_t C = m->dims[L];
    // The last two layers, the loss, their backward and their update as one launch (mlp_tail_kernel) when they fit one
    // workgroup's LDS; the layers below run as usual on either side of it.
    const bool fused_tail = S.mlp_fused_tail > 0 && L >= 3 && B <= MLP_TAIL_MAX_B && m->dims[L - 2] <= MLP_TAIL_MAX_D0 &&
                            m->dims[L - 1] <= MLP_TAIL_MAX_D1 && C <= MLP_TAIL_MAX_C;
    const int top = fused_tail ? L - 2 : L; // layers [0, top) run op by op
    if (int rc = mlp_forward(m, x, B, top)) return rc;
    if (fused_tail) {
        MlpTailArgs t{};
        t.h0 = m->act[L - 3]; t.y = y;
        t.W1 = m->W[L - 2]; t.b1 = m->b[L - 2]; t.W2 = m->W[L - 1]; t.b2 = m->b[L - 1];
        t.dW1 = m->dW[L - 2]; t.db1 = m->db[L - 2]; t.dW2 = m->dW[L - 1]; t.db2 = m->db[L - 1];
        t.h1 = m->act[L - 2]; t.logits = m->act[L - 1];
        t.g0 = m->grad[L - 3]; t.db0 = m->db[L - 3];
        t.row_loss = m->row_loss; t.loss_out = loss_out; t.lr = lr;
        t.B = (int32_t)B; t.D0 = (int32_t)m->dims[L - 2]; t.D1 = (int32_t)m->dims[L - 1]; t.C = (int32_t)C;
        hipLaunchKernelGGL(mlp_tail_kernel, dim3(1), dim3(MLP_TAIL_THREADS), 0, S.stream, t);
    }
    const bool one_block = B <= 256; // loss, its gradient, the mean and the last bias gradient in one launch
    if (fused_tail) {
        // done by the tail launch
    } else if (one_block) {
        hipLaunchKernelGGL(cross_entropy_kernel, dim3(1), dim3((unsigned)((B + 63) / 64 * 64)), 0, S.stream, m->act[L - 1], y, B, C, m->grad[L - 1], m->row_loss, loss_out, m->db[L - 1]);
    } else {
        hipLaunchKernelGGL(cross_entropy_kernel, dim3((unsigned)((B + 63) / 64)), dim3(64), 0, S.stream, m->act[L - 1], y, B, C, m->grad[L - 1], m->row_loss, (float*)nullptr, (float*)nullptr);
        hipLaunchKernelGGL(ordered_mean_kernel, dim3(1), dim3(64), 0, S.stream, m->row_loss, B, loss_out);
    }
    BatchDesc bd{};
    for (int d = 0; d < MAX_BATCH_RANK; ++d) bd.shape[d] = 1;
    bool first_done = false; // layer 0 updated by its own fused launch
    for (int l = top - 1; l >= 0; --l) {
        const int64_t I = m->dims[l], O = m->dims[l + 1];
        const float* in = l == 0 ? x : m->act[l - 1];
        const float* gl = m->grad[l];
        const bool from_gemm = B <= 128; // hidden layers: summed in the store of the GEMM that produced this gradient (below)
        // the first layer's weight gradient and update as one launch beside the fused tail (the two together leave
        // the step with the first layer's forward, the tail and this)
        const bool first_fused = S.mlp_fused_tail >= 2 && l == 0 && B <= MLP_TAIL_MAX_B && O <= MLP_TAIL_MAX_D0 && I <= 0x7fffffffLL / MLP_TAIL_MAX_D0;
        if (fused_tail && l == top - 1) {
            // done by the tail launch
        } else if (one_block && l == L - 1) {
            // done by the cross-entropy launch
        } else if (from_gemm && l < L - 1) {
            // done by the dX product of layer l+1
        } else if (B * O >= (int64_t)1 << 18) { // large: stream the gradient once at HBM rate
            if (int rc = matvec_dispatch(gl, 1, O, S.one, 0, m->db[l], O, B, bd, 1, 0)) return rc;
        } else {
            hipLaunchKernelGGL(column_sum_kernel, dim3((unsigned)((O + 63) / 64)), dim3(64), 0, S.stream, gl, B, O, m->db[l]);
        }
        // dW = in^T(view) . g        (tenmo/matmul.mojo:46-48)
        // dX = g . W^T(view)         (tenmo/matmul.mojo:36-38); the network input needs no gradient (:34)
        Epilogue ep; // ReLU backward in the GEMM store: zero where the forward activation was not positive
        if (l > 0) {
            ep.mask = m->act[l - 1];
            if (from_gemm) ep.colsum = m->db[l - 1]; // bias gradient of layer l-1 = column sums of its (masked) gradient
        }
        // both consume the same upstream gradient and are independent: one launch for the two when they are small
        if (first_fused) {
            MlpFirstArgs f{};
            f.x = in; f.g = gl; f.db = m->db[0]; f.W = m->W[0]; f.b = m->b[0]; f.dW = m->dW[0];
            f.lr = lr; f.B = (int32_t)B; f.I = (int32_t)I; f.O = (int32_t)O;
            hipLaunchKernelGGL(mlp_first_layer_kernel, dim3((unsigned)((I + MLP_FIRST_ROWS - 1) / MLP_FIRST_ROWS)), dim3(MLP_TAIL_THREADS), 0, S.stream, f);
            first_done = true;
            continue;
        }
        int paired = 1;
        if (l > 0) paired = gemm_pair_dispatch(in, 1, I, gl, O, 1, m->dW[l], I, O, B, gl, O, 1, m->W[l], 1, O, m->grad[l - 1], B, I, O, ep);
        if (paired < 0) return paired;
        if (paired != 0) {
            if (int rc = gemm_dispatch(in, 1, I, gl, O, 1, m->dW[l], I, O, B, bd, 1, 0)) return rc;
            if (l > 0)
                if (int rc = gemm_dispatch(gl, O, 1, m->W[l], 1, O, m->grad[l - 1], B, I, O, bd, 1, 0, ep)) return rc;
        }
    }
    // every parameter tensor (below the fused tail, which updates its own) in one launch
    for (int l0 = first_done ? 1 : 0; l0 < top; l0 += SGD_MAX_TENSORS / 2) {
        SgdArgs sa{};
        int64_t largest = 0;
        for (int l = l0; l < top && sa.count + 2 <= SGD_MAX_TENSORS; ++l) {
            const int64_t wn = m->dims[l] * m->dims[l + 1], bn = m->dims[l + 1];
            sa.p[sa.count] = m->W[l]; sa.g[sa.count] = m->dW[l]; sa.n[sa.count] = wn; ++sa.count;
            sa.p[sa.count] = m->b[l]; sa.g[sa.count] = m->db[l]; sa.n[sa.count] = bn; ++sa.count;
            largest = std::max(largest, wn);
        }
        hipLaunchKernelGGL(sgd_multi_kernel, dim3(grid_for(largest), (unsigned)sa.count), dim3(256), 0, S.stream, sa, lr);
    }
    return 0;
}

int tenmo_hip_mlp_step(tenmo_mlp* m, const float* x, const int32_t* y, int64_t B, float lr, float* loss_out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (!m || B < 1 || B > m->max_batch) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mlp_step: batch outside 1..max_batch");
    if (!x || !y || !loss_out) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mlp_step: null pointer");
    if (int rc = mlp_step_enqueue(m, x, y, B, lr, loss_out)) return rc;
    return finish(sync);
}

int tenmo_hip_mlp_step_graph(tenmo_mlp* m, const float* x, const int32_t* y, int64_t B, float lr, float* loss_out, int32_t sync) {
    if (int rc = ensure_ready()) return rc;
    if (!m || B < 1 || B > m->max_batch) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mlp_step_graph: batch outside 1..max_batch");
    if (!x || !y || !loss_out) return fail(TENMO_ERR_INVALID_ARGUMENT, "tenmo_hip_mlp_step_graph: null pointer");
    if (S.stream == nullptr) return fail(TENMO_ERR_UNSUPPORTED, "tenmo_hip_mlp_step_graph: cannot capture on the null stream");
    // the captured kernels read fixed staging buffers; this step's inputs are copied in eagerly
    HIP_TRY(hipMemcpyAsync(m->x_stage, x, (size_t)B * m->dims[0] * 4, hipMemcpyDeviceToDevice, S.stream));
    HIP_TRY(hipMemcpyAsync(m->y_stage, y, (size_t)B * 4, hipMemcpyDeviceToDevice, S.stream));
    float* ws;
    if (int rc = workspace(1, &ws)) return rc; // scratch must exist before capture: no allocation may happen inside it
    // the captured kernels hold the scratch pointer: a capture made before the scratch buffer grew is stale
    for (int attempt = 0; !m->exec || m->g_batch != B || m->g_lr != lr || m->g_loss != loss_out || m->g_ws != ws || m->g_fused != S.mlp_fused_tail; ++attempt) {
        if (m->exec) { HIP_TRY(hipStreamSynchronize(S.stream)); HIP_TRY(hipGraphExecDestroy(m->exec)); m->exec = nullptr; }
        HIP_TRY(hipStreamBeginCapture(S.stream, hipStreamCaptureModeThreadLocal));
        S.capturing = true; S.ws_wanted = 0;
        const int rc = mlp_step_enqueue(m, m->x_stage, m->y_stage, B, lr, loss_out);
        S.capturing = false;
        hipGraph_t graph = nullptr;
        const hipError_t e = hipStreamEndCapture(S.stream, &graph);
        if (rc) {
            if (graph) (void)hipGraphDestroy(graph);
            // a kernel selection wanted more scratch than there is: grow it out here, where allocating is allowed, and capture again
            if (S.ws_wanted > S.ws_bytes && attempt < 4) {
                if (int rc2 = workspace(S.ws_wanted, &ws)) return rc2;
                continue;
            }
            return rc;
        }
        if (e != hipSuccess) return fail(TENMO_ERR_HIP, "hipStreamEndCapture failed: %s", hipGetErrorString(e));
        const hipError_t ei = hipGraphInstantiate(&m->exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (ei != hipSuccess) { m->exec = nullptr; return fail(TENMO_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(ei)); }
        m->g_batch = B; m->g_lr = lr; m->g_loss = loss_out; m->g_ws = ws; m->g_fused = S.mlp_fused_tail;
    }
    HIP_TRY(hipGraphLaunch(m->exec, S.stream));
    return finish(sync);
}

int tenmo_hip_mlp_get_params(tenmo_mlp* m, int32_t l, float* Wh, float* bh) {
    if (int rc = ensure_ready()) return rc;
    if (!m || l < 0 || l >= m->L) return fail(TENMO_ERR_INVALID_ARGUMENT, "layer out of range");
    HIP_TRY(hipStreamSynchronize(S.stream));
    if (Wh) HIP_TRY(hipMemcpy(Wh, m->W[l], (size_t)m->dims[l] * m->dims[l + 1] * 4, hipMemcpyDeviceToHost));
    if (bh) HIP_TRY(hipMemcpy(bh, m->b[l], (size_t)m->dims[l + 1] * 4, hipMemcpyDeviceToHost));
    return 0;
}

int tenmo_hip_mlp_get_grads(tenmo_mlp* m, int32_t l, float* Wh, float* bh) {
    if (int rc = ensure_ready()) return rc;
    if (!m || l < 0 || l >= m->L) return fail(TENMO_ERR_INVALID_ARGUMENT, "layer out of range");
    HIP_TRY(hipStreamSynchronize(S.stream));
    if (Wh) HIP_TRY(hipMemcpy(Wh, m->dW[l], (size_t)m->dims[l] * m->dims[l + 1] * 4, hipMemcpyDeviceToHost));
    if (bh) HIP_TRY(hipMemcpy(bh, m->db[l], (size_t)m->dims[l + 1] * 4, hipMemcpyDeviceToHost));
    return 0;
}

} // extern "C"
