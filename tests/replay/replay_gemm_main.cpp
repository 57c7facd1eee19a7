// Address check of whole GEMM launches on the CPU: runs tenmo_hip_gemm_f32 of the CPU build of the library (see
// hip/hip_runtime.h in this directory) on operands that are heap blocks of exactly the operands' sizes.  Built with
// -fsanitize=address, an access of any kernel one byte outside an operand ends the run with the sanitizer's report;
// otherwise the result is compared with a float64 product.  Test infrastructure.
//
//   replay_gemm [late] CASE...      CASE = M,N,K,a_layout,b_layout,batch,b_shared,accumulate[,knob=value...]
//     a_layout / b_layout: n (row-major as given), t (a transposed view of the transposed storage) or g (row-major
//     storage of twice the width of which every second element is used: no unit stride, the element-wise loader)
//     batch: number of matrices (0: no batch dimension); b_shared: 1 = every batch uses the same B
//     a case may carry check=0: do not compute the float64 product (large shapes: the addresses are the point)
//   CASE = bwd:M,N,K,a_layout,b_layout,a_batch,b_batch[,knob=value...]   tenmo_hip_matmul_backward of A[a_batch, M, K] . B[b_batch, K, N]
//     (a batch of 0: no batch dimension; 1: one that broadcasts): both gradients against float64, accumulated onto a start value
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../../include/tenmo_hip.h"

extern "C" void replay_register(const void* p, size_t bytes);
extern "C" void replay_set_late_loads(int on);

static uint32_t g_rng = 12345;
static float next_float() {
    g_rng = g_rng * 1664525u + 1013904223u;
    return (float)((int32_t)(g_rng >> 8) % 2001 - 1000) / 1000.0f;
}

// relative Frobenius distance of C from the float64 product (not instrumented: it only reads what it is given)
__attribute__((no_sanitize("address"))) static double reference_error(const float* A, const float* B, const float* Cm, const float* C0, int64_t nb, bool b_shared,
                                                                      int64_t M, int64_t N, int64_t K, int64_t a_mat, int64_t b_mat, int64_t a_rs, int64_t a_cs,
                                                                      int64_t b_rs, int64_t b_cs) {
    double num = 0.0, den = 0.0;
    std::vector<double> row((size_t)N);
    for (int64_t b = 0; b < nb; ++b) {
        const float* Ab = A + b * a_mat;
        const float* Bb = B + (b_shared ? 0 : b * b_mat);
        for (int64_t m = 0; m < M; ++m) {
            for (int64_t n = 0; n < N; ++n) row[(size_t)n] = C0 ? (double)C0[(size_t)((b * M + m) * N + n)] : 0.0;
            for (int64_t k = 0; k < K; ++k) {
                const double a = (double)Ab[m * a_rs + k * a_cs];
                const float* bk = Bb + k * b_rs;
                for (int64_t n = 0; n < N; ++n) row[(size_t)n] += a * (double)bk[n * b_cs];
            }
            for (int64_t n = 0; n < N; ++n) {
                const double d = (double)Cm[(b * M + m) * N + n] - row[(size_t)n];
                num += d * d;
                den += row[(size_t)n] * row[(size_t)n];
            }
        }
    }
    return std::sqrt(num / (den > 0 ? den : 1.0));
}

static int run_case(const std::string& spec) {
    std::vector<std::string> f;
    size_t pos = 0;
    while (pos <= spec.size()) {
        const size_t c = spec.find(',', pos);
        f.push_back(spec.substr(pos, c == std::string::npos ? std::string::npos : c - pos));
        if (c == std::string::npos) break;
        pos = c + 1;
    }
    if (f.size() < 8) { fprintf(stderr, "bad case %s\n", spec.c_str()); return 2; }
    const int64_t M = atoll(f[0].c_str()), N = atoll(f[1].c_str()), K = atoll(f[2].c_str());
    const bool ta = f[3] == "t", tb = f[4] == "t", ga = f[3] == "g", gb = f[4] == "g";
    const int64_t batch = atoll(f[5].c_str());
    const bool b_shared = atoi(f[6].c_str()) != 0;
    const int accumulate = atoi(f[7].c_str());
    bool check = true;
    std::vector<std::pair<std::string, int>> knobs;
    for (size_t i = 8; i < f.size(); ++i) {
        const size_t eq = f[i].find('=');
        if (eq == std::string::npos) continue;
        const std::string name = f[i].substr(0, eq);
        const int value = atoi(f[i].c_str() + eq + 1);
        if (name == "check") check = value != 0;
        else knobs.push_back({name, value});
    }
    const int64_t nb = batch > 0 ? batch : 1, nbb = b_shared ? 1 : nb;
    const int64_t a_mat = M * K * (ga ? 2 : 1), b_mat = K * N * (gb ? 2 : 1);
    const size_t a_n = (size_t)(nb * a_mat), b_n = (size_t)(nbb * b_mat), c_n = (size_t)(nb * M * N);
    // exactly-sized blocks: the sanitizer's red zones start at the operands' last byte
    float* A = (float*)malloc(a_n * 4 ? a_n * 4 : 1);
    float* B = (float*)malloc(b_n * 4 ? b_n * 4 : 1);
    float* Cm = (float*)malloc(c_n * 4 ? c_n * 4 : 1);
    std::vector<float> C0;
    for (size_t i = 0; i < a_n; ++i) A[i] = next_float();
    for (size_t i = 0; i < b_n; ++i) B[i] = next_float();
    for (size_t i = 0; i < c_n; ++i) Cm[i] = next_float();
    if (check && accumulate) C0.assign(Cm, Cm + c_n);
    replay_register(A, a_n * 4); replay_register(B, b_n * 4); replay_register(Cm, c_n * 4);
    // element (m, k) of A: storage [M][K] (n) or [K][M] (t); element (k, n) of B: storage [K][N] (n) or [N][K] (t)
    const int64_t a_rs = ga ? 2 * K : ta ? 1 : K, a_cs = ga ? 2 : ta ? M : 1, b_rs = gb ? 2 * N : tb ? 1 : N, b_cs = gb ? 2 : tb ? K : 1;
    const int64_t bshape[1] = {nb}, astr[1] = {a_mat}, bstr[1] = {b_shared ? 0 : b_mat};
    for (auto& kv : knobs) tenmo_hip_set_tuning(kv.first.c_str(), kv.second);
    const int rc = tenmo_hip_gemm_f32(A, 0, a_rs, a_cs, B, 0, b_rs, b_cs, Cm, M, N, K, batch > 0 ? 1 : 0, bshape, astr, bstr, accumulate, 1);
    for (auto& kv : knobs) tenmo_hip_set_tuning(kv.first.c_str(), -1);
    int bad = 0;
    if (rc != 0) { fprintf(stderr, "%s: error %d: %s\n", spec.c_str(), rc, tenmo_hip_last_error()); bad = 1; }
    double err = -1.0;
    if (rc == 0 && check) {
        err = reference_error(A, B, Cm, accumulate ? C0.data() : nullptr, nb, b_shared, M, N, K, a_mat, b_mat, a_rs, a_cs, b_rs, b_cs);
        if (!(err <= 2e-6)) bad = 1;
    }
    printf("%s: rc %d, relative error %.3g%s\n", spec.c_str(), rc, err, bad ? "  <-- FAILED" : "");
    fflush(stdout);
    replay_register(A, 0); replay_register(B, 0); replay_register(Cm, 0);
    free(A); free(B); free(Cm);
    return bad;
}

static tenmo_view view_of(const float* p, int64_t batch, int64_t rows, int64_t cols, bool transposed) {
    tenmo_view v;
    memset(&v, 0, sizeof(v));
    v.data = p;
    int r = 0;
    if (batch > 0) { v.shape[r] = batch; v.strides[r] = rows * cols; ++r; }
    v.shape[r] = rows; v.strides[r] = transposed ? 1 : cols; ++r;
    v.shape[r] = cols; v.strides[r] = transposed ? rows : 1; ++r;
    v.rank = r;
    return v;
}

__attribute__((no_sanitize("address"))) static double gradient_error(const float* got, const std::vector<double>& want) {
    double num = 0.0, den = 0.0;
    for (size_t i = 0; i < want.size(); ++i) { const double d = (double)got[i] - want[i]; num += d * d; den += want[i] * want[i]; }
    return std::sqrt(num / (den > 0 ? den : 1.0));
}

static int run_backward_case(const std::string& spec) {
    std::vector<std::string> f;
    size_t pos = 4;
    while (pos <= spec.size()) {
        const size_t c = spec.find(',', pos);
        f.push_back(spec.substr(pos, c == std::string::npos ? std::string::npos : c - pos));
        if (c == std::string::npos) break;
        pos = c + 1;
    }
    if (f.size() < 7) { fprintf(stderr, "bad case %s\n", spec.c_str()); return 2; }
    const int64_t M = atoll(f[0].c_str()), N = atoll(f[1].c_str()), K = atoll(f[2].c_str());
    const bool ta = f[3] == "t", tb = f[4] == "t";
    const int64_t ba = atoll(f[5].c_str()), bb = atoll(f[6].c_str());
    std::vector<std::pair<std::string, int>> knobs;
    for (size_t i = 7; i < f.size(); ++i) {
        const size_t eq = f[i].find('=');
        if (eq != std::string::npos) knobs.push_back({f[i].substr(0, eq), atoi(f[i].c_str() + eq + 1)});
    }
    const int64_t na = ba > 0 ? ba : 1, nb = bb > 0 ? bb : 1, nc = na > nb ? na : nb;
    const size_t a_n = (size_t)(na * M * K), b_n = (size_t)(nb * K * N), c_n = (size_t)(nc * M * N);
    float* A = (float*)malloc(a_n * 4); float* B = (float*)malloc(b_n * 4); float* dC = (float*)malloc(c_n * 4);
    float* gA = (float*)malloc(a_n * 4); float* gB = (float*)malloc(b_n * 4);
    for (size_t i = 0; i < a_n; ++i) { A[i] = next_float(); gA[i] = next_float(); }
    for (size_t i = 0; i < b_n; ++i) { B[i] = next_float(); gB[i] = next_float(); }
    for (size_t i = 0; i < c_n; ++i) dC[i] = next_float();
    // storage: A[b] is [M][K] (n) or [K][M] (t); the gradients are dense at the VIEW's shape [.., M, K] / [.., K, N]
    const int64_t a_rs = ta ? 1 : K, a_cs = ta ? M : 1, b_rs = tb ? 1 : N, b_cs = tb ? K : 1;
    std::vector<double> wantA(a_n), wantB(b_n);
    for (size_t i = 0; i < a_n; ++i) wantA[i] = gA[i];
    for (size_t i = 0; i < b_n; ++i) wantB[i] = gB[i];
    for (int64_t c = 0; c < nc; ++c) {
        const int64_t ia = na > 1 ? c : 0, ib = nb > 1 ? c : 0;
        const float* Ab = A + ia * M * K; const float* Bb = B + ib * K * N; const float* Gb = dC + c * M * N;
        for (int64_t m = 0; m < M; ++m)
            for (int64_t k = 0; k < K; ++k) {
                double s = 0.0;
                for (int64_t n = 0; n < N; ++n) s += (double)Gb[m * N + n] * (double)Bb[k * b_rs + n * b_cs];
                wantA[(size_t)(ia * M * K + m * K + k)] += s;
            }
        for (int64_t k = 0; k < K; ++k)
            for (int64_t n = 0; n < N; ++n) {
                double s = 0.0;
                for (int64_t m = 0; m < M; ++m) s += (double)Ab[m * a_rs + k * a_cs] * (double)Gb[m * N + n];
                wantB[(size_t)(ib * K * N + k * N + n)] += s;
            }
    }
    replay_register(A, a_n * 4); replay_register(B, b_n * 4); replay_register(dC, c_n * 4); replay_register(gA, a_n * 4); replay_register(gB, b_n * 4);
    tenmo_view va = view_of(A, ba, M, K, ta), vb = view_of(B, bb, K, N, tb);
    for (auto& kv : knobs) tenmo_hip_set_tuning(kv.first.c_str(), kv.second);
    const int rc = tenmo_hip_matmul_backward(&va, &vb, dC, gA, gB, 1);
    for (auto& kv : knobs) tenmo_hip_set_tuning(kv.first.c_str(), -1);
    int bad = 0;
    double ea = -1, eb = -1;
    if (rc != 0) { fprintf(stderr, "%s: error %d: %s\n", spec.c_str(), rc, tenmo_hip_last_error()); bad = 1; }
    else { ea = gradient_error(gA, wantA); eb = gradient_error(gB, wantB); if (!(ea <= 2e-6 && eb <= 2e-6)) bad = 1; }
    printf("%s: rc %d, relative error %.3g / %.3g%s\n", spec.c_str(), rc, ea, eb, bad ? "  <-- FAILED" : "");
    fflush(stdout);
    replay_register(A, 0); replay_register(B, 0); replay_register(dC, 0); replay_register(gA, 0); replay_register(gB, 0);
    free(A); free(B); free(dC); free(gA); free(gB);
    return bad;
}

int main(int argc, char** argv) {
    if (tenmo_hip_init(0) != 0) { fprintf(stderr, "init: %s\n", tenmo_hip_last_error()); return 2; }
    int bad = 0;
    for (int i = 1; i < argc; ++i) {
        if (!strcmp(argv[i], "late")) { replay_set_late_loads(1); continue; }
        if (!strcmp(argv[i], "early")) { replay_set_late_loads(0); continue; }
        bad |= strncmp(argv[i], "bwd:", 4) == 0 ? run_backward_case(argv[i]) : run_case(argv[i]);
    }
    tenmo_hip_shutdown();
    return bad;
}
