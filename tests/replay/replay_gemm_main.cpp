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
//   CASE = mv:m,k,layout,batch,pad,accumulate   out[m] = Mx[m,k] . v[k]; layout n (rows of k, pitch k + pad) or t (a transposed view of [k][m + pad])
//   CASE = vm:k,n,layout,batch,pad,accumulate[,entry=noalloc]   out[n] = v[k] . Mx[k,n]; the matrix shared by every batch when batch < 0
//   CASE = ce:M,C,target_is_int64,label_smoothing_percent[,unaligned]    cross-entropy forward (all outputs) and backward (mean), addresses only
//     (unaligned 1 / 2 / 3: the softmax, also the gradient, also the logits begin one float into their blocks)
//   CASE = conv:N,C_in,H_pad,W_pad,C_out,KH,KW,stride,dilation    convolution forward and backward (all three gradients), addresses only
//   CASE = mlp:batch,d0,d1,d2,d3,fused    two training steps of a 3-layer MLP (tenmo_hip_mlp_step), addresses only
//   CASE = misc:n      dot, column sum ([n/64+1, 64.. ] shapes derived from n), SGD with and without momentum, addresses only
//   CASE = vbw:m,k,matrix_batch,vector_batch,generic    matrix . vector and vector . matrix through the view-level entry points, each with its
//     backward (outer-product and vector gradients), addresses only
//   CASE = bwd:M,N,K,a_layout,b_layout,a_batch,b_batch[,knob=value...]   tenmo_hip_matmul_backward of A[a_batch, M, K] . B[b_batch, K, N]
//     (a batch of 0: no batch dimension; 1: one that broadcasts; skip=1: A's matrices lie two matrices apart): both gradients against float64,
//     accumulated onto a start value
//   CASE = lin:M,N,K,a_layout,n,a_batch,0[,fused=0|1][,knob=value...]   tenmo_hip_linear_backward of X[a_batch, M, K] . W[K, N] + b[N]: the three
//     gradients against float64; fused=1: the call must take as many kernel launches with the bias gradient as without it (the sums
//     come out of the weight-gradient launch), fused=0: more
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
extern "C" long replay_launch_count();
extern "C" const char* replay_last_kernel();

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
    std::string ran;
    std::vector<std::pair<std::string, int>> knobs;
    for (size_t i = 8; i < f.size(); ++i) {
        const size_t eq = f[i].find('=');
        if (eq == std::string::npos) continue;
        const std::string name = f[i].substr(0, eq);
        const int value = atoi(f[i].c_str() + eq + 1);
        if (name == "check") check = value != 0;
        else if (name == "ran") { // the kernel that must have served the product (a part of its launch expression; ';' stands for ',')
            ran = f[i].substr(eq + 1);
            for (char& c : ran) if (c == ';') c = ',';
        }
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
    if (rc == 0 && !ran.empty() && !strstr(replay_last_kernel(), ran.c_str())) {
        fprintf(stderr, "%s: served by %s\n", spec.c_str(), replay_last_kernel());
        bad = 1;
    }
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

__attribute__((no_sanitize("address"))) static double gradient_error(const float* got, const std::vector<double>& want) {
    double num = 0.0, den = 0.0;
    for (size_t i = 0; i < want.size(); ++i) { const double d = (double)got[i] - want[i]; num += d * d; den += want[i] * want[i]; }
    return std::sqrt(num / (den > 0 ? den : 1.0));
}

// mv / vm on exactly-sized blocks; the vector has one element per k and no padding
static int run_vector_case(const std::string& spec, bool is_mv) {
    std::vector<std::string> f;
    size_t pos = 3;
    while (pos <= spec.size()) {
        const size_t c = spec.find(',', pos);
        f.push_back(spec.substr(pos, c == std::string::npos ? std::string::npos : c - pos));
        if (c == std::string::npos) break;
        pos = c + 1;
    }
    if (f.size() < 6) { fprintf(stderr, "bad case %s\n", spec.c_str()); return 2; }
    const int64_t d0 = atoll(f[0].c_str()), d1 = atoll(f[1].c_str());   // mv: m, k   vm: k, n
    const bool t = f[2] == "t";
    int64_t batch = atoll(f[3].c_str());
    const int64_t pad = atoll(f[4].c_str());
    const int accumulate = atoi(f[5].c_str());
    bool noalloc = false, join = false;
    for (size_t i = 6; i < f.size(); ++i) {
        if (f[i] == "entry=noalloc") noalloc = true;
        if (f[i] == "join=1") join = true; // K slices added inside the streaming launch; must equal the two-launch result bit for bit
    }
    const bool shared_matrix = batch < 0;
    if (batch < 0) batch = -batch;
    const int64_t nb = batch > 0 ? batch : 1, nmat = shared_matrix ? 1 : nb;
    const int64_t rows = is_mv ? d0 : d0, cols = d1;       // logical matrix [rows][cols]: mv [m][k], vm [k][n]
    const int64_t pitch = (t ? rows : cols) + pad, lines = t ? cols : rows;
    const int64_t mat_elems = lines * pitch - pad;        // the last line carries no padding: the block ends with the matrix
    const int64_t rs = t ? 1 : pitch, cs = t ? pitch : 1;
    const int64_t vec_len = is_mv ? cols : rows, out_len = is_mv ? rows : cols;
    const size_t m_n = (size_t)(nmat * lines * pitch - pad), v_n = (size_t)(nb * vec_len), o_n = (size_t)(nb * out_len);
    float* Mx = (float*)malloc(m_n * 4); float* v = (float*)malloc(v_n * 4); float* out = (float*)malloc(o_n * 4);
    for (size_t i = 0; i < m_n; ++i) Mx[i] = next_float();
    for (size_t i = 0; i < v_n; ++i) v[i] = next_float();
    for (size_t i = 0; i < o_n; ++i) out[i] = next_float();
    std::vector<double> want(o_n);
    for (int64_t b = 0; b < nb; ++b) {
        const float* Mb = Mx + (shared_matrix ? 0 : b * lines * pitch);
        for (int64_t o = 0; o < out_len; ++o) {
            double s2 = accumulate ? (double)out[b * out_len + o] : 0.0;
            for (int64_t r = 0; r < vec_len; ++r)
                s2 += (is_mv ? (double)Mb[o * rs + r * cs] : (double)Mb[r * rs + o * cs]) * (double)v[b * vec_len + r];
            want[(size_t)(b * out_len + o)] = s2;
        }
    }
    (void)mat_elems;
    replay_register(Mx, m_n * 4); replay_register(v, v_n * 4); replay_register(out, o_n * 4);
    const int64_t bshape[1] = {nb}, mstr[1] = {shared_matrix ? 0 : lines * pitch}, vstr[1] = {vec_len};
    auto product = [&](float* dst) {
        if (is_mv) return tenmo_hip_mv_f32(Mx, 0, rs, cs, v, 0, 1, dst, rows, cols, batch > 0 ? 1 : 0, bshape, mstr, vstr, accumulate, 1);
        if (noalloc) return tenmo_hip_vm_f32_noalloc(v, 0, 1, Mx, 0, rs, cs, dst, rows, cols, batch > 0 ? 1 : 0, bshape, vstr, mstr, accumulate, 1);
        return tenmo_hip_vm_f32(v, 0, 1, Mx, 0, rs, cs, dst, rows, cols, batch > 0 ? 1 : 0, bshape, vstr, mstr, accumulate, 1);
    };
    std::vector<float> two_launches;
    long launches_apart = 0;
    int rc = 0;
    if (join) { // first the separate reduction into a copy of the same initial contents
        two_launches.assign(out, out + o_n);
        replay_register(two_launches.data(), o_n * 4);
        const long before = replay_launch_count();
        rc = product(two_launches.data());
        launches_apart = replay_launch_count() - before;
        replay_register(two_launches.data(), 0);
        tenmo_hip_set_tuning("cols_join", 1);
    }
    const long before = replay_launch_count();
    if (rc == 0) rc = product(out);
    const long launches = replay_launch_count() - before;
    if (join) tenmo_hip_set_tuning("cols_join", 0);
    int bad = 0;
    double err = -1;
    if (rc != 0) { fprintf(stderr, "%s: error %d: %s\n", spec.c_str(), rc, tenmo_hip_last_error()); bad = 1; }
    else { err = gradient_error(out, want); if (!(err <= 1e-5)) bad = 1; } // (one output can be a sum with cancellation: the stated tolerance, not a tighter one)
    if (join && rc == 0 && memcmp(out, two_launches.data(), o_n * 4) != 0) { fprintf(stderr, "%s: joined slices differ from the two-launch result\n", spec.c_str()); bad = 1; }
    // a product cut into K slices takes one launch less when they are joined inside the streaming launch
    if (join && rc == 0 && launches_apart > 1 && launches != launches_apart - 1) { fprintf(stderr, "%s: %ld launches joined, %ld apart\n", spec.c_str(), launches, launches_apart); bad = 1; }
    printf("%s: rc %d, relative error %.3g, %ld launch%s%s\n", spec.c_str(), rc, err, launches, launches == 1 ? "" : "es", bad ? "  <-- FAILED" : "");
    fflush(stdout);
    replay_register(Mx, 0); replay_register(v, 0); replay_register(out, 0);
    free(Mx); free(v); free(out);
    return bad;
}

static std::vector<int64_t> numbers_of(const std::string& spec, size_t from) {
    std::vector<int64_t> out;
    size_t pos = from;
    while (pos <= spec.size()) {
        const size_t c = spec.find(',', pos);
        out.push_back(atoll(spec.substr(pos, c == std::string::npos ? std::string::npos : c - pos).c_str()));
        if (c == std::string::npos) break;
        pos = c + 1;
    }
    return out;
}

static float* exact_block(size_t n, bool fill = true) {
    float* p = (float*)malloc(n ? n * 4 : 1);
    for (size_t i = 0; i < n && fill; ++i) p[i] = next_float();
    replay_register(p, n ? n * 4 : 1);
    return p;
}
static void drop_block(void* p) { replay_register(p, 0); free(p); }

// entry points whose numbers the parity tests check: here only that every access stays inside exactly-sized operands
static int run_address_only_case(const std::string& spec) {
    int rc = 0;
    if (spec.compare(0, 3, "ce:") == 0) {
        const std::vector<int64_t> a = numbers_of(spec, 3);
        if (a.size() < 4) return 2;
        const int64_t M = a[0], C = a[1];
        const bool i64 = a[2] != 0;
        const float ls = (float)a[3] / 100.f;
        float* logits = exact_block((size_t)(M * C));
        void* target = malloc((size_t)M * (i64 ? 8 : 4));
        replay_register(target, (size_t)M * (i64 ? 8 : 4));
        for (int64_t m = 0; m < M; ++m) {
            const int64_t t = (m % 7 == 3) ? -100 : (m * 31) % C;
            if (i64) ((int64_t*)target)[m] = t; else ((int32_t*)target)[m] = (int32_t)t;
        }
        // a fifth number: softmax (1), softmax and gradient (2) or all three arrays (3) begin one float into their blocks: no 16-byte alignment
        const int64_t shift = a.size() > 4 ? a[4] : 0;
        float* logits_block = shift >= 3 ? exact_block((size_t)(M * C) + 1) : nullptr;
        if (logits_block) { drop_block(logits); logits = logits_block + 1; }
        float* softmax_block = exact_block((size_t)(M * C) + (shift >= 1), false); float* per = exact_block((size_t)M, false); float* sum = exact_block(1, false);
        int32_t* valid = (int32_t*)exact_block(1, false); float* up = exact_block(1); float* grad_block = exact_block((size_t)(M * C) + (shift >= 2));
        float* softmax = softmax_block + (shift >= 1); float* grad = grad_block + (shift >= 2);
        rc = tenmo_hip_cross_entropy_forward_f32(logits, target, i64, M, C, -100, ls, softmax, per, sum, valid, 1);
        if (rc == 0) rc = tenmo_hip_cross_entropy_forward_f32(logits, target, i64, M, C, -100, ls, nullptr, per, sum, valid, 1);
        if (rc == 0) rc = tenmo_hip_cross_entropy_backward_f32(softmax, target, i64, up, M, C, -100, ls, 2, valid[0], grad, 0, 1);
        if (rc == 0) rc = tenmo_hip_cross_entropy_backward_f32(softmax, target, i64, up, M, C, -100, ls, 1, valid[0], grad, 1, 1);
        if (logits_block) drop_block(logits_block); else drop_block(logits);
        drop_block(target); drop_block(softmax_block); drop_block(per); drop_block(sum); drop_block(valid); drop_block(up); drop_block(grad_block);
    } else if (spec.compare(0, 5, "conv:") == 0) {
        const std::vector<int64_t> a = numbers_of(spec, 5);
        if (a.size() < 9) return 2;
        const int64_t N = a[0], Ci = a[1], H = a[2], W = a[3], Co = a[4], KH = a[5], KW = a[6], st = a[7], dil = a[8];
        const int64_t Ho = (H - (KH + (KH - 1) * (dil - 1))) / st + 1, Wo = (W - (KW + (KW - 1) * (dil - 1))) / st + 1;
        float* img = exact_block((size_t)(N * Ci * H * W)); float* ker = exact_block((size_t)(Co * Ci * KH * KW)); float* bias = exact_block((size_t)Co);
        float* out = exact_block((size_t)(N * Co * Ho * Wo), false); float* gout = exact_block((size_t)(N * Co * Ho * Wo));
        float* gimg = exact_block((size_t)(N * Ci * H * W)); float* gker = exact_block((size_t)(Co * Ci * KH * KW)); float* gbias = exact_block((size_t)Co);
        rc = tenmo_hip_conv2d_forward_f32(img, N, Ci, H, W, ker, Co, KH, KW, bias, st, dil, out, 1);
        if (rc == 0) rc = tenmo_hip_conv2d_backward_f32(img, N, Ci, H, W, ker, Co, KH, KW, st, dil, gout, gimg, gker, gbias, 0, 1);
        if (rc == 0) rc = tenmo_hip_conv2d_backward_f32(img, N, Ci, H, W, ker, Co, KH, KW, st, dil, gout, gimg, gker, gbias, 1, 1);
        drop_block(img); drop_block(ker); drop_block(bias); drop_block(out); drop_block(gout); drop_block(gimg); drop_block(gker); drop_block(gbias);
    } else if (spec.compare(0, 4, "mlp:") == 0) {
        const std::vector<int64_t> a = numbers_of(spec, 4);
        if (a.size() < 6) return 2;
        const int64_t B = a[0], dims[4] = {a[1], a[2], a[3], a[4]};
        std::vector<std::vector<float>> W(3), bvec(3);
        const float* Wp[3];
        const float* bp[3];
        for (int l = 0; l < 3; ++l) {
            W[l].resize((size_t)(dims[l] * dims[l + 1])); bvec[l].resize((size_t)dims[l + 1]);
            for (float& w : W[l]) w = 0.1f * next_float();
            for (float& w : bvec[l]) w = 0.1f * next_float();
            Wp[l] = W[l].data(); bp[l] = bvec[l].data();
        }
        tenmo_mlp* m = tenmo_hip_mlp_create(3, dims, Wp, bp, B);
        float* x = exact_block((size_t)(B * dims[0]));
        int32_t* y = (int32_t*)exact_block((size_t)B, false);
        for (int64_t i = 0; i < B; ++i) y[i] = (int32_t)((i * 7) % dims[3]);
        float* loss = exact_block(1, false);
        tenmo_hip_set_tuning("mlp_fused_tail", (int)a[5]);
        rc = m ? 0 : -1;
        for (int step = 0; step < 2 && rc == 0; ++step) rc = tenmo_hip_mlp_step(m, x, y, B, 0.05f, loss, 1);
        tenmo_hip_set_tuning("mlp_fused_tail", 0);
        if (rc == 0 && !(loss[0] == loss[0])) rc = -100; // NaN
        tenmo_hip_mlp_destroy(m);
        drop_block(x); drop_block(y); drop_block(loss);
    } else {
        const std::vector<int64_t> a = numbers_of(spec, 5);
        if (a.empty()) return 2;
        const int64_t n = a[0];
        float* x = exact_block((size_t)n); float* y = exact_block((size_t)n); float* d = exact_block(1, false);
        rc = tenmo_hip_dot_f32(x, 0, 1, y, 0, 1, n, d, 1);
        float* vel = exact_block((size_t)n);
        if (rc == 0) rc = tenmo_hip_sgd_step_f32(x, y, nullptr, n, 0.01f, 0.f, 0.f, 1);
        if (rc == 0) rc = tenmo_hip_sgd_step_f32(x, y, vel, n, 0.01f, 0.9f, 1e-4f, 1);
        if (rc == 0 && n > 1) rc = tenmo_hip_sgd_step_f32(x + 1, y, vel, n - 1, 0.01f, 0.9f, 1e-4f, 1); // (parameters that are not 16-byte aligned)
        const int64_t rows = n / 64 + 1, cols = 64 + n % 61;
        float* G = exact_block((size_t)(rows * cols)); float* cs = exact_block((size_t)cols);
        if (rc == 0) rc = tenmo_hip_column_sum_f32(G, 0, cols, rows, cols, cs, 1, 1);
        drop_block(x); drop_block(y); drop_block(d); drop_block(vel); drop_block(G); drop_block(cs);
    }
    if (rc != 0) fprintf(stderr, "%s: error %d: %s\n", spec.c_str(), rc, tenmo_hip_last_error());
    printf("%s: rc %d, relative error n/a\n", spec.c_str(), rc);
    fflush(stdout);
    return rc != 0;
}

// (generic: row-major storage of twice the width of which every second element is used: no unit stride)
static tenmo_view view_of(const float* p, int64_t batch, int64_t rows, int64_t cols, bool transposed, bool generic = false) {
    tenmo_view v;
    memset(&v, 0, sizeof(v));
    v.data = p;
    int r = 0;
    if (batch > 0) { v.shape[r] = batch; v.strides[r] = rows * cols * (generic ? 2 : 1); ++r; }
    v.shape[r] = rows; v.strides[r] = generic ? 2 * cols : transposed ? 1 : cols; ++r;
    v.shape[r] = cols; v.strides[r] = generic ? 2 : transposed ? rows : 1; ++r;
    v.rank = r;
    return v;
}

// mv and vm with their gradients through the view-level entry points, addresses only (the parity tests check the numbers):
// vbw:m,k,matrix_batch,vector_batch,generic   M[matrix_batch, m, k] (generic: every second element of its storage), v[vector_batch, k]
// (a batch of 0: no batch dimension); then the same matrix as [k', n] = [m, k] under u[vector_batch, m]
static int run_vector_backward_case(const std::string& spec) {
    const std::vector<int64_t> a = numbers_of(spec, 4);
    if (a.size() < 5) return 2;
    const int64_t m = a[0], k = a[1], bm = a[2], bv = a[3];
    const bool generic = a[4] != 0;
    const int64_t nm = bm > 0 ? bm : 1, nv = bv > 0 ? bv : 1, nb = nm > nv ? nm : nv;
    float* Mx = exact_block((size_t)(nm * m * k * (generic ? 4 : 1)));
    float* v = exact_block((size_t)(nv * k)); float* u = exact_block((size_t)(nv * m));
    float* out_mv = exact_block((size_t)(nb * m), false); float* out_vm = exact_block((size_t)(nb * k), false);
    float* dy_mv = exact_block((size_t)(nb * m)); float* dy_vm = exact_block((size_t)(nb * k));
    float* gM = exact_block((size_t)(nm * m * k)); float* gv = exact_block((size_t)(nv * k)); float* gu = exact_block((size_t)(nv * m));
    tenmo_view vM = view_of(Mx, bm, m, k, false, generic);
    tenmo_view vv, vu;
    memset(&vv, 0, sizeof(vv));
    vv.data = v;
    int r = 0;
    if (bv > 0) { vv.shape[r] = bv; vv.strides[r] = k; ++r; }
    vv.shape[r] = k; vv.strides[r] = 1; ++r;
    vv.rank = r;
    vu = vv;
    vu.data = u;
    vu.shape[r - 1] = m;
    if (bv > 0) vu.strides[0] = m;
    int rc = tenmo_hip_matrix_vector_nd(&vM, &vv, out_mv, 1);
    if (rc == 0) rc = tenmo_hip_mv_backward(&vM, &vv, dy_mv, gM, gv, 1);
    if (rc == 0) rc = tenmo_hip_vector_matmul_nd(&vu, &vM, out_vm, 1);
    if (rc == 0) rc = tenmo_hip_vm_backward(&vu, &vM, dy_vm, gu, gM, 1);
    if (rc != 0) fprintf(stderr, "%s: error %d: %s\n", spec.c_str(), rc, tenmo_hip_last_error());
    printf("%s: rc %d, relative error n/a\n", spec.c_str(), rc);
    fflush(stdout);
    drop_block(Mx); drop_block(v); drop_block(u); drop_block(out_mv); drop_block(out_vm); drop_block(dy_mv); drop_block(dy_vm); drop_block(gM); drop_block(gv); drop_block(gu);
    return rc != 0;
}

static int run_backward_case(const std::string& spec) {
    const bool linear = spec.compare(0, 4, "lin:") == 0;
    int want_fused = -1;
    int64_t a_skip = 1; // skip=1: A's matrices are every second one of its storage (their rows do not stack into one taller matrix)
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
    const bool ta = f[3] == "t", tb = f[4] == "t", ga = f[3] == "g", gb = f[4] == "g";
    const int64_t ba = atoll(f[5].c_str()), bb = atoll(f[6].c_str());
    std::vector<std::pair<std::string, int>> knobs;
    for (size_t i = 7; i < f.size(); ++i) {
        const size_t eq = f[i].find('=');
        if (eq == std::string::npos) continue;
        if (f[i].substr(0, eq) == "fused") want_fused = atoi(f[i].c_str() + eq + 1);
        else if (f[i].substr(0, eq) == "skip") a_skip = atoi(f[i].c_str() + eq + 1) > 0 ? 2 : 1;
        else knobs.push_back({f[i].substr(0, eq), atoi(f[i].c_str() + eq + 1)});
    }
    const int64_t na = ba > 0 ? ba : 1, nb = bb > 0 ? bb : 1, nc = na > nb ? na : nb;
    const size_t a_n = (size_t)(na * M * K), b_n = (size_t)(nb * K * N), c_n = (size_t)(nc * M * N); // elements of the views = of the gradients
    const int64_t a_mat = M * K * (ga ? 2 : 1) * a_skip, b_mat = K * N * (gb ? 2 : 1);                 // storage per matrix (of A: distance between matrices)
    const size_t a_store = (size_t)(na * a_mat), b_store = (size_t)(nb * b_mat);
    float* A = (float*)malloc(a_store * 4); float* B = (float*)malloc(b_store * 4); float* dC = (float*)malloc(c_n * 4);
    float* gA = (float*)malloc(a_n * 4); float* gB = (float*)malloc(b_n * 4);
    float* gbias = (float*)malloc((size_t)N * 4 ? (size_t)N * 4 : 1);
    std::vector<double> want_bias((size_t)N);
    for (int64_t n = 0; n < N; ++n) { gbias[n] = next_float(); want_bias[(size_t)n] = gbias[n]; }
    for (size_t i = 0; i < a_store; ++i) A[i] = next_float();
    for (size_t i = 0; i < b_store; ++i) B[i] = next_float();
    for (size_t i = 0; i < a_n; ++i) gA[i] = next_float();
    for (size_t i = 0; i < b_n; ++i) gB[i] = next_float();
    for (size_t i = 0; i < c_n; ++i) dC[i] = next_float();
    // storage: A[b] is [M][K] (n), [K][M] (t) or [M][2K] with every second element used (g); the gradients are dense at the VIEW's shape
    const int64_t a_rs = ga ? 2 * K : ta ? 1 : K, a_cs = ga ? 2 : ta ? M : 1, b_rs = gb ? 2 * N : tb ? 1 : N, b_cs = gb ? 2 : tb ? K : 1;
    std::vector<double> wantA(a_n), wantB(b_n);
    for (size_t i = 0; i < a_n; ++i) wantA[i] = gA[i];
    for (size_t i = 0; i < b_n; ++i) wantB[i] = gB[i];
    for (int64_t c = 0; c < nc; ++c) {
        const int64_t ia = na > 1 ? c : 0, ib = nb > 1 ? c : 0;
        const float* Ab = A + ia * a_mat; const float* Bb = B + ib * b_mat; const float* Gb = dC + c * M * N;
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
        for (int64_t m = 0; m < M; ++m)
            for (int64_t n = 0; n < N; ++n) want_bias[(size_t)n] += (double)Gb[m * N + n];
    }
    replay_register(gbias, (size_t)N * 4);
    replay_register(A, a_store * 4); replay_register(B, b_store * 4); replay_register(dC, c_n * 4); replay_register(gA, a_n * 4); replay_register(gB, b_n * 4);
    tenmo_view va = view_of(A, ba, M, K, ta, ga), vb = view_of(B, bb, K, N, tb, gb);
    if (ba > 0) va.strides[0] = a_mat;
    for (auto& kv : knobs) tenmo_hip_set_tuning(kv.first.c_str(), kv.second);
    int bad = 0;
    long without_bias = 0;
    if (linear) { // the same call without the bias gradient, into copies of the gradients: the number of launches to compare with
        std::vector<float> sA(gA, gA + a_n), sB(gB, gB + b_n);
        replay_register(sA.data(), a_n * 4); replay_register(sB.data(), b_n * 4);
        const long before = replay_launch_count();
        if (tenmo_hip_linear_backward(&va, &vb, dC, sA.data(), sB.data(), nullptr, 1) != 0) bad = 1;
        without_bias = replay_launch_count() - before;
        replay_register(sA.data(), 0); replay_register(sB.data(), 0);
    }
    const long before = replay_launch_count();
    const int rc = linear ? tenmo_hip_linear_backward(&va, &vb, dC, gA, gB, gbias, 1) : tenmo_hip_matmul_backward(&va, &vb, dC, gA, gB, 1);
    const long launches = replay_launch_count() - before;
    for (auto& kv : knobs) tenmo_hip_set_tuning(kv.first.c_str(), -1);
    double ea = -1, eb = -1, ebias = -1;
    if (rc != 0) { fprintf(stderr, "%s: error %d: %s\n", spec.c_str(), rc, tenmo_hip_last_error()); bad = 1; }
    else { ea = gradient_error(gA, wantA); eb = gradient_error(gB, wantB); if (!(ea <= 2e-6 && eb <= 2e-6)) bad = 1; }
    if (linear && rc == 0) {
        std::vector<float> got(gbias, gbias + N);
        ebias = gradient_error(got.data(), want_bias);
        if (!(ebias <= 2e-6)) bad = 1;
        if (want_fused == 1 && launches != without_bias) bad = 1;
        if (want_fused == 0 && launches <= without_bias) bad = 1;
        printf("%s: %ld launches, %ld without the bias gradient; bias gradient error %.3g\n", spec.c_str(), launches, without_bias, ebias);
    }
    printf("%s: rc %d, relative error %.3g / %.3g%s\n", spec.c_str(), rc, ea, eb, bad ? "  <-- FAILED" : "");
    fflush(stdout);
    replay_register(gbias, 0);
    free(gbias);
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
        if (strncmp(argv[i], "bwd:", 4) == 0 || strncmp(argv[i], "lin:", 4) == 0) bad |= run_backward_case(argv[i]);
        else if (strncmp(argv[i], "ce:", 3) == 0 || strncmp(argv[i], "conv:", 5) == 0 || strncmp(argv[i], "misc:", 5) == 0 || strncmp(argv[i], "mlp:", 4) == 0)
            bad |= run_address_only_case(argv[i]);
        else if (strncmp(argv[i], "vbw:", 4) == 0) bad |= run_vector_backward_case(argv[i]);
        else if (strncmp(argv[i], "mv:", 3) == 0) bad |= run_vector_case(argv[i], true);
        else if (strncmp(argv[i], "vm:", 3) == 0) bad |= run_vector_case(argv[i], false);
        else bad |= run_case(argv[i]);
    }
    tenmo_hip_shutdown();
    return bad;
}
