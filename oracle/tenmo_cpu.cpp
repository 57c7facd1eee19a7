// CPU oracle for Tenmo's fp32 matrix-product path — TEST INFRASTRUCTURE ONLY.
//
// A plain C++ restatement of the reference's CPU algorithms, used (a) by the tests as the
// checker for the HIP library and (b) by the benchmark as the CPU baseline timed beside the
// GPU.  The product never links, loads or calls this file.
//
// What is restated, and from where (paths relative to the reference tree):
//   contiguity predicate            tenmo/strides.mojo:239-266
//   rank classification             tenmo/matmul.mojo:258-272
//   2-D matmul (tile table, paths)  tenmo/matmul_cpu.mojo:80-135, :163-547
//   batched/broadcast matmul        tenmo/matmul_cpu.mojo:568-625, :628-956
//   broadcast rules                 tenmo/broadcasthelper.mojo:33-62, :123-132, :201-216
//   matrix x vector (+ backward)    tenmo/matrixvector.mojo:205-286, :19-201
//   vector x matrix (+ backward)    tenmo/vectormatrix.mojo:210-338, :18-206
//   dot                             tenmo/dotproduct.mojo:56-123
//   sum over broadcast axes         tenmo/sum_mean_reduction.mojo:185-211
//   MLP harness (Linear, bias add, ReLU, cross-entropy, SGD)
//       tenmo/net.mojo:179-216, addition.mojo:73-112, broadcast.mojo:66-88, relu.mojo:99-141,
//       crossentropy.mojo:285-432 and :775-793 with :451-481, optim.mojo:93-120
//
// Parity status.  Every function below is pinned by the reference's own literal test vectors
// (tests/golden/*.json, transcribed from the reference's tests) and by fp64 brute force on
// random inputs.  NOT pinned bit-for-bit (no Mojo toolchain exists to run the reference):
// whether Mojo contracts the scalar `acc += a*b` tails into a fused multiply-add, and the last
// ulp of Mojo's exp/log inside the cross-entropy.  Both are far inside the stated tolerances.
#include "tenmo_cpu.h"
#include "mm_args.h"

#include <omp.h>
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <limits>
#include <set>
#include <string>
#include <vector>

namespace {

thread_local std::string g_err;
int fail(const std::string& m) { g_err = m; return -1; }

int g_forced_width = 0;

struct Isa {
    row_tile_fn (*select)(int, int, int);
    int (*lanes)();
    void (*vm_contig)(const float*, int64_t, int64_t, const float*, int64_t, int64_t, int64_t, int64_t, float*);
    void (*axpy_row)(float, const float*, int64_t, float*, int64_t);
};

Isa pick_isa() {
    int want = g_forced_width;
    bool has512 = __builtin_cpu_supports("avx512f");
    bool has2 = __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
    if ((want == 0 || want == 16) && has512) return {isa_avx512::select, isa_avx512::lanes, isa_avx512::vm_contig, isa_avx512::axpy_row};
    if ((want == 0 || want == 8 || want == 16) && has2 && want != 1) return {isa_avx2::select, isa_avx2::lanes, isa_avx2::vm_contig, isa_avx2::axpy_row};
    return {isa_generic::select, isa_generic::lanes, isa_generic::vm_contig, isa_generic::axpy_row};
}

int physical_cores() {
    // unique (package, core) pairs from sysfs; falls back to the OpenMP processor count
    std::set<std::pair<int, int>> cores;
    for (int cpu = 0; cpu < 4096; ++cpu) {
        std::string base = "/sys/devices/system/cpu/cpu" + std::to_string(cpu) + "/topology/";
        std::ifstream fc(base + "core_id"), fp(base + "physical_package_id");
        if (!fc.good() || !fp.good()) break;
        int c = -1, p = -1;
        fc >> c; fp >> p;
        cores.insert({p, c});
    }
    int n = (int)cores.size();
    int avail = omp_get_num_procs();
    if (n <= 0 || n > avail) n = avail;
    return std::max(1, n);
}

int threads_or_default(int nthreads) { return nthreads > 0 ? nthreads : physical_cores(); }

bool contiguous(int rank, const int64_t* shape, const int64_t* strides) {
    if (rank == 0) return true;
    int64_t expected = 1;
    for (int i = rank - 1; i >= 0; --i) {
        if (shape[i] > 1 && strides[i] != expected) return false;
        expected *= shape[i];
    }
    return true;
}
bool contiguous(const oracle_view* v) { return contiguous(v->rank, v->shape, v->strides); }

std::string shape_str(const int64_t* s, int r) {
    std::string o = "(";
    for (int i = 0; i < r; ++i) o += (i ? ", " : "") + std::to_string(s[i]);
    return o + ")";
}

// right-aligned broadcast of two batch shapes (broadcasthelper.mojo:33-62); false if incompatible
bool broadcast_batch(const int64_t* sa, int ra, const int64_t* sb, int rb, int64_t* out, int* rout) {
    int r = std::max(ra, rb);
    for (int d = 0; d < r; ++d) {
        int ia = d - (r - ra), ib = d - (r - rb);
        int64_t da = ia >= 0 ? sa[ia] : 1, db = ib >= 0 ? sb[ib] : 1;
        if (da == db) out[d] = da;
        else if (da == 1) out[d] = db;
        else if (db == 1) out[d] = da;
        else return false;
    }
    *rout = r;
    return true;
}

// offset of batch `b` (row-major over batch_shape) in an operand whose own batch dims are
// right-aligned and read with stride 0 where its size is 1 (matmul_cpu.mojo:710-724)
int64_t batch_offset(int64_t b, const int64_t* bshape, int brank, const int64_t* oshape, const int64_t* ostrides, int orank) {
    int64_t off = 0, divisor = 1;
    for (int d = brank - 1; d >= 0; --d) {
        int64_t coord = (b / divisor) % bshape[d];
        int od = d - (brank - orank);
        if (od >= 0 && oshape[od] > 1) off += coord * ostrides[od];
        divisor *= bshape[d];
    }
    return off;
}

void tile_table(int64_t m, int64_t n, int64_t p, int* tm, int* tn, int* tp) {
    *tm = m > 256 ? 128 : (m > 64 ? 64 : 32); // matmul_cpu.mojo:87
    *tn = n > 64 ? 64 : 32;                   // :88
    *tp = p > 256 ? 256 : (p > 64 ? 128 : 64); // :89
}

int64_t product(const int64_t* s, int r) { int64_t x = 1; for (int i = 0; i < r; ++i) x *= s[i]; return x; }

} // namespace

extern "C" {

const char* oracle_last_error(void) { return g_err.c_str(); }
int oracle_simd_width(void) { return pick_isa().lanes(); }
void oracle_force_simd_width(int w) { g_forced_width = w; }
int oracle_num_physical_cores(void) { return physical_cores(); }

int oracle_is_contiguous(int32_t rank, const int64_t* shape, const int64_t* strides) { return contiguous(rank, shape, strides) ? 1 : 0; }

int oracle_classify_matmul(int32_t ra, const int64_t* a, int32_t rb, const int64_t* b) {
    if (ra <= 1 && rb <= 1) return 0;
    if (ra == 1 && rb >= 2) return 1;
    if (ra >= 2 && rb == 1) return 2;
    if (ra >= 2 && rb >= 2) return a[ra - 1] == b[rb - 2] ? 3 : -1;
    return -1; // rank 0 against rank >= 2: the reference's final branch would index an empty shape
}

int oracle_mm2d_f32(const oracle_view* A, const oracle_view* B, float* C, int nthreads, int* path_out, int* tiles_out) {
    if (A->rank != 2 || B->rank != 2)
        return fail("validate_matrix_shapes_2d: matmul_2d expects rank == 2. Got A = " + shape_str(A->shape, A->rank) + ", B = " + shape_str(B->shape, B->rank));
    if (A->shape[1] != B->shape[0])
        return fail("validate_matrix_shapes_2d: inner dimensions mismatch in matmul_2d: A(m," + std::to_string(A->shape[1]) + ") vs B(" + std::to_string(B->shape[0]) + ",n)");
    const int64_t m = A->shape[0], n = A->shape[1], p = B->shape[1];
    int tm, tn, tp;
    tile_table(m, n, p, &tm, &tn, &tp);
    if (tiles_out) { tiles_out[0] = tm; tiles_out[1] = tn; tiles_out[2] = tp; }
    std::memset(C, 0, sizeof(float) * (size_t)(m * p)); // NDBuffer.zeros, matmul_cpu.mojo:183

    MmArgs g{A->data, B->data, C, A->strides[0], A->strides[1], B->strides[0], B->strides[1], n, p, 0, 1};
    g.path = contiguous(B) ? (contiguous(A) ? 0 : 1) : 2;       // :206, :209
    if (path_out) *path_out = g.path;
    Isa isa = pick_isa();
    row_tile_fn fn = isa.select(tm, tn, tp);
    if (!fn) return fail("tile dispatch: no instantiation");
    const int64_t tiles = (m + tm - 1) / tm;
    const int nt = threads_or_default(nthreads);
    const int64_t a_off = A->offset, b_off = B->offset;
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t t = 0; t < tiles; ++t) {
        int64_t i0 = t * tm, i1 = std::min<int64_t>(i0 + tm, m);
        fn(g, a_off, b_off, 0, i0, i1);
    }
    return 0;
}

int64_t oracle_result_shape(int mode, const oracle_view* A, const oracle_view* B, int64_t* out_shape, int32_t* out_rank) {
    // mode 3: A[...,m,k] B[...,k,p];  mode 2: M[...,m,k] v[...,k];  mode 1: v[...,k] M[...,k,n]
    int ta = (mode == 1) ? 1 : 2, tb = (mode == 2) ? 1 : 2; // trailing (non-batch) dims of each operand
    if (A->rank < ta || B->rank < tb) return fail("operand rank too small");
    int64_t ka = A->shape[A->rank - 1], kb = B->shape[B->rank - tb];
    if (ka != kb) return fail("inner dims must match, got " + std::to_string(ka) + " and " + std::to_string(kb));
    int br = 0;
    if (!broadcast_batch(A->shape, A->rank - ta, B->shape, B->rank - tb, out_shape, &br))
        return fail("cannot broadcast shapes: " + shape_str(A->shape, A->rank - ta) + ", " + shape_str(B->shape, B->rank - tb));
    if (mode != 1) out_shape[br++] = A->shape[A->rank - 2];
    if (mode != 2) out_shape[br++] = B->shape[B->rank - 1];
    if (br > ORACLE_MAX_RANK) return fail("rank exceeds max_rank");
    *out_rank = br;
    return product(out_shape, br);
}

int oracle_mmnd_f32(const oracle_view* A, const oracle_view* B, float* C, int nthreads,
                    int64_t* out_shape, int32_t* out_rank, int64_t work_item_limit) {
    if (A->rank < 2 || B->rank < 2) return fail("matmul_nd: inputs must be at least 2D");
    int64_t oshape[ORACLE_MAX_RANK + 2]; int32_t orank = 0;
    int64_t total = oracle_result_shape(3, A, B, oshape, &orank);
    if (total < 0) return -1;
    if (out_shape) std::copy(oshape, oshape + orank, out_shape);
    if (out_rank) *out_rank = orank;
    const int ar = A->rank, br = B->rank, batch_rank = orank - 2;
    const int64_t m = A->shape[ar - 2], k = A->shape[ar - 1], p = B->shape[br - 1];
    int64_t total_batch = product(oshape, batch_rank);
    if (total_batch == 0) total_batch = 1; // matmul_cpu.mojo:666-667
    int tm, tn, tp;
    tile_table(m, k, p, &tm, &tn, &tp);
    if (work_item_limit <= 0) std::memset(C, 0, sizeof(float) * (size_t)total);

    MmArgs g{A->data, B->data, C, A->strides[ar - 2], A->strides[ar - 1], B->strides[br - 2], B->strides[br - 1], k, p, 0, 0};
    g.path = contiguous(B) ? (contiguous(A) ? 0 : 1) : 2; // whole-buffer predicate, :694-695
    Isa isa = pick_isa();
    row_tile_fn fn = isa.select(tm, tn, tp);
    if (!fn) return fail("tile dispatch: no instantiation");
    const int64_t tiles_i = (m + tm - 1) / tm;
    int64_t items = total_batch * tiles_i;
    if (work_item_limit > 0) items = std::min(items, work_item_limit);
    const int nt = threads_or_default(nthreads);
#pragma omp parallel for schedule(static) num_threads(nt)
    for (int64_t f = 0; f < items; ++f) {
        int64_t b = f / tiles_i, t = f % tiles_i;
        int64_t a_base = A->offset + batch_offset(b, oshape, batch_rank, A->shape, A->strides, ar - 2);
        int64_t b_base = B->offset + batch_offset(b, oshape, batch_rank, B->shape, B->strides, br - 2);
        int64_t i0 = t * tm, i1 = std::min<int64_t>(i0 + tm, m);
        if (work_item_limit > 0) std::memset(C + b * m * p + i0 * p, 0, sizeof(float) * (size_t)((i1 - i0) * p));
        fn(g, a_base, b_base, b * m * p, i0, i1);
    }
    return 0;
}

int oracle_mmnd_f64acc(const oracle_view* A, const oracle_view* B, double* C, int nthreads) {
    if (A->rank < 2 || B->rank < 2) return fail("matmul_nd: inputs must be at least 2D");
    int64_t oshape[ORACLE_MAX_RANK + 2]; int32_t orank = 0;
    if (oracle_result_shape(3, A, B, oshape, &orank) < 0) return -1;
    const int ar = A->rank, br = B->rank, batch_rank = orank - 2;
    const int64_t m = A->shape[ar - 2], k = A->shape[ar - 1], p = B->shape[br - 1];
    const int64_t a_rs = A->strides[ar - 2], a_cs = A->strides[ar - 1], b_rs = B->strides[br - 2], b_cs = B->strides[br - 1];
    int64_t total_batch = std::max<int64_t>(1, product(oshape, batch_rank));
    const int nt = threads_or_default(nthreads);
#pragma omp parallel for schedule(dynamic, 4) num_threads(nt)
    for (int64_t f = 0; f < total_batch * m; ++f) {
        int64_t b = f / m, i = f % m;
        int64_t a_base = A->offset + batch_offset(b, oshape, batch_rank, A->shape, A->strides, ar - 2) + i * a_rs;
        int64_t b_base = B->offset + batch_offset(b, oshape, batch_rank, B->shape, B->strides, br - 2);
        double* c = C + (b * m + i) * p;
        for (int64_t j = 0; j < p; ++j) c[j] = 0.0;
        for (int64_t kk = 0; kk < k; ++kk) {
            const double a = (double)A->data[a_base + kk * a_cs];
            const float* brow = B->data + b_base + kk * b_rs;
            if (b_cs == 1) for (int64_t j = 0; j < p; ++j) c[j] += a * (double)brow[j];
            else for (int64_t j = 0; j < p; ++j) c[j] += a * (double)brow[j * b_cs];
        }
    }
    return 0;
}

// ---- mv / vm / dot ------------------------------------------------------------------------

namespace {
struct VecMatGeom {
    int64_t oshape[ORACLE_MAX_RANK + 2]; int32_t orank; int batch_rank; int64_t total_batch;
};
int geom(int mode, const oracle_view* A, const oracle_view* B, VecMatGeom* g) {
    if (oracle_result_shape(mode, A, B, g->oshape, &g->orank) < 0) return -1;
    g->batch_rank = g->orank - 1;
    g->total_batch = product(g->oshape, g->batch_rank); // an empty batch dim yields no iterations
    return 0;
}
} // namespace

int oracle_mv_f32(const oracle_view* M, const oracle_view* v, float* out) {
    if (M->rank < 2) return fail("MatrixVectorMulNd: matrix must have at least 2 dimensions");
    if (v->rank < 1) return fail("MatrixVectorMulNd: vector must have at least 1 dimension");
    if (M->shape[M->rank - 1] != v->shape[v->rank - 1]) return fail("MatrixVectorMulNd: inner dimensions must match");
    VecMatGeom g; if (geom(2, M, v, &g)) return -1;
    const int64_t m = M->shape[M->rank - 2], k = M->shape[M->rank - 1];
    const int64_t rs = M->strides[M->rank - 2], cs = M->strides[M->rank - 1], vs = v->strides[v->rank - 1];
    for (int64_t b = 0; b < g.total_batch; ++b) {
        int64_t mb = M->offset + batch_offset(b, g.oshape, g.batch_rank, M->shape, M->strides, M->rank - 2);
        int64_t vb = v->offset + batch_offset(b, g.oshape, g.batch_rank, v->shape, v->strides, v->rank - 1);
        for (int64_t i = 0; i < m; ++i) {          // matrixvector.mojo:274-284
            float acc = 0.f;
            for (int64_t j = 0; j < k; ++j) acc += M->data[mb + i * rs + j * cs] * v->data[vb + j * vs];
            out[b * m + i] = acc;
        }
    }
    return 0;
}

int oracle_mv_f64acc(const oracle_view* M, const oracle_view* v, double* out) {
    VecMatGeom g; if (geom(2, M, v, &g)) return -1;
    const int64_t m = M->shape[M->rank - 2], k = M->shape[M->rank - 1];
    const int64_t rs = M->strides[M->rank - 2], cs = M->strides[M->rank - 1], vs = v->strides[v->rank - 1];
    for (int64_t b = 0; b < g.total_batch; ++b) {
        int64_t mb = M->offset + batch_offset(b, g.oshape, g.batch_rank, M->shape, M->strides, M->rank - 2);
        int64_t vb = v->offset + batch_offset(b, g.oshape, g.batch_rank, v->shape, v->strides, v->rank - 1);
#pragma omp parallel for schedule(static)
        for (int64_t i = 0; i < m; ++i) {
            double acc = 0.0;
            for (int64_t j = 0; j < k; ++j) acc += (double)M->data[mb + i * rs + j * cs] * (double)v->data[vb + j * vs];
            out[b * m + i] = acc;
        }
    }
    return 0;
}

int oracle_vm_f32(const oracle_view* v, const oracle_view* M, float* out) {
    if (v->rank < 1) return fail("VectorMatmulNd: vector must have rank >= 1");
    if (M->rank < 2) return fail("VectorMatmulNd: matrix must have rank >= 2");
    if (v->shape[v->rank - 1] != M->shape[M->rank - 2]) return fail("VectorMatmulNd: inner dimensions must match");
    VecMatGeom g; if (geom(1, v, M, &g)) return -1;
    const int64_t k = v->shape[v->rank - 1], n = M->shape[M->rank - 1];
    const int64_t rs = M->strides[M->rank - 2], cs = M->strides[M->rank - 1], vs = v->strides[v->rank - 1];
    const bool m_contig = contiguous(M); // vectormatrix.mojo:250
    Isa isa = pick_isa();
    for (int64_t b = 0; b < g.total_batch; ++b) {
        int64_t vb = v->offset + batch_offset(b, g.oshape, g.batch_rank, v->shape, v->strides, v->rank - 1);
        int64_t mb = M->offset + batch_offset(b, g.oshape, g.batch_rank, M->shape, M->strides, M->rank - 2);
        if (m_contig && (cs == 1 || n <= 1)) {
            isa.vm_contig(v->data, vb, vs, M->data, mb, rs, k, n, out + b * n);
        } else {                                   // :326-336 (also a "contiguous" M whose unit dim is skipped)
            for (int64_t j = 0; j < n; ++j) {
                float acc = 0.f;
                for (int64_t i = 0; i < k; ++i) acc += v->data[vb + i * vs] * M->data[mb + i * rs + j * cs];
                out[b * n + j] = acc;
            }
        }
    }
    return 0;
}

int oracle_vm_f64acc(const oracle_view* v, const oracle_view* M, double* out) {
    VecMatGeom g; if (geom(1, v, M, &g)) return -1;
    const int64_t k = v->shape[v->rank - 1], n = M->shape[M->rank - 1];
    const int64_t rs = M->strides[M->rank - 2], cs = M->strides[M->rank - 1], vs = v->strides[v->rank - 1];
    for (int64_t b = 0; b < g.total_batch; ++b) {
        int64_t vb = v->offset + batch_offset(b, g.oshape, g.batch_rank, v->shape, v->strides, v->rank - 1);
        int64_t mb = M->offset + batch_offset(b, g.oshape, g.batch_rank, M->shape, M->strides, M->rank - 2);
        double* o = out + b * n;
        for (int64_t j = 0; j < n; ++j) o[j] = 0.0;
        for (int64_t i = 0; i < k; ++i) {
            double x = (double)v->data[vb + i * vs];
            for (int64_t j = 0; j < n; ++j) o[j] += x * (double)M->data[mb + i * rs + j * cs];
        }
    }
    return 0;
}

int oracle_mv_backward_f32(const oracle_view* M, const oracle_view* v, const float* dy, float* dM, float* dv) {
    VecMatGeom g; if (geom(2, M, v, &g)) return -1;
    const int64_t m = M->shape[M->rank - 2], k = M->shape[M->rank - 1];
    const int64_t rs = M->strides[M->rank - 2], cs = M->strides[M->rank - 1], vs = v->strides[v->rank - 1];
    Isa isa = pick_isa();
    // dense row-major strides of the two parents' gradient boxes
    int64_t gm_str[ORACLE_MAX_RANK], gv_str[ORACLE_MAX_RANK];
    { int64_t acc = 1; for (int d = M->rank - 1; d >= 0; --d) { gm_str[d] = acc; acc *= M->shape[d]; } }
    { int64_t acc = 1; for (int d = v->rank - 1; d >= 0; --d) { gv_str[d] = acc; acc *= v->shape[d]; } }
    if (dM) {
        std::memset(dM, 0, sizeof(float) * (size_t)product(M->shape, M->rank));
        for (int64_t b = 0; b < g.total_batch; ++b) {  // matrixvector.mojo:66-126
            int64_t vb = v->offset + batch_offset(b, g.oshape, g.batch_rank, v->shape, v->strides, v->rank - 1);
            int64_t gb = batch_offset(b, g.oshape, g.batch_rank, M->shape, gm_str, M->rank - 2);
            for (int64_t i = 0; i < m; ++i)
                isa.axpy_row(dy[b * m + i], v->data + vb, vs, dM + gb + i * k, k);
        }
    }
    if (dv) {
        std::memset(dv, 0, sizeof(float) * (size_t)product(v->shape, v->rank));
        for (int64_t b = 0; b < g.total_batch; ++b) {  // :162-196
            int64_t mb = M->offset + batch_offset(b, g.oshape, g.batch_rank, M->shape, M->strides, M->rank - 2);
            int64_t gb = batch_offset(b, g.oshape, g.batch_rank, v->shape, gv_str, v->rank - 1);
            for (int64_t j = 0; j < k; ++j) {
                float acc = 0.f;
                for (int64_t i = 0; i < m; ++i) acc += M->data[mb + i * rs + j * cs] * dy[b * m + i];
                dv[gb + j] += acc;
            }
        }
    }
    return 0;
}

int oracle_vm_backward_f32(const oracle_view* v, const oracle_view* M, const float* dy, float* dv, float* dM) {
    VecMatGeom g; if (geom(1, v, M, &g)) return -1;
    const int64_t k = v->shape[v->rank - 1], n = M->shape[M->rank - 1];
    const int64_t rs = M->strides[M->rank - 2], cs = M->strides[M->rank - 1], vs = v->strides[v->rank - 1];
    Isa isa = pick_isa();
    int64_t gm_str[ORACLE_MAX_RANK], gv_str[ORACLE_MAX_RANK];
    { int64_t acc = 1; for (int d = M->rank - 1; d >= 0; --d) { gm_str[d] = acc; acc *= M->shape[d]; } }
    { int64_t acc = 1; for (int d = v->rank - 1; d >= 0; --d) { gv_str[d] = acc; acc *= v->shape[d]; } }
    if (dv) {
        std::memset(dv, 0, sizeof(float) * (size_t)product(v->shape, v->rank));
        for (int64_t b = 0; b < g.total_batch; ++b) {  // vectormatrix.mojo:65-100
            int64_t mb = M->offset + batch_offset(b, g.oshape, g.batch_rank, M->shape, M->strides, M->rank - 2);
            int64_t gb = batch_offset(b, g.oshape, g.batch_rank, v->shape, gv_str, v->rank - 1);
            for (int64_t i = 0; i < k; ++i) {
                float acc = 0.f;
                for (int64_t j = 0; j < n; ++j) acc += dy[b * n + j] * M->data[mb + i * rs + j * cs];
                dv[gb + i] += acc;
            }
        }
    }
    if (dM) {
        std::memset(dM, 0, sizeof(float) * (size_t)product(M->shape, M->rank));
        for (int64_t b = 0; b < g.total_batch; ++b) {  // :125-188
            int64_t vb = v->offset + batch_offset(b, g.oshape, g.batch_rank, v->shape, v->strides, v->rank - 1);
            int64_t gb = batch_offset(b, g.oshape, g.batch_rank, M->shape, gm_str, M->rank - 2);
            for (int64_t i = 0; i < k; ++i)
                isa.axpy_row(v->data[vb + i * vs], dy + b * n, 1, dM + gb + i * n, n);
        }
    }
    return 0;
}

int oracle_dot_f32(const oracle_view* a, const oracle_view* b, float* out) {
    if (a->rank > 1 || b->rank > 1) return fail("Tensor -> dot: not supported for rank > 1");
    int64_t na = a->rank ? a->shape[0] : 1, nb = b->rank ? b->shape[0] : 1;
    int64_t sa = a->rank ? a->strides[0] : 0, sb = b->rank ? b->strides[0] : 0;
    // a one-element operand is broadcast to the other's length first (dotproduct.mojo:67-74)
    if (na == 1 && nb > 1) { na = nb; sa = 0; }
    else if (nb == 1 && na > 1) { nb = na; sb = 0; }
    if (na != nb) return fail("Tensor -> dot: size does not match " + std::to_string(na) + " vs " + std::to_string(nb));
    float acc = 0.f;
    for (int64_t i = 0; i < na; ++i) acc += a->data[a->offset + i * sa] * b->data[b->offset + i * sb];
    *out = acc;
    return 0;
}

int oracle_sum_over_broadcasted_axes_f32(const float* src, int32_t sr, const int64_t* sshape,
                                         int32_t dr, const int64_t* dshape, float* dst) {
    if (dr > sr) return fail("sum_over_broadcasted_axes: target rank exceeds source rank");
    const int lead = sr - dr;
    for (int d = 0; d < dr; ++d)
        if (dshape[d] != sshape[lead + d] && dshape[d] != 1) return fail("sum_over_broadcasted_axes: shapes not compatible");
    int64_t dstr[ORACLE_MAX_RANK];
    { int64_t acc = 1; for (int d = dr - 1; d >= 0; --d) { dstr[d] = (dshape[d] == 1) ? 0 : acc; acc *= dshape[d]; } }
    const int64_t total = product(sshape, sr);
    std::memset(dst, 0, sizeof(float) * (size_t)std::max<int64_t>(1, product(dshape, dr)));
    // source elements visited in row-major order: each target element receives its addends in
    // ascending order of the reduced coordinates, as successive single-axis reductions would.
    int64_t idx[ORACLE_MAX_RANK + 2] = {0};
    for (int64_t f = 0; f < total; ++f) {
        int64_t off = 0;
        for (int d = 0; d < dr; ++d) off += idx[lead + d] * dstr[d];
        dst[off] += src[f];
        for (int d = sr - 1; d >= 0; --d) { if (++idx[d] < sshape[d]) break; idx[d] = 0; }
    }
    return 0;
}

// ---- MLP-step harness ---------------------------------------------------------------------

struct oracle_mlp {
    int L;
    std::vector<int64_t> dims;
    std::vector<std::vector<float>> W, b, dW, db;
    std::vector<std::vector<float>> z, h, mask; // per layer: pre-activation+bias, activation, relu mask
    std::vector<std::vector<float>> dz, dh;
    std::vector<float> softmax, scratch;
    int64_t max_batch;
};

static oracle_view view2(const float* p, int64_t r, int64_t c, int64_t rs, int64_t cs) {
    oracle_view v{}; v.data = p; v.offset = 0; v.rank = 2; v.shape[0] = r; v.shape[1] = c; v.strides[0] = rs; v.strides[1] = cs; return v;
}

oracle_mlp* oracle_mlp_create(int L, const int64_t* dims, const float* const* W, const float* const* b, int64_t max_batch) {
    auto* m = new oracle_mlp();
    m->L = L; m->dims.assign(dims, dims + L + 1); m->max_batch = max_batch;
    m->W.resize(L); m->b.resize(L); m->dW.resize(L); m->db.resize(L);
    m->z.resize(L); m->h.resize(L); m->mask.resize(L); m->dz.resize(L); m->dh.resize(L);
    int64_t widest = 0;
    for (int l = 0; l < L; ++l) {
        int64_t in = dims[l], out = dims[l + 1];
        m->W[l].assign(W[l], W[l] + in * out);
        m->b[l].assign(b[l], b[l] + out);
        m->dW[l].assign(in * out, 0.f); m->db[l].assign(out, 0.f);
        m->z[l].assign(max_batch * out, 0.f); m->h[l].assign(max_batch * out, 0.f); m->mask[l].assign(max_batch * out, 0.f);
        m->dz[l].assign(max_batch * out, 0.f); m->dh[l].assign(max_batch * std::max(in, out), 0.f);
        widest = std::max(widest, std::max(in, out));
    }
    m->softmax.assign(max_batch * dims[L], 0.f);
    m->scratch.assign(max_batch * widest, 0.f);
    return m;
}
void oracle_mlp_destroy(oracle_mlp* m) { delete m; }

static int mlp_forward(oracle_mlp* m, const float* x, int64_t B, int nthreads) {
    const float* in = x;
    for (int l = 0; l < m->L; ++l) {
        int64_t I = m->dims[l], O = m->dims[l + 1];
        oracle_view a = view2(in, B, I, I, 1), w = view2(m->W[l].data(), I, O, O, 1);
        if (oracle_mm2d_f32(&a, &w, m->z[l].data(), nthreads, nullptr, nullptr)) return -1; // Linear: x.W  (net.mojo:191-197)
        float* z = m->z[l].data();
        for (int64_t r = 0; r < B; ++r) for (int64_t c = 0; c < O; ++c) z[r * O + c] += m->b[l][c]; // + b broadcast (:198-201)
        if (l + 1 < m->L) {                                                                            // ReLU and mask, relu.mojo:120-123
            float* h = m->h[l].data(); float* k = m->mask[l].data();
            for (int64_t e = 0; e < B * O; ++e) { h[e] = z[e] > 0.f ? z[e] : 0.f; k[e] = z[e] > 0.f ? 1.f : 0.f; }
            in = h;
        }
    }
    return 0;
}

int oracle_mlp_forward(oracle_mlp* m, const float* x, int64_t B, float* logits, int nthreads) {
    if (B > m->max_batch) return fail("batch exceeds max_batch");
    if (mlp_forward(m, x, B, nthreads)) return -1;
    std::memcpy(logits, m->z[m->L - 1].data(), sizeof(float) * (size_t)(B * m->dims[m->L]));
    return 0;
}

float oracle_mlp_step(oracle_mlp* m, const float* x, const int32_t* y, int64_t B, float lr, int nthreads) {
    if (B > m->max_batch) { fail("batch exceeds max_batch"); return NAN; }
    if (mlp_forward(m, x, B, nthreads)) return NAN;
    const int L = m->L;
    const int64_t C = m->dims[L];
    const float* logits = m->z[L - 1].data();
    float* sm = m->softmax.data();
    // fused cross-entropy forward, mean reduction (crossentropy.mojo:327-427)
    float loss_sum = 0.f;
    for (int64_t r = 0; r < B; ++r) {
        const float* row = logits + r * C;
        float mx = -std::numeric_limits<float>::max();
        for (int64_t c = 0; c < C; ++c) mx = std::max(mx, row[c]);
        float sum_exp = 0.f;
        for (int64_t c = 0; c < C; ++c) { float e = std::exp(row[c] - mx); sum_exp += e; sm[r * C + c] = e; }
        float lse = std::log(std::max(sum_exp, 1e-7f)); // Epsilon[float32], common_utils.mojo:220-221
        loss_sum += -(row[y[r]] - mx - lse);
        float inv = 1.f / sum_exp;
        for (int64_t c = 0; c < C; ++c) sm[r * C + c] *= inv;
    }
    float loss = loss_sum / (float)B;
    // backward seed: (softmax - onehot) * (upstream 1 / valid_count)   (:775-793, :451-481)
    float* dz = m->dz[L - 1].data();
    const float scale = 1.0f / (float)B;
    for (int64_t r = 0; r < B; ++r)
        for (int64_t c = 0; c < C; ++c) dz[r * C + c] = (sm[r * C + c] - (c == y[r] ? 1.f : 0.f)) * scale;
    for (int l = L - 1; l >= 0; --l) {
        int64_t I = m->dims[l], O = m->dims[l + 1];
        const float* in = (l == 0) ? x : m->h[l - 1].data();
        float* g = m->dz[l].data();
        // bias gradient = column sums of the incoming gradient (broadcast.mojo:81-87), rows ascending
        for (int64_t c = 0; c < O; ++c) m->db[l][c] = 0.f;
        for (int64_t r = 0; r < B; ++r) for (int64_t c = 0; c < O; ++c) m->db[l][c] += g[r * O + c];
        // dW = x^T(view) . g  -> path 1b ; dX = g . W^T(view) -> path 2   (matmul.mojo:33-52)
        oracle_view xt = view2(in, I, B, 1, I), gv = view2(g, B, O, O, 1);
        if (oracle_mm2d_f32(&xt, &gv, m->dW[l].data(), nthreads, nullptr, nullptr)) return NAN;
        if (l > 0) { // the network input does not require grad (matmul.mojo:34)
            oracle_view wt = view2(m->W[l].data(), O, I, 1, O);
            if (oracle_mm2d_f32(&gv, &wt, m->dh[l].data(), nthreads, nullptr, nullptr)) return NAN;
            float* gprev = m->dz[l - 1].data(); const float* dh = m->dh[l].data(); const float* k = m->mask[l - 1].data();
            for (int64_t e = 0; e < B * I; ++e) gprev[e] = dh[e] * k[e]; // ReLU backward, relu.mojo:21-46
        }
    }
    for (int l = 0; l < L; ++l) { // SGD, optim.mojo:93-120 with weight_decay 0
        for (size_t e = 0; e < m->W[l].size(); ++e) m->W[l][e] -= lr * m->dW[l][e];
        for (size_t e = 0; e < m->b[l].size(); ++e) m->b[l][e] -= lr * m->db[l][e];
    }
    return loss;
}

int oracle_mlp_get_params(oracle_mlp* m, int l, float* W, float* b) {
    if (l < 0 || l >= m->L) return fail("layer out of range");
    if (W) std::copy(m->W[l].begin(), m->W[l].end(), W);
    if (b) std::copy(m->b[l].begin(), m->b[l].end(), b);
    return 0;
}
int oracle_mlp_get_grads(oracle_mlp* m, int l, float* dW, float* db) {
    if (l < 0 || l >= m->L) return fail("layer out of range");
    if (dW) std::copy(m->dW[l].begin(), m->dW[l].end(), dW);
    if (db) std::copy(m->db[l].begin(), m->db[l].end(), db);
    return 0;
}

// ---- class-index cross-entropy (tenmo/crossentropy.mojo:285-432) --------------------------------
// Row loop with the reference's three passes: max, exp + sum_exp (+ sum of logits under label
// smoothing), loss from the target's logit, then the softmax normalisation.  The row losses are
// added in row order (scalar_loss += loss, :394); valid rows are those whose target differs from
// ignore_index (:369-389).
int oracle_cross_entropy_forward_f32(const float* logits, const int64_t* target, int64_t M, int64_t C, int64_t ignore_index,
                                     float label_smoothing, float* softmax, float* per_sample_loss, float* loss_sum, int32_t* valid_count) {
    if (M < 0 || C < 1) return fail("cross entropy needs M >= 0 and C >= 1");
    if (!(label_smoothing >= 0.f && label_smoothing <= 1.f)) return fail("CrossEntropyLoss: label_smoothing must be in [0, 1]");
    const bool has_ls = label_smoothing > 0.f;
    float scalar_loss = 0.f;
    int32_t valid = 0;
    for (int64_t row = 0; row < M; ++row) {
        const float* x = logits + row * C;
        float max_val = -std::numeric_limits<float>::max();          // min_finite, :332
        for (int64_t c = 0; c < C; ++c) max_val = std::max(max_val, x[c]);
        float sum_exp = 0.f, sum_logits = 0.f;
        for (int64_t c = 0; c < C; ++c) {
            const float e = std::exp(x[c] - max_val);
            sum_exp += e;
            if (has_ls) sum_logits += x[c];
            if (softmax) softmax[row * C + c] = e;
        }
        const float log_sum_exp = std::log(std::max(sum_exp, 1e-7f)); // Epsilon[float32], :366-367
        float loss = 0.f;
        if (target[row] != ignore_index) {
            const int64_t t = target[row];
            if (t < 0 || t >= C) return fail("cross entropy: target index outside [0, C)"); // validated at :116-123
            const float log_softmax_tgt = x[t] - max_val - log_sum_exp;
            loss = -log_softmax_tgt;
            if (has_ls) {
                const float inv_C = 1.f / (float)C;
                const float mean_log_softmax = sum_logits * inv_C - max_val - log_sum_exp;
                loss = (1.f - label_smoothing) * loss - label_smoothing * mean_log_softmax;
            }
            ++valid;
        }
        if (per_sample_loss) per_sample_loss[row] = loss;
        scalar_loss += loss;
        if (softmax) {
            const float inv = 1.f / sum_exp;
            for (int64_t c = 0; c < C; ++c) softmax[row * C + c] *= inv;
        }
    }
    if (loss_sum) *loss_sum = scalar_loss;
    if (valid_count) *valid_count = valid;
    return 0;
}

// Gradient with respect to the logits (tenmo/crossentropy.mojo:744-770 with scale_grad_by_upstream
// :451-481): (softmax - (1-ls)*onehot - ls/C) * ignore_mask * upstream / (valid_count for mean).
// reduction: 0 none (upstream has M entries), 1 sum, 2 mean.
int oracle_cross_entropy_backward_f32(const float* softmax, const int64_t* target, const float* upstream, int64_t M, int64_t C,
                                      int64_t ignore_index, float label_smoothing, int reduction, int32_t valid_count, float* grad) {
    if (reduction < 0 || reduction > 2) return fail("reduction must be 0, 1 or 2");
    const float ls = label_smoothing;
    const float ls_uniform = ls / (float)C;
    for (int64_t row = 0; row < M; ++row) {
        const bool valid = target[row] != ignore_index;
        float scale;
        if (reduction == 0) scale = upstream[row];
        else scale = upstream[0] / (float)((reduction == 2 && valid_count > 0) ? valid_count : 1);
        for (int64_t c = 0; c < C; ++c) {
            const float onehot = (valid && c == target[row]) ? 1.f : 0.f;
            float g = softmax[row * C + c];
            if (ls > 0.f) g = (g - onehot * (1.f - ls)) - ls_uniform;
            else g = g - onehot;
            g = g * (valid ? 1.f : 0.f);
            grad[row * C + c] = g * scale;
        }
    }
    return 0;
}

// One SGD step on one tensor (tenmo/optim.mojo:93-160): g += weight_decay * p when weight_decay > 0;
// with a velocity buffer v = momentum * v + g and p -= lr * v, otherwise p -= lr * g.
int oracle_sgd_step_f32(float* param, const float* grad, float* velocity, int64_t n, float lr, float momentum, float weight_decay) {
    for (int64_t i = 0; i < n; ++i) {
        const float p = param[i];
        float g = grad[i];
        if (weight_decay > 0.f) g += p * weight_decay;
        if (velocity) {
            const float v = momentum * velocity[i] + g;
            velocity[i] = v;
            param[i] = p - lr * v;
        } else {
            param[i] = p - lr * g;
        }
    }
    return 0;
}

// Fused im2col + convolution + bias, FusedIm2Col.forward (tenmo/cnn.mojo:308-507), on an image that is
// already padded (Conv2dFused.invoke pads first, :118-125, :229-235).  Per output position the sum starts
// from the bias (:432, :479) and adds img * kernel over ci, then ky, then kx ascending (:435-470,
// :481-498) in fp32; the reference's SIMD lanes run over output channels, which does not change the
// order inside one output element.  Output sizes as in :358-365.
int oracle_conv2d_forward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                              const float* kernel, int64_t c_out, int64_t kh, int64_t kw, const float* bias,
                              int64_t stride, int64_t dilation, float* out) {
    if (c_in < 1 || c_out < 1 || kh < 1 || kw < 1 || stride < 1 || dilation < 1) return fail("conv2d: sizes, stride and dilation must be positive");
    const int64_t dkh = kh + (kh - 1) * (dilation - 1), dkw = kw + (kw - 1) * (dilation - 1);
    const int64_t h_out = (h_pad - dkh) / stride + 1, w_out = (w_pad - dkw) / stride + 1;
    if (h_pad < dkh || w_pad < dkw || h_out <= 0 || w_out <= 0) return fail("conv2d: Invalid output dimensions");
    for (int64_t n = 0; n < n_images; ++n)
        for (int64_t y = 0; y < h_out; ++y)
            for (int64_t x = 0; x < w_out; ++x)
                for (int64_t co = 0; co < c_out; ++co) {
                    float accum = bias ? bias[co] : 0.f;
                    for (int64_t ci = 0; ci < c_in; ++ci)
                        for (int64_t ky = 0; ky < kh; ++ky)
                            for (int64_t kx = 0; kx < kw; ++kx) {
                                const float img = padded_image[((n * c_in + ci) * h_pad + y * stride + ky * dilation) * w_pad + x * stride + kx * dilation];
                                const float kv = kernel[((co * c_in + ci) * kh + ky) * kw + kx];
                                accum += img * kv;
                            }
                    out[((n * c_out + co) * h_out + y) * w_out + x] = accum;
                }
    return 0;
}

// The three gradients of the fused convolution, FusedCol2ImBackward (tenmo/cnn.mojo:546-948), for the upstream
// gradient grad_out [N, C_out, H_out, W_out]; a null output is skipped.  Bias: the sum over (n, y, x) per channel
// (:669-713).  Kernel: grad_out viewed [C_out, N*H_out*W_out] times the patch matrix (:716-815; the reference
// builds the patches and calls Tensor.matmul — here the same sums in the order n, y, x).  Padded image: the
// scatter loop of :818-948 in its order (n, y, x, co, ci, ky, kx), with its skip of zero upstream values.
int oracle_conv2d_backward_f32(const float* padded_image, int64_t n_images, int64_t c_in, int64_t h_pad, int64_t w_pad,
                               const float* kernel, int64_t c_out, int64_t kh, int64_t kw, int64_t stride, int64_t dilation,
                               const float* grad_out, float* grad_padded_image, float* grad_kernel, float* grad_bias) {
    if (c_in < 1 || c_out < 1 || kh < 1 || kw < 1 || stride < 1 || dilation < 1) return fail("conv2d backward: sizes, stride and dilation must be positive");
    const int64_t dkh = kh + (kh - 1) * (dilation - 1), dkw = kw + (kw - 1) * (dilation - 1);
    if (h_pad < dkh || w_pad < dkw) return fail("conv2d backward: Invalid output dimensions");
    const int64_t h_out = (h_pad - dkh) / stride + 1, w_out = (w_pad - dkw) / stride + 1;
    auto go = [&](int64_t n, int64_t co, int64_t y, int64_t x) { return grad_out[((n * c_out + co) * h_out + y) * w_out + x]; };
    if (grad_bias)
        for (int64_t co = 0; co < c_out; ++co) {
            float acc = 0.f;
            for (int64_t n = 0; n < n_images; ++n)
                for (int64_t y = 0; y < h_out; ++y)
                    for (int64_t x = 0; x < w_out; ++x) acc += go(n, co, y, x);
            grad_bias[co] = acc;
        }
    if (grad_kernel)
        for (int64_t co = 0; co < c_out; ++co)
            for (int64_t ci = 0; ci < c_in; ++ci)
                for (int64_t ky = 0; ky < kh; ++ky)
                    for (int64_t kx = 0; kx < kw; ++kx) {
                        float acc = 0.f;
                        for (int64_t n = 0; n < n_images; ++n)
                            for (int64_t y = 0; y < h_out; ++y)
                                for (int64_t x = 0; x < w_out; ++x)
                                    acc += go(n, co, y, x) * padded_image[((n * c_in + ci) * h_pad + y * stride + ky * dilation) * w_pad + x * stride + kx * dilation];
                        grad_kernel[((co * c_in + ci) * kh + ky) * kw + kx] = acc;
                    }
    if (grad_padded_image) {
        for (int64_t i = 0; i < n_images * c_in * h_pad * w_pad; ++i) grad_padded_image[i] = 0.f;
        for (int64_t n = 0; n < n_images; ++n)
            for (int64_t y = 0; y < h_out; ++y)
                for (int64_t x = 0; x < w_out; ++x)
                    for (int64_t co = 0; co < c_out; ++co) {
                        const float g = go(n, co, y, x);
                        if (g == 0.f) continue;
                        for (int64_t ci = 0; ci < c_in; ++ci)
                            for (int64_t ky = 0; ky < kh; ++ky)
                                for (int64_t kx = 0; kx < kw; ++kx)
                                    grad_padded_image[((n * c_in + ci) * h_pad + y * stride + ky * dilation) * w_pad + x * stride + kx * dilation] +=
                                        g * kernel[((co * c_in + ci) * kh + ky) * kw + kx];
                    }
    }
    return 0;
}

} // extern "C"
