// CPU oracle (test infrastructure): arguments shared by the per-ISA matmul kernels.
#pragma once
#include <cstdint>

struct MmArgs {
    const float* A;
    const float* B;
    float* C;
    int64_t a_rs, a_cs, b_rs, b_cs; // row / column strides of the two trailing dims, in elements
    int64_t n, p;                   // inner dim, result columns
    int path;                       // 0 = 1a, 1 = 1b, 2 = scalar path 2
    int tile_j_in_path2;            // 1 for the 2-D kernel, 0 for the batched one
};

using row_tile_fn = void (*)(const MmArgs&, int64_t A_base, int64_t B_base, int64_t C_base, int64_t i_start, int64_t i_end);

#define ORACLE_DECLARE_ISA(NS)                                                                         \
    namespace NS {                                                                                     \
    row_tile_fn select(int tm, int tn, int tp);                                                        \
    int lanes();                                                                                       \
    void vm_contig(const float* v, int64_t v_base, int64_t v_stride, const float* M, int64_t M_base,   \
                   int64_t m_rs, int64_t k, int64_t n, float* out);                                    \
    void axpy_row(float s, const float* src, int64_t src_stride, float* dst, int64_t len);             \
    }
ORACLE_DECLARE_ISA(isa_avx512)
ORACLE_DECLARE_ISA(isa_avx2)
ORACLE_DECLARE_ISA(isa_generic)
