// CPU oracle (test infrastructure): the shared matmul kernels compiled for one ISA level.
#define ORACLE_NS isa_avx2
#define ORACLE_W 8
#include "mm_kernels.inc"
