// CPU oracle (test infrastructure): the shared matmul kernels compiled for one ISA level.
#define ORACLE_NS isa_avx512
#define ORACLE_W 16
#include "mm_kernels.inc"
