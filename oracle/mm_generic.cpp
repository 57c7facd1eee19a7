// CPU oracle (test infrastructure): the shared matmul kernels compiled for one ISA level.
#define ORACLE_NS isa_generic
#define ORACLE_W 1
#include "mm_kernels.inc"
