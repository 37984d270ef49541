// Skinny bf16 matrix products for at most 32 rows (see gemm_skinny.inc).
#define SKINNY_MT 2
#include "gemm_skinny.inc"
