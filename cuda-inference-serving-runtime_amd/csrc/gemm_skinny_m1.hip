// Skinny bf16 matrix products for at most 16 rows (see gemm_skinny.inc).
#define SKINNY_MT 1
#include "gemm_skinny.inc"
