// Skinny bf16 matrix products for at most 48 rows (see gemm_skinny.inc).
#define SKINNY_MT 3
#include "gemm_skinny.inc"
