// Skinny bf16 matrix products for at most 64 rows (see gemm_skinny.inc).
#define SKINNY_MT 4
#include "gemm_skinny.inc"
