// The narrow products with 1 tile(s) of four activation rows (gemm_narrow.inc).
#define NARROW_TILES 1
#include "gemm_narrow.inc"
