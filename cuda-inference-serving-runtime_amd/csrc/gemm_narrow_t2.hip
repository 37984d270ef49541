// The narrow products with 2 tile(s) of four activation rows (gemm_narrow.inc).
#define NARROW_TILES 2
#include "gemm_narrow.inc"
