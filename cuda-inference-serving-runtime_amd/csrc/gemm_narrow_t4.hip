// The narrow products with 4 tile(s) of four activation rows (gemm_narrow.inc).
#define NARROW_TILES 4
#include "gemm_narrow.inc"
