// Paged matrix-core attention for head sizes up to 128 (see attention_mfma.inc).
#define DPAD 128
#include "attention_mfma.inc"
