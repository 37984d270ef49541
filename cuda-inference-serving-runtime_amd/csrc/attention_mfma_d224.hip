// Paged matrix-core attention for head sizes up to 224 (see attention_mfma.inc).
#define DPAD 224
#include "attention_mfma.inc"
