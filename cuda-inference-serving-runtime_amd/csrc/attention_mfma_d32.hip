// Paged matrix-core attention for head sizes up to 32 (see attention_mfma.inc).
#define DPAD 32
#include "attention_mfma.inc"
