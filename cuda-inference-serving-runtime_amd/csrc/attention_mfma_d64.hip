// Paged matrix-core attention for head sizes up to 64 (see attention_mfma.inc).
#define DPAD 64
#include "attention_mfma.inc"
