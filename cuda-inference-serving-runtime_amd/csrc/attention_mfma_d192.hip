// Paged matrix-core attention for head sizes up to 192 (see attention_mfma.inc).
#define DPAD 192
#include "attention_mfma.inc"
