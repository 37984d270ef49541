// Paged matrix-core attention for head sizes up to 160 (see attention_mfma.inc).
#define DPAD 160
#include "attention_mfma.inc"
