// Paged matrix-core attention for head sizes up to 96 (see attention_mfma.inc).
#define DPAD 96
#include "attention_mfma.inc"
