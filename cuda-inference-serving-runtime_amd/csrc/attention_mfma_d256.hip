// Paged matrix-core attention for head sizes up to 256 (see attention_mfma.inc).
#define DPAD 256
#include "attention_mfma.inc"
