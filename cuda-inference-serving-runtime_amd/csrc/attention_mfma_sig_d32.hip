// Paged matrix-core attention with sigmoid weights that are not normed over the keys, head sizes up to 32
// (see attention_mfma.inc).
#define DPAD 32
#define ATTN_SIGMOID 1
#include "attention_mfma.inc"
