// Paged matrix-core attention with sigmoid weights that are not normed over the keys, head sizes up to 192
// (see attention_mfma.inc).
#define DPAD 192
#define ATTN_SIGMOID 1
#include "attention_mfma.inc"
