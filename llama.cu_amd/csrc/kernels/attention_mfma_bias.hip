// The matrix-core attention kernels of attention_mfma.hip once more, with a bias inside the scores
// that grows with the distance between key and query: slope[h] * (j - p) is added to the scaled
// score of key j for the query at position p of head h.  Every entry point takes, as its last
// argument, head_slopes [heads] (32-bit, on the device); the scale must be positive.  A library
// of its own, so that the kernels without a bias carry nothing for it.
#define LCU_SCORE_BIAS 1
#include "attention_mfma.hip"
