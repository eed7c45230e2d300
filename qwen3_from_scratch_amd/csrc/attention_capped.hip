// The paged attention kernels of attention.hip once more, with scores that are bent before the
// softmax: cap * tanh(score * scale / cap). The source is the same; the score's way into the
// exponent is the one thing that differs (see `ScoreScale` there), and the cap is set by
// q3_set_score_cap before a launch. Only the matrix-core kernels are built here.
#define Q3_SCORE_CAP 1
#include "attention.hip"
