/* The sampling hook every backend reads (include/model.h:105-111 of the reference).  The
 * reference defines it in its CLI (src/run.c:83); run-hip and the test library take it from here. */
#include "model.h"
int (*model_pick)(const float *logits, int n) = NULL;
