// dummy_short: 10 back-to-back kernels of 5 x 256 (see dummy_common.h).
#define DUMMY_NUM_KERNELS 10
#include "dummy_common.h"
