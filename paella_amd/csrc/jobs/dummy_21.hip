// dummy_21: 21 back-to-back kernels of 5 x 256 (see dummy_common.h).
#define DUMMY_NUM_KERNELS 21
#include "dummy_common.h"
