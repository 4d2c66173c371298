// dummy_20: 20 back-to-back kernels of 5 x 256 (see dummy_common.h).
#define DUMMY_NUM_KERNELS 20
#include "dummy_common.h"
