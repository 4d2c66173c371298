#pragma once
// Host/device decoration used by the llis headers.  The reference spells it CUDA_HOSTDEV
// (reference include/llis/utils/gpu.h:4-8); job sources written against it keep compiling.

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define LLIS_HOSTDEV __host__ __device__
#define LLIS_DEVICE __device__
#else
#define LLIS_HOSTDEV
#define LLIS_DEVICE
#endif

#ifndef CUDA_HOSTDEV
#define CUDA_HOSTDEV LLIS_HOSTDEV
#endif
