// Forwarding header: the reference spreads its runtime interface over runtime/include/brt/backends/cuda/device/common/util.h and
// its neighbours; here one header (brt.h) holds it, and this path exists so that an op-kernel
// source written against the reference's include lines compiles unchanged.
#ifndef BRT_BACKENDS_CUDA_DEVICE_COMMON_UTIL_H_
#define BRT_BACKENDS_CUDA_DEVICE_COMMON_UTIL_H_
#include "../../../../../brt.h"
#endif
