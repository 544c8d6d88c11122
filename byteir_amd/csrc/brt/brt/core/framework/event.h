// Forwarding header: the reference spreads its runtime interface over runtime/include/brt/core/framework/event.h and
// its neighbours; here one header (brt.h) holds it, and this path exists so that an op-kernel
// source written against the reference's include lines compiles unchanged.
#ifndef BRT_CORE_FRAMEWORK_EVENT_H_
#define BRT_CORE_FRAMEWORK_EVENT_H_
#include "../../../brt.h"
#endif
