#ifndef ACL_MI355_RUNTIME_IWEIGHTSMANAGER_H
#define ACL_MI355_RUNTIME_IWEIGHTSMANAGER_H
#include "arm_compute/runtime/IMemoryManager.h"
#endif
