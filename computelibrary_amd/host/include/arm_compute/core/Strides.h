#ifndef ACL_MI355_CORE_STRIDES_H
#define ACL_MI355_CORE_STRIDES_H
#include "arm_compute/core/Dimensions.h"
#endif
