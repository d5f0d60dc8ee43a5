#ifndef ACL_MI355_CORE_COORDINATES_H
#define ACL_MI355_CORE_COORDINATES_H
#include "arm_compute/core/Dimensions.h"
#endif
