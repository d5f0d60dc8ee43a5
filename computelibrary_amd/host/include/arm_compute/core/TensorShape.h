#ifndef ACL_MI355_CORE_TENSORSHAPE_H
#define ACL_MI355_CORE_TENSORSHAPE_H
#include "arm_compute/core/Dimensions.h"
#endif
