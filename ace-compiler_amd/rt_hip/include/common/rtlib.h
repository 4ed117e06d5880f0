/* Hand-written mains include "common/rtlib.h" (rtlib/include/common/rtlib.h in
 * the reference); same runtime. */
#ifndef RT_HIP_RTLIB_SHIM_H
#define RT_HIP_RTLIB_SHIM_H
#include "rt_hip.h"
#endif
