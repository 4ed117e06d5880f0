/* Programs emitted for the ANT runtime start with `#include "rt_ant/rt_ant.h"`
 * (rtlib/include/rt_ant/rt_ant.h:9-28 in the reference); with this directory on
 * the include path that line resolves to the HIP-backed runtime. */
#ifndef RT_HIP_RT_ANT_SHIM_H
#define RT_HIP_RT_ANT_SHIM_H
#include "rt_hip.h"
#endif
