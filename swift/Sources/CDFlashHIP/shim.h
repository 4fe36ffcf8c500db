/* Umbrella header of the CDFlashHIP Clang module: the library's C ABI plus the handful of HIP
 * runtime calls the Swift shim uses to own device memory. */
#ifndef CDFLASHHIP_SHIM_H
#define CDFLASHHIP_SHIM_H

#include "../../../include/dflash_hip.h"
#include "../../../include/dflash_cache.h"
#include "hip_min.h"

#endif
