/* device/device_defines.h of the reference: BLOCK_SIZE, WARP_SIZE, DEVICE_NUM_BLOCKS, __THREADS_PER_SAMPLE__ (device/device_defines.h:4-15) */
#include "fitre_shim.h"
