/* core/structdefs.h of the reference: SCRATCH_AREA, DEVICE_DATASET and friends (core/structdefs.h:25-83) */
#include "fitre_types.h"
