/* device/gen_random.h of the reference: getRandomVector (device/gen_random.h:6-13) */
#include "fitre_shim.h"
#include "fitre_solver.h"
