/* utilities/print_utils.h of the reference: readVector, writeVector (utilities/print_utils.h) */
#include "fitre_shim.h"
