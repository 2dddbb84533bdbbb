/* solvers/kfac_utils.h of the reference: computeKFACStorageIndices (solvers/kfac_utils.h) */
#include "fitre_kfac.h"
