/* solvers/kfac_trust_region.h of the reference: subsampledTrustRegionKFAC (solvers/kfac_trust_region.h) */
#include "fitre_solver.h"
