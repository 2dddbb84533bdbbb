/* solvers/kfac_inverses.h of the reference: computeOmegaZ, computeLambdaDelta (solvers/kfac_inverses.h:28-34) */
#include "fitre_kfac.h"
