/* solvers/kfac_natural_gradient.h of the reference: computeNaturalGradient (solvers/kfac_natural_gradient.h) */
#include "fitre_kfac.h"
