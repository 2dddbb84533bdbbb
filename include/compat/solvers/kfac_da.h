/* solvers/kfac_da.h of the reference: augmentData (solvers/kfac_da.h) */
#include "fitre_input.h"
