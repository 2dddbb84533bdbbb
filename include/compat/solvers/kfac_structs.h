/* solvers/kfac_structs.h of the reference: KFAC_CURVATURE_INFO (solvers/kfac_structs.h:13-52) */
#include "fitre_kfac.h"
