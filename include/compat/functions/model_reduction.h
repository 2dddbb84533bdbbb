/* functions/model_reduction.h of the reference: computeQuadraticModel (functions/model_reduction.h:9-12) */
#include "fitre_hv.h"
