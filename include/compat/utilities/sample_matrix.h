/* utilities/sample_matrix.h of the reference: selectColumnMatrix (utilities/sample_matrix.h) */
#include "fitre_input.h"
