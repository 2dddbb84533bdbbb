/* functions/cnn_hessian_vec.h of the reference: cnnHv (functions/cnn_hessian_vec.h:9-13) */
#include "fitre_hv.h"
