/* functions/eval_hessian_vec.h of the reference: hessianVec (functions/eval_hessian_vec.h:9) */
#include "fitre_fc.h"
