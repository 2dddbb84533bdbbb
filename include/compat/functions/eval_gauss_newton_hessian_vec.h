/* functions/eval_gauss_newton_hessian_vec.h of the reference: gaussNewtonHessianVec (functions/eval_gauss_newton_hessian_vec.h:9) */
#include "fitre_fc.h"
