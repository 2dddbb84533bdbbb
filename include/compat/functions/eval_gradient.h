/* functions/eval_gradient.h of the reference: computeGradient, evaluateModel, nnForwardPass, applyLayerActivation (functions/eval_gradient.h:9-25) */
#include "fitre_fc.h"
