/* functions/cnn_eval_model.h of the reference: evaluateCNNModel (functions/cnn_eval_model.h) */
#include "fitre_cnn.h"
