/* functions/cnn_gradient.h of the reference: computeCNNGradient (functions/cnn_gradient.h:9-12) */
#include "fitre_cnn.h"
