/* functions/cnn_accuracy.h of the reference: computeAccuracy and the generalization-error sweeps (functions/cnn_accuracy.h) */
#include "fitre_cnn.h"
#include "fitre_input.h"
