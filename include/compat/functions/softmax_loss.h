/* functions/softmax_loss.h of the reference: computeCrossEntropyError, computeDistributionErrors (functions/softmax_loss.h) */
#include "fitre_cnn.h"
