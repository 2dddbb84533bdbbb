/* functions/cnn_backward.h of the reference: cnnBackward, cnnBackwardMemRequired (functions/cnn_backward.h:11-16) */
#include "fitre_cnn.h"
