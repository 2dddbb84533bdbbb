/* functions/cnn_forward.h of the reference: cnnForward, cnnForwardMemRequired (functions/cnn_forward.h:9-13) */
#include "fitre_cnn.h"
