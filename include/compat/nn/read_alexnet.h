/* nn/read_alexnet.h of the reference: readAlexNetCNN (nn/read_alexnet.h) */
#include "fitre_cnn.h"
