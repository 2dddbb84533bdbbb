/* nn/read_nn.h of the reference: readLenetCNN (nn/read_nn.h) */
#include "fitre_cnn.h"
