/* nn/read_vgg.h of the reference: readVGG11 / 13 / 16 / 19, makeLayer (nn/read_vgg.h) */
#include "fitre_cnn.h"
