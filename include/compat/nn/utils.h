/* nn/utils.h of the reference: computeParamSize, the offset builders, getDimensions (nn/utils.h) */
#include "fitre_cnn.h"
