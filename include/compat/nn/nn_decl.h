/* nn/nn_decl.h of the reference: CNN_MODEL, CONV_LAYER, POOL_LAYER, FC_LAYER, NN_MODEL (nn/nn_decl.h:64-155) */
#include "fitre_nn.h"
