/* augmentation/dev_normalize.h of the reference: normalizeCIFAR10 (augmentation/dev_normalize.h) */
#include "fitre_input.h"
