/* augmentation/dev_flip.h of the reference: flipData (augmentation/dev_flip.h) */
#include "fitre_input.h"
