/* augmentation/dev_crop.h of the reference: randomCrop (augmentation/dev_crop.h) */
#include "fitre_input.h"
