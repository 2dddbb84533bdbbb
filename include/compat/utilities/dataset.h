/* utilities/dataset.h of the reference: the data-set readers (utilities/dataset.h) */
#include "fitre_dataset.h"
