/* core/datadefs.h of the reference: real and its constants (core/datadefs.h:1-12) */
#include "fitre_types.h"
