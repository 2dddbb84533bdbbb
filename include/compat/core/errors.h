/* core/errors.h of the reference: the ERROR_* exit codes (core/errors.h) */
#include "fitre_types.h"
