/* device/handles.h of the reference: the vendor-library handles (device/handles.h:13-18), opaque here, and the BLAS names */
#include "fitre_blas_compat.h"
