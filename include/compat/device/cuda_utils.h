/* device/cuda_utils.h of the reference: cuda_malloc, copy_host_device, ... and the cublasCheckError family (device/cuda_utils.h:15-31) */
#include "fitre_shim.h"
#include "fitre_blas_compat.h"
