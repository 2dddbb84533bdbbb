/* device/cuda_environment.h of the reference: cuda_env_init, cuda_allocate_workspace, cuda_env_cleanup (device/cuda_environment.h:6-9) */
#include "fitre_shim.h"
